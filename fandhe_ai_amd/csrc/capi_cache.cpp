// C entry points of the paged-KV cache row: the host block table by itself (usable without a device)
// and the one-layer device-resident cache that appends through fa_paged_kv_append and attends through
// fa_paged_attention_forward.
#include <algorithm>
#include <exception>
#include <new>
#include <string>
#include <vector>

#include "../../include/fandhe_rocm.h"
#include "block_table.hpp"
#include "runtime.hpp"
#include "validate.hpp"

using namespace fa;

struct fa_block_table {
    uint32_t magic;
    BlockTable t;
};

struct fa_paged_cache {
    uint32_t magic;
    fa_context *ctx;
    uint64_t block_size, max_blocks, embed_dim;
    fa_dtype dtype;
    fa_paged_layout layout;
    fa_buffer *k_pool, *v_pool;
    BlockTable table;
    bool poisoned;
};

namespace {
constexpr uint32_t kTableMagic = 0xFA0B7AB1u, kCacheMagic = 0xFA0CAC4Eu;

fa_status check_table(const fa_block_table *bt) {
    if (!bt || bt->magic != kTableMagic) return fail(FA_ERR_INVALID_ARGUMENT, "not a block table handle");
    return FA_OK;
}
fa_status check_cache(const fa_paged_cache *c) {
    if (!c || c->magic != kCacheMagic) return fail(FA_ERR_INVALID_ARGUMENT, "not a paged cache handle");
    return FA_OK;
}
fa_status table_result(const std::string &err, const char *op) {
    if (err.empty()) return FA_OK;
    return fail(FA_ERR_INVALID_ARGUMENT, std::string(op) + ": " + err);
}
void fill_state(const BlockTable &t, uint64_t max_blocks, fa_block_table_state *out) {
    out->seq_len = t.seq_len();
    out->has_batch = t.has_batch ? 1 : 0;
    out->batch = t.batch;
    out->used_blocks = t.used_blocks();
    out->free_blocks = t.free_blocks(max_blocks);
    out->next_unused = t.next_unused;
    out->returned = t.returned.size();
}
}  // namespace

extern "C" {

fa_status fa_block_table_create(fa_block_table **out) {
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "block_table_create: null out");
    fa_block_table *bt = new (std::nothrow) fa_block_table();
    if (!bt) return fail(FA_ERR_ALLOCATION_FAILED, "block_table_create: out of host memory");
    bt->magic = kTableMagic;
    *out = bt;
    return FA_OK;
}

fa_status fa_block_table_destroy(fa_block_table *bt) {
    if (fa_status s = check_table(bt)) return s;
    bt->magic = 0;
    delete bt;
    return FA_OK;
}

fa_status fa_block_table_clone(const fa_block_table *bt, fa_block_table **out) {
    if (fa_status s = check_table(bt)) return s;
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "block_table_clone: null out");
    try {
        fa_block_table *c = new fa_block_table(*bt);
        *out = c;
    } catch (const std::exception &) {
        return fail(FA_ERR_ALLOCATION_FAILED, "block_table_clone: out of host memory");
    }
    return FA_OK;
}

fa_status fa_block_table_alloc(fa_block_table *bt, uint64_t max_blocks, uint32_t *id, int32_t *got) {
    if (fa_status s = check_table(bt)) return s;
    if (!id || !got) return fail(FA_ERR_INVALID_ARGUMENT, "block_table_alloc: null out");
    *got = bt->t.alloc((size_t)max_blocks, id) ? 1 : 0;
    return FA_OK;
}

fa_status fa_block_table_return(fa_block_table *bt, uint32_t id) {
    if (fa_status s = check_table(bt)) return s;
    try {
        bt->t.returned.push_back(id);
    } catch (const std::exception &) {
        return fail(FA_ERR_ALLOCATION_FAILED, "block_table_return: out of host memory");
    }
    return FA_OK;
}

fa_status fa_block_table_reset(fa_block_table *bt) {
    if (fa_status s = check_table(bt)) return s;
    bt->t.reset();
    return FA_OK;
}

fa_status fa_block_table_state_get(const fa_block_table *bt, uint64_t max_blocks, fa_block_table_state *out) {
    if (fa_status s = check_table(bt)) return s;
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "block_table_state: null out");
    fill_state(bt->t, max_blocks, out);
    return FA_OK;
}

fa_status fa_block_table_extend_for_append(fa_block_table *bt, uint64_t max_blocks, uint64_t block_size, uint64_t b,
                                           uint64_t l_new, uint32_t *slots, uint64_t slots_capacity, uint64_t *n_slots) {
    if (fa_status s = check_table(bt)) return s;
    if (!n_slots) return fail(FA_ERR_INVALID_ARGUMENT, "extend_for_append: null n_slots");
    if (block_size == 0) return fail(FA_ERR_INVALID_ARGUMENT, "extend_for_append: block_size 0");
    // the table changes only if everything succeeds, including the caller's buffer being large enough
    BlockTable next;
    std::vector<uint32_t> out;
    try {
        next = bt->t;
    } catch (const std::exception &) {
        return fail(FA_ERR_ALLOCATION_FAILED, "extend_for_append: out of host memory");
    }
    if (fa_status s = table_result(next.extend_for_append((size_t)max_blocks, (size_t)block_size, (size_t)b, (size_t)l_new, &out),
                                   "extend_for_append"))
        return s;
    if (out.size() > slots_capacity || (!out.empty() && !slots))
        return fail(FA_ERR_INVALID_ARGUMENT, "extend_for_append: slot buffer too small");
    for (size_t i = 0; i < out.size(); ++i) slots[i] = out[i];
    *n_slots = out.size();
    bt->t = std::move(next);
    return FA_OK;
}

fa_status fa_block_table_flatten(const fa_block_table *bt, uint64_t max_blocks_per_seq, uint32_t *out, uint64_t out_capacity,
                                 uint64_t *n_out) {
    if (fa_status s = check_table(bt)) return s;
    if (!n_out) return fail(FA_ERR_INVALID_ARGUMENT, "flatten_tables: null n_out");
    std::vector<uint32_t> flat;
    if (fa_status s = table_result(bt->t.flatten_tables((size_t)max_blocks_per_seq, &flat), "flatten_tables")) return s;
    if (flat.size() > out_capacity || (!flat.empty() && !out))
        return fail(FA_ERR_INVALID_ARGUMENT, "flatten_tables: output buffer too small");
    for (size_t i = 0; i < flat.size(); ++i) out[i] = flat[i];
    *n_out = flat.size();
    return FA_OK;
}

fa_status fa_block_table_rewind_to(fa_block_table *bt, uint64_t new_len, uint64_t block_size) {
    if (fa_status s = check_table(bt)) return s;
    if (block_size == 0) return fail(FA_ERR_INVALID_ARGUMENT, "rewind_to: block_size 0");
    BlockTable next;
    try {
        next = bt->t;
    } catch (const std::exception &) {
        return fail(FA_ERR_ALLOCATION_FAILED, "rewind_to: out of host memory");
    }
    if (fa_status s = table_result(next.rewind_to((size_t)new_len, (size_t)block_size), "rewind_to")) return s;
    bt->t = std::move(next);
    return FA_OK;
}

fa_status fa_paged_cache_check_config(uint64_t block_size, uint64_t max_blocks, uint64_t embed_dim, fa_dtype dtype) {
    if (dtype != FA_F32 && dtype != FA_BF16) return fail(FA_ERR_INVALID_ARGUMENT, "paged cache: pools are f32 or bf16");
    return table_result(check_cache_config((size_t)block_size, (size_t)max_blocks, (size_t)embed_dim, dtype_size(dtype)),
                        "paged cache config");
}

fa_status fa_paged_cache_create(fa_context *ctx, uint64_t block_size, uint64_t max_blocks, uint64_t embed_dim, fa_dtype dtype,
                                fa_paged_cache **out) {
    if (fa_status s = fa_paged_cache_check_config(block_size, max_blocks, embed_dim, dtype)) return s;
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "paged_cache_create: null out");
    if (fa_status s = check_ctx(ctx)) return s;
    // slot numbers are 32-bit (paged_kv_device.rs:99-107)
    if (max_blocks * block_size > 0xffffffffull)
        return fail(FA_ERR_INVALID_ARGUMENT, "paged_cache_create: max_blocks * block_size exceeds UINT32_MAX");
    fa_paged_cache *c = new (std::nothrow) fa_paged_cache();
    if (!c) return fail(FA_ERR_ALLOCATION_FAILED, "paged_cache_create: out of host memory");
    c->magic = kCacheMagic;
    c->ctx = ctx;
    c->block_size = block_size;
    c->max_blocks = max_blocks;
    c->embed_dim = embed_dim;
    c->dtype = dtype;
    c->layout = fa_paged_layout{max_blocks, block_size, embed_dim};
    c->k_pool = c->v_pool = nullptr;
    c->poisoned = false;
    uint64_t numel = max_blocks * block_size * embed_dim;
    fa_status s = fa_alloc_zeroed(ctx, dtype, numel, &c->k_pool);
    if (s == FA_OK) s = fa_alloc_zeroed(ctx, dtype, numel, &c->v_pool);
    if (s != FA_OK) {
        if (c->k_pool) fa_buffer_free(ctx, c->k_pool);
        delete c;
        return s;
    }
    *out = c;
    return FA_OK;
}

fa_status fa_paged_cache_destroy(fa_context *ctx, fa_paged_cache *c) {
    if (fa_status s = check_cache(c)) return s;
    if (c->k_pool) fa_buffer_free(ctx, c->k_pool);
    if (c->v_pool) fa_buffer_free(ctx, c->v_pool);
    c->magic = 0;
    delete c;
    return FA_OK;
}

fa_status fa_paged_cache_state_get(const fa_paged_cache *c, fa_block_table_state *out, int32_t *poisoned) {
    if (fa_status s = check_cache(c)) return s;
    if (out) fill_state(c->table, c->max_blocks, out);
    if (poisoned) *poisoned = c->poisoned ? 1 : 0;
    return FA_OK;
}

fa_status fa_paged_cache_pools(fa_paged_cache *c, fa_buffer **k_pool, fa_buffer **v_pool) {
    if (fa_status s = check_cache(c)) return s;
    if (k_pool) *k_pool = c->k_pool;
    if (v_pool) *v_pool = c->v_pool;
    return FA_OK;
}

fa_status fa_paged_cache_block_tables(const fa_paged_cache *c, uint64_t max_blocks_per_seq, uint32_t *out, uint64_t out_capacity,
                                      uint64_t *n_out) {
    if (fa_status s = check_cache(c)) return s;
    if (!n_out) return fail(FA_ERR_INVALID_ARGUMENT, "paged_cache_block_tables: null n_out");
    std::vector<uint32_t> flat;
    if (fa_status s = table_result(c->table.flatten_tables((size_t)max_blocks_per_seq, &flat), "flatten_tables")) return s;
    if (flat.size() > out_capacity || (!flat.empty() && !out))
        return fail(FA_ERR_INVALID_ARGUMENT, "paged_cache_block_tables: output buffer too small");
    for (size_t i = 0; i < flat.size(); ++i) out[i] = flat[i];
    *n_out = flat.size();
    return FA_OK;
}

fa_status fa_paged_cache_append(fa_context *ctx, fa_paged_cache *c, const fa_buffer *k_new, const fa_buffer *v_new, uint64_t b,
                                uint64_t l_new) {
    if (fa_status s = check_cache(c)) return s;
    if (c->poisoned) return fail(FA_ERR_STORE_POISONED, "paged cache is poisoned: build a new one");
    if (ctx != c->ctx) return fail(FA_ERR_DEVICE_MISMATCH, "paged_cache_append: cache belongs to another context");
    // allocation and slot computation on a copy; committed only after the device write was queued
    BlockTable next;
    std::vector<uint32_t> slots;
    try {
        next = c->table;
    } catch (const std::exception &) {
        return fail(FA_ERR_ALLOCATION_FAILED, "paged_cache_append: out of host memory");
    }
    if (fa_status s = table_result(next.extend_for_append((size_t)c->max_blocks, (size_t)c->block_size, (size_t)b, (size_t)l_new, &slots),
                                   "paged_cache_append"))
        return s;
    if (l_new == 0) return FA_OK;                         // validated only; the batch stays undetermined
    fa_status s = fa_paged_kv_append(ctx, k_new, v_new, c->k_pool, c->v_pool, slots.data(), slots.size(), &c->layout);
    if (s != FA_OK) {
        // argument errors are raised before anything is written; a failure after that may have left
        // part of the rows in the pool
        if (s != FA_ERR_INVALID_ARGUMENT && s != FA_ERR_SHAPE_MISMATCH && s != FA_ERR_DEVICE_MISMATCH && s != FA_ERR_UNSUPPORTED &&
            s != FA_ERR_CAPTURE_IN_PROGRESS)
            c->poisoned = true;
        return s;
    }
    c->table = std::move(next);
    return FA_OK;
}

fa_status fa_paged_cache_attention(fa_context *ctx, const fa_paged_cache *cc, const fa_buffer *q, uint64_t b, uint64_t l_new,
                                   uint64_t num_heads, uint64_t num_kv_heads, float scale, fa_buffer *out) {
    if (fa_status s = check_cache(cc)) return s;
    fa_paged_cache *c = const_cast<fa_paged_cache *>(cc);
    if (c->poisoned) return fail(FA_ERR_STORE_POISONED, "paged cache is poisoned: build a new one");
    if (ctx != c->ctx) return fail(FA_ERR_DEVICE_MISMATCH, "paged_cache_attention: cache belongs to another context");
    if (c->table.has_batch && c->table.batch != b) return fail(FA_ERR_INVALID_ARGUMENT, "paged_cache_attention: batch does not match the cache");
    const uint64_t s_total = c->table.seq_len();
    if (l_new > s_total) return fail(FA_ERR_INVALID_ARGUMENT, "paged_cache_attention: l_new exceeds the cached length (append first)");
    uint64_t max_blocks_per_seq = 1;
    for (const auto &row : c->table.tables) max_blocks_per_seq = std::max<uint64_t>(max_blocks_per_seq, row.size());
    fa_paged_args args{c->layout, b, l_new, num_heads, (l_new == 0 || b == 0) ? 1 : max_blocks_per_seq, scale, num_kv_heads};
    if (l_new == 0 || b == 0) {
        // the argument contract (heads divide the width, finite scale) is checked as for a non-empty call
        return paged_args_check(&args);
    }
    if (s_total > 0xffffffffull) return fail(FA_ERR_INVALID_ARGUMENT, "paged_cache_attention: sequence length exceeds 32 bits");
    std::vector<uint32_t> tables, lens;
    if (fa_status s = table_result(c->table.flatten_tables((size_t)max_blocks_per_seq, &tables), "paged_cache_attention")) return s;
    try {
        lens.assign((size_t)b, (uint32_t)s_total);
    } catch (const std::exception &) {
        return fail(FA_ERR_ALLOCATION_FAILED, "paged_cache_attention: out of host memory");
    }
    fa_status s = fa_paged_attention_forward(ctx, q, c->k_pool, c->v_pool, tables.data(), tables.size(), lens.data(), lens.size(),
                                             &args, out);
    if (s != FA_OK && s != FA_ERR_INVALID_ARGUMENT && s != FA_ERR_SHAPE_MISMATCH && s != FA_ERR_DEVICE_MISMATCH &&
        s != FA_ERR_UNSUPPORTED && s != FA_ERR_CAPTURE_IN_PROGRESS)
        c->poisoned = true;
    return s;
}

fa_status fa_paged_cache_rewind_to(fa_paged_cache *c, uint64_t new_len) {
    if (fa_status s = check_cache(c)) return s;
    BlockTable next;
    try {
        next = c->table;
    } catch (const std::exception &) {
        return fail(FA_ERR_ALLOCATION_FAILED, "paged_cache_rewind_to: out of host memory");
    }
    if (fa_status s = table_result(next.rewind_to((size_t)new_len, (size_t)c->block_size), "paged_cache_rewind_to")) return s;
    c->table = std::move(next);
    return FA_OK;
}

fa_status fa_paged_cache_clear(fa_paged_cache *c) {
    if (fa_status s = check_cache(c)) return s;
    c->table.reset();
    return FA_OK;
}

fa_status fa_paged_cache_snapshot_table(const fa_paged_cache *c, fa_block_table **out) {
    if (fa_status s = check_cache(c)) return s;
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "paged_cache_snapshot_table: null out");
    try {
        fa_block_table *bt = new fa_block_table();
        bt->magic = kTableMagic;
        bt->t = c->table;
        *out = bt;
    } catch (const std::exception &) {
        return fail(FA_ERR_ALLOCATION_FAILED, "paged_cache_snapshot_table: out of host memory");
    }
    return FA_OK;
}

fa_status fa_paged_cache_restore_table(fa_paged_cache *c, const fa_block_table *saved) {
    if (fa_status s = check_cache(c)) return s;
    if (fa_status s = check_table(saved)) return s;
    try {
        c->table = saved->t;
    } catch (const std::exception &) {
        return fail(FA_ERR_ALLOCATION_FAILED, "paged_cache_restore_table: out of host memory");
    }
    return FA_OK;
}

}  // extern "C"
