// Host-side argument validation for the paged KV entry points.  Pure
// functions: they run before anything touches the device and are callable
// without one.  Behaviour follows crates/tensor-core/src/paged_kv.rs:59-373;
// the one extension is num_kv_heads for grouped-query attention.
#include "validate.hpp"

#include <algorithm>
#include <cmath>
#include <string>
#include <vector>

namespace fa {

static const uint64_t kMaxBlockSize = 256;            // PAGED_KV_MAX_BLOCK_SIZE
static const uint64_t kMaxWorkspaceElems = 1ull << 30; // PAGED_ATTENTION_MAX_WORKSPACE_ELEMS

static fa_status invalid(const std::string &msg) { return fail(FA_ERR_INVALID_ARGUMENT, "paged_kv: " + msg); }

static bool mul(uint64_t a, uint64_t b, uint64_t *r) { return !__builtin_mul_overflow(a, b, r); }

fa_status paged_layout_check(const fa_paged_layout *l) {
    if (!l) return invalid("null layout");
    uint64_t bs = l->block_size;
    if (bs == 0 || bs > kMaxBlockSize || (bs & (bs - 1)) != 0)
        return invalid("block_size must be a power of two in 1..256 (got " + std::to_string(bs) + ")");
    if (l->num_blocks == 0 || l->num_blocks >= (uint64_t)UINT32_MAX)
        return invalid("num_blocks must be in 1..u32::MAX-1 (got " + std::to_string(l->num_blocks) + ")");
    if (l->embed_dim == 0 || l->embed_dim > (uint64_t)INT32_MAX)
        return invalid("embed_dim must be in 1..i32::MAX (got " + std::to_string(l->embed_dim) + ")");
    uint64_t elems, bytes;
    if (!mul(l->num_blocks, bs, &elems) || !mul(elems, l->embed_dim, &elems))
        return invalid("pool element count overflows");
    if (!mul(elems, 4, &bytes) || !mul(bytes, 2, &bytes) || bytes > (uint64_t)INT64_MAX)
        return invalid("pool byte size exceeds isize::MAX");
    return FA_OK;
}

uint64_t paged_kv_heads(const fa_paged_args *a) { return a->num_kv_heads == 0 ? a->num_heads : a->num_kv_heads; }

fa_status paged_args_check(const fa_paged_args *a) {
    if (!a) return invalid("null args");
    if (fa_status s = paged_layout_check(&a->layout)) return s;
    if (a->batch > (uint64_t)INT32_MAX) return invalid("batch exceeds i32::MAX");
    if (a->l_new > (uint64_t)INT32_MAX) return invalid("l_new exceeds i32::MAX");
    if (a->max_blocks_per_seq > (uint64_t)INT32_MAX) return invalid("max_blocks_per_seq exceeds i32::MAX");
    uint64_t hkv = paged_kv_heads(a);
    if (a->num_heads == 0 || hkv == 0 || a->layout.embed_dim % hkv != 0)
        return invalid("the number of heads must be positive and divide embed_dim");
    if (a->num_heads % hkv != 0) return invalid("num_heads must be a multiple of num_kv_heads");
    if (!std::isfinite(a->scale)) return invalid("scale must be finite");
    return FA_OK;
}

}  // namespace fa

using namespace fa;

extern "C" {

fa_status fa_validate_paged_kv_append(uint64_t k_new_numel, uint64_t v_new_numel, uint64_t k_pool_numel,
                                      uint64_t v_pool_numel, const uint32_t *slot_mapping, uint64_t rows,
                                      const fa_paged_layout *layout) {
    if (fa_status s = paged_layout_check(layout)) return s;
    if (rows != 0 && !slot_mapping) return invalid("null slot_mapping");
    uint64_t expect;
    if (!mul(rows, layout->embed_dim, &expect)) return invalid("appended element count overflows");
    if (k_new_numel != expect || v_new_numel != expect)
        return invalid("k_new / v_new hold " + std::to_string(k_new_numel) + " / " + std::to_string(v_new_numel) +
                       " elements, slot_mapping.len() * E = " + std::to_string(expect));
    if (rows > (uint64_t)INT32_MAX) return invalid("more than i32::MAX appended rows");
    uint64_t pool_rows = layout->num_blocks * layout->block_size;
    uint64_t pool = pool_rows * layout->embed_dim;
    if (k_pool_numel != pool || v_pool_numel != pool)
        return invalid("pool sizes do not match the layout (expected " + std::to_string(pool) + ")");
    std::vector<uint32_t> sorted;
    try {
        sorted.assign(slot_mapping, slot_mapping + rows);
    } catch (...) {
        return invalid("cannot allocate the slot check buffer");
    }
    for (uint32_t sl : sorted)
        if ((uint64_t)sl >= pool_rows)
            return invalid("slot " + std::to_string(sl) + " is not below the pool row count " + std::to_string(pool_rows));
    std::sort(sorted.begin(), sorted.end());
    for (size_t i = 1; i < sorted.size(); ++i)
        if (sorted[i] == sorted[i - 1]) return invalid("duplicate slot in slot_mapping");
    return FA_OK;
}

fa_status fa_validate_paged_attention(uint64_t q_numel, uint64_t k_pool_numel, uint64_t v_pool_numel,
                                      const uint32_t *block_tables, uint64_t n_tables, const uint32_t *seq_lens,
                                      uint64_t n_seq, const fa_paged_args *args, fa_paged_plan *plan) {
    if (fa_status s = paged_args_check(args)) return s;
    const fa_paged_layout *l = &args->layout;
    uint64_t dh = l->embed_dim / paged_kv_heads(args);
    uint64_t e_q, out_numel;
    if (!mul(args->num_heads, dh, &e_q)) return invalid("query width overflows");
    if (!mul(args->batch, args->l_new, &out_numel) || !mul(out_numel, e_q, &out_numel))
        return invalid("output element count overflows");
    if (q_numel != out_numel)
        return invalid("q holds " + std::to_string(q_numel) + " elements, B * L_new * E = " + std::to_string(out_numel));
    uint64_t pool = l->num_blocks * l->block_size * l->embed_dim;
    if (k_pool_numel != pool || v_pool_numel != pool) return invalid("pool sizes do not match the layout");
    uint64_t tables_len;
    if (!mul(args->batch, args->max_blocks_per_seq, &tables_len)) return invalid("block table size overflows");
    if (n_tables != tables_len)
        return invalid("block_tables.len() = " + std::to_string(n_tables) + ", B * max_blocks_per_seq = " +
                       std::to_string(tables_len));
    if (n_seq != args->batch) return invalid("seq_lens.len() does not equal B");
    if ((n_tables != 0 && !block_tables) || (n_seq != 0 && !seq_lens)) return invalid("null table pointer");
    uint64_t max_seq;
    if (!mul(args->max_blocks_per_seq, l->block_size, &max_seq)) return invalid("max sequence length overflows");
    uint64_t s_max = 0;
    for (uint64_t b = 0; b < args->batch; ++b) {
        uint64_t sl = seq_lens[b];
        if (sl < args->l_new || sl > max_seq)
            return invalid("row " + std::to_string(b) + ": seq_len " + std::to_string(sl) + " outside [" +
                           std::to_string(args->l_new) + ", " + std::to_string(max_seq) + "]");
        s_max = std::max(s_max, sl);
        uint64_t used = (sl + l->block_size - 1) / l->block_size;
        for (uint64_t slot = 0; slot < used; ++slot) {
            uint64_t id = block_tables[b * args->max_blocks_per_seq + slot];
            if (id >= l->num_blocks)
                return invalid("row " + std::to_string(b) + " entry " + std::to_string(slot) + ": block id " +
                               std::to_string(id) + " is not below num_blocks (sentinel included)");
        }
    }
    uint64_t query_rows;
    if (!mul(args->batch, args->num_heads, &query_rows) || !mul(query_rows, args->l_new, &query_rows))
        return invalid("query row count overflows");
    if (query_rows > (uint64_t)INT32_MAX) return invalid("B * H * L_new exceeds i32::MAX");
    if (s_max > (uint64_t)INT32_MAX) return invalid("sequence length exceeds i32::MAX");
    uint64_t ws;
    if (!mul(query_rows, s_max, &ws)) return invalid("workspace element count overflows");
    if (ws > kMaxWorkspaceElems) return invalid("workspace of " + std::to_string(ws) + " elements exceeds the cap");
    if (plan) {
        plan->out_numel = out_numel;
        plan->s_max = s_max;
        plan->query_rows = query_rows;
        plan->workspace_elems = ws;
    }
    return FA_OK;
}

}  // extern "C"
