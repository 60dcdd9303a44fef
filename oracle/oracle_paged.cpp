// CPU oracle (test infrastructure only, see oracle.h): paged KV validators,
// append and attention.  Follows crates/tensor-core/src/paged_kv.rs and
// crates/backend-cpu/src/paged_kv.rs; the only extension is grouped-query
// attention (K/V pools num_kv_heads * Dh wide, kv head = h / group), which
// degenerates to the reference when num_kv_heads == num_heads.
#include "oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

static const uint64_t kMaxBlockSize = 256;                 // paged_kv.rs:32
static const uint64_t kMaxWorkspace = 1ull << 30;          // paged_kv.rs:36
static const uint64_t kIsizeMax = (uint64_t)INT64_MAX;

static bool mul_ok(uint64_t a, uint64_t b, uint64_t *r) { return !__builtin_mul_overflow(a, b, r); }

// crates/tensor-core/src/paged_kv.rs:82-131
extern "C" int orc_paged_layout_check(const orc_paged_layout *l) {
    uint64_t bs = l->block_size;
    if (bs == 0 || bs > kMaxBlockSize || (bs & (bs - 1)) != 0) return -1;
    if (l->num_blocks == 0 || l->num_blocks >= (uint64_t)UINT32_MAX) return -1;
    if (l->embed_dim == 0 || l->embed_dim > (uint64_t)INT32_MAX) return -1;
    uint64_t elems, bytes;
    if (!mul_ok(l->num_blocks, bs, &elems) || !mul_ok(elems, l->embed_dim, &elems)) return -1;
    if (!mul_ok(elems, 4, &bytes) || !mul_ok(bytes, 2, &bytes)) return -1;
    if (bytes > kIsizeMax) return -1;
    return 0;
}

static uint64_t kv_heads_of(const orc_paged_args *a) {
    return a->num_kv_heads == 0 ? a->num_heads : a->num_kv_heads;
}

// crates/tensor-core/src/paged_kv.rs:160-198
extern "C" int orc_paged_args_check(const orc_paged_args *a) {
    if (orc_paged_layout_check(&a->layout) != 0) return -1;
    if (a->batch > (uint64_t)INT32_MAX || a->l_new > (uint64_t)INT32_MAX ||
        a->max_blocks_per_seq > (uint64_t)INT32_MAX)
        return -1;
    uint64_t hkv = kv_heads_of(a);
    if (a->num_heads == 0 || hkv == 0) return -1;
    if (a->layout.embed_dim % hkv != 0) return -1;
    if (a->num_heads % hkv != 0) return -1;
    if (!std::isfinite(a->scale)) return -1;
    return 0;
}

// crates/tensor-core/src/paged_kv.rs:222-268
extern "C" int64_t orc_validate_paged_kv_append(uint64_t k_new_numel, uint64_t v_new_numel,
                                                uint64_t k_pool_numel, uint64_t v_pool_numel,
                                                const uint32_t *slot_mapping, uint64_t rows,
                                                const orc_paged_layout *l) {
    if (orc_paged_layout_check(l) != 0) return -1;
    uint64_t expect;
    if (!mul_ok(rows, l->embed_dim, &expect)) return -1;
    if (k_new_numel != expect || v_new_numel != expect) return -1;
    if (rows > (uint64_t)INT32_MAX) return -1;
    uint64_t pool_rows = l->num_blocks * l->block_size;
    uint64_t pool = pool_rows * l->embed_dim;
    if (k_pool_numel != pool || v_pool_numel != pool) return -1;
    std::vector<uint32_t> sorted(slot_mapping, slot_mapping + rows);
    for (uint32_t s : sorted)
        if ((uint64_t)s >= pool_rows) return -1;
    std::sort(sorted.begin(), sorted.end());
    for (size_t i = 1; i < sorted.size(); ++i)
        if (sorted[i] == sorted[i - 1]) return -1;
    return (int64_t)rows;
}

// crates/tensor-core/src/paged_kv.rs:277-373
extern "C" int orc_validate_paged_attention(uint64_t q_numel, uint64_t k_pool_numel,
                                            uint64_t v_pool_numel, const uint32_t *block_tables,
                                            uint64_t n_tables, const uint32_t *seq_lens,
                                            uint64_t n_seq, const orc_paged_args *a,
                                            orc_paged_plan *plan) {
    if (orc_paged_args_check(a) != 0) return -1;
    const orc_paged_layout *l = &a->layout;
    uint64_t dh = l->embed_dim / kv_heads_of(a);
    uint64_t e_q;
    if (!mul_ok(a->num_heads, dh, &e_q)) return -1;
    uint64_t out_numel;
    if (!mul_ok(a->batch, a->l_new, &out_numel) || !mul_ok(out_numel, e_q, &out_numel)) return -1;
    if (q_numel != out_numel) return -1;
    uint64_t pool = l->num_blocks * l->block_size * l->embed_dim;
    if (k_pool_numel != pool || v_pool_numel != pool) return -1;
    uint64_t tables_len;
    if (!mul_ok(a->batch, a->max_blocks_per_seq, &tables_len)) return -1;
    if (n_tables != tables_len) return -1;
    if (n_seq != a->batch) return -1;
    uint64_t max_seq;
    if (!mul_ok(a->max_blocks_per_seq, l->block_size, &max_seq)) return -1;
    uint64_t s_max = 0;
    for (uint64_t b = 0; b < a->batch; ++b) {
        uint64_t sl = seq_lens[b];
        if (sl < a->l_new || sl > max_seq) return -1;
        s_max = std::max(s_max, sl);
        uint64_t used = (sl + l->block_size - 1) / l->block_size;
        for (uint64_t slot = 0; slot < used; ++slot)
            if ((uint64_t)block_tables[b * a->max_blocks_per_seq + slot] >= l->num_blocks) return -1;
    }
    uint64_t query_rows;
    if (!mul_ok(a->batch, a->num_heads, &query_rows) || !mul_ok(query_rows, a->l_new, &query_rows))
        return -1;
    if (query_rows > (uint64_t)INT32_MAX || s_max > (uint64_t)INT32_MAX) return -1;
    uint64_t ws;
    if (!mul_ok(query_rows, s_max, &ws)) return -1;
    if (ws > kMaxWorkspace) return -1;
    if (plan) {
        plan->out_numel = out_numel;
        plan->s_max = s_max;
        plan->query_rows = query_rows;
        plan->workspace_elems = ws;
    }
    return 0;
}

// crates/backend-cpu/src/paged_kv.rs:33-66
extern "C" int orc_paged_kv_append(const void *k_new, const void *v_new, void *k_pool,
                                   void *v_pool, const uint32_t *slot_mapping, uint64_t rows,
                                   const orc_paged_layout *l, size_t elem_bytes) {
    size_t row_bytes = (size_t)l->embed_dim * elem_bytes;
    uint64_t pool_rows = l->num_blocks * l->block_size;
    for (uint64_t r = 0; r < rows; ++r) {
        uint64_t slot = slot_mapping[r];
        if (slot >= pool_rows) return -1;
        std::memcpy((char *)k_pool + slot * row_bytes, (const char *)k_new + r * row_bytes, row_bytes);
        std::memcpy((char *)v_pool + slot * row_bytes, (const char *)v_new + r * row_bytes, row_bytes);
    }
    return 0;
}

// crates/backend-cpu/src/paged_kv.rs:69-93 (row_offset) and :96-178 (attention)
template <typename LoadQ, typename LoadKV>
static int attention_impl(LoadQ q_at, LoadKV k_at, LoadKV v_at, const uint32_t *block_tables,
                          const uint32_t *seq_lens, const orc_paged_args *a, float *out) {
    const uint64_t e_kv = a->layout.embed_dim, bs = a->layout.block_size;
    const uint64_t hkv = kv_heads_of(a), dh = e_kv / hkv, group = a->num_heads / hkv;
    const uint64_t e_q = a->num_heads * dh;
    int status = 0;
    int nt = orc_get_threads();
    const int64_t work = (int64_t)(a->batch * a->num_heads);
#pragma omp parallel num_threads(nt) if (nt > 1 && work > 1)
    {
        std::vector<float> weights;
#pragma omp for schedule(dynamic, 1)
        for (int64_t bh = 0; bh < work; ++bh) {
            uint64_t b = (uint64_t)bh / a->num_heads, h = (uint64_t)bh % a->num_heads;
            uint64_t kvh = h / group;
            uint64_t s_total = seq_lens[b];
            if (s_total < a->l_new) {
#pragma omp atomic write
                status = -1;
                continue;
            }
            uint64_t s_prev = s_total - a->l_new;
            weights.resize((size_t)s_total);
            for (uint64_t i = 0; i < a->l_new; ++i) {
                uint64_t q_off = (b * a->l_new + i) * e_q + h * dh;
                uint64_t limit = s_prev + i + 1;
                float mx = -INFINITY;
                bool bad = false;
                for (uint64_t j = 0; j < limit; ++j) {
                    uint64_t blk = block_tables[b * a->max_blocks_per_seq + j / bs];
                    if (blk >= a->layout.num_blocks) { bad = true; break; }
                    uint64_t off = (blk * bs + j % bs) * e_kv + kvh * dh;
                    float acc = 0.0f;
                    for (uint64_t d = 0; d < dh; ++d) {
                        float qs = q_at(q_off + d) * a->scale;
                        acc = std::fmaf(qs, k_at(off + d), acc);
                    }
                    weights[j] = acc;
                    if (acc > mx) mx = acc;
                }
                if (bad) {
#pragma omp atomic write
                    status = -1;
                    continue;
                }
                float sum = 0.0f;
                for (uint64_t j = 0; j < limit; ++j) {
                    weights[j] = std::exp(weights[j] - mx);
                    sum += weights[j];
                }
                float *o_row = out + q_off;
                for (uint64_t d = 0; d < dh; ++d) o_row[d] = 0.0f;
                for (uint64_t j = 0; j < limit; ++j) {
                    float p = weights[j] / sum;
                    uint64_t blk = block_tables[b * a->max_blocks_per_seq + j / bs];
                    uint64_t off = (blk * bs + j % bs) * e_kv + kvh * dh;
                    for (uint64_t d = 0; d < dh; ++d) o_row[d] = std::fmaf(p, v_at(off + d), o_row[d]);
                }
            }
        }
    }
    return status;
}

extern "C" int orc_paged_attention_f32(const float *q, const float *k_pool, const float *v_pool,
                                       const uint32_t *block_tables, const uint32_t *seq_lens,
                                       const orc_paged_args *a, float *out) {
    if (orc_paged_args_check(a) != 0) return -1;
    struct F32At {
        const float *p;
        float operator()(uint64_t i) const { return p[i]; }
    };
    return attention_impl(F32At{q}, F32At{k_pool}, F32At{v_pool}, block_tables, seq_lens, a, out);
}

extern "C" int orc_paged_attention_bf16(const uint16_t *q, const uint16_t *k_pool,
                                        const uint16_t *v_pool, const uint32_t *block_tables,
                                        const uint32_t *seq_lens, const orc_paged_args *a,
                                        float *out_f32) {
    if (orc_paged_args_check(a) != 0) return -1;
    struct Bf16At {
        const uint16_t *p;
        float operator()(uint64_t i) const { return orc_bf16_to_f32(p[i]); }
    };
    return attention_impl(Bf16At{q}, Bf16At{k_pool}, Bf16At{v_pool}, block_tables, seq_lens, a,
                          out_f32);
}

// Straight f64 softmax(QK^T)V over the gathered rows: pins the two functions
// above on small cases (different precision, different loop structure).
extern "C" int orc_paged_attention_f64(const double *q, const double *k_pool,
                                       const double *v_pool, const uint32_t *block_tables,
                                       const uint32_t *seq_lens, const orc_paged_args *a,
                                       double *out) {
    if (orc_paged_args_check(a) != 0) return -1;
    const uint64_t e_kv = a->layout.embed_dim, bs = a->layout.block_size;
    const uint64_t hkv = kv_heads_of(a), dh = e_kv / hkv, group = a->num_heads / hkv;
    const uint64_t e_q = a->num_heads * dh;
    for (uint64_t b = 0; b < a->batch; ++b)
        for (uint64_t i = 0; i < a->l_new; ++i)
            for (uint64_t h = 0; h < a->num_heads; ++h) {
                uint64_t limit = seq_lens[b] - a->l_new + i + 1;
                const double *qr = q + (b * a->l_new + i) * e_q + h * dh;
                std::vector<double> s((size_t)limit);
                double mx = -INFINITY;
                for (uint64_t j = 0; j < limit; ++j) {
                    uint64_t row = (uint64_t)block_tables[b * a->max_blocks_per_seq + j / bs] * bs + j % bs;
                    const double *kr = k_pool + row * e_kv + (h / group) * dh;
                    double acc = 0.0;
                    for (uint64_t d = 0; d < dh; ++d) acc += qr[d] * kr[d];
                    s[j] = acc * (double)a->scale;
                    mx = std::max(mx, s[j]);
                }
                double sum = 0.0;
                for (uint64_t j = 0; j < limit; ++j) {
                    s[j] = std::exp(s[j] - mx);
                    sum += s[j];
                }
                double *o = out + (b * a->l_new + i) * e_q + h * dh;
                for (uint64_t d = 0; d < dh; ++d) o[d] = 0.0;
                for (uint64_t j = 0; j < limit; ++j) {
                    uint64_t row = (uint64_t)block_tables[b * a->max_blocks_per_seq + j / bs] * bs + j % bs;
                    const double *vr = v_pool + row * e_kv + (h / group) * dh;
                    for (uint64_t d = 0; d < dh; ++d) o[d] += s[j] / sum * vr[d];
                }
            }
    return 0;
}
