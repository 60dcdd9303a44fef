// Paged KV cache kernels: row scatter (append), a generic attention kernel
// that keeps the reference's per-row summation order, and the decode fast
// path (bf16, head_dim 128, 16-token pages, one query token, grouped-query).
#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {
using namespace fa::dev;

namespace {

// ------------------------------------------------------------------ append
// crates/backend-cpu/src/paged_kv.rs:33-66: pool row slot[r] <- new row r.
template <typename U>
__global__ void __launch_bounds__(256)
    append_kernel(const U *__restrict__ k_new, const U *__restrict__ v_new, U *__restrict__ k_pool,
                  U *__restrict__ v_pool, const uint32_t *__restrict__ slots, uint64_t units_per_row,
                  uint64_t pool_rows) {
    uint64_t r = blockIdx.x;
    uint64_t slot = slots[r];
    if (slot >= pool_rows) return;          // never true for host-validated tables
    const U *ks = k_new + r * units_per_row, *vs = v_new + r * units_per_row;
    U *kd = k_pool + slot * units_per_row, *vd = v_pool + slot * units_per_row;
    for (uint64_t i = threadIdx.x; i < units_per_row; i += 256) {
        kd[i] = ks[i];
        vd[i] = vs[i];
    }
}

// ------------------------------------------------------- generic attention
template <bool BF16>
__device__ __forceinline__ float ld(const void *p, uint64_t i) {
    if (BF16) return bf16_to_f32(((const uint16_t *)p)[i]);
    return ((const float *)p)[i];
}

// One block per query row (b, h, i).  Scores: each thread owns whole dot
// products (d ascending, fused multiply-add on q*scale) exactly as
// crates/backend-cpu/src/paged_kv.rs:131-147; the weighted sum over V runs
// j ascending per output element as in :158-172.  Only max and the sum of
// exponentials are reduced across threads.
template <bool BF16>
__global__ void __launch_bounds__(128)
    attention_generic_kernel(const void *__restrict__ q, const void *__restrict__ k_pool,
                             const void *__restrict__ v_pool, const uint32_t *__restrict__ tables,
                             const uint32_t *__restrict__ seq_lens, PagedShape ps, float *__restrict__ workspace,
                             uint64_t s_stride, void *__restrict__ out) {
    extern __shared__ float q_s[];                  // head_dim floats
    __shared__ float red[2];
    __shared__ int bad_s;
    const uint32_t dh = ps.head_dim, bs = ps.block_size;
    const uint32_t group = ps.num_heads / ps.num_kv_heads;
    const uint64_t e_q = (uint64_t)ps.num_heads * dh, e_kv = ps.e_kv;
    uint32_t row = blockIdx.x;
    uint32_t i = row % ps.l_new, h = (row / ps.l_new) % ps.num_heads, b = row / (ps.l_new * ps.num_heads);
    uint32_t kvh = h / group;
    uint32_t s_total = seq_lens[b];
    uint64_t q_off = ((uint64_t)b * ps.l_new + i) * e_q + (uint64_t)h * dh;
    bool bad = s_total < ps.l_new || (uint64_t)s_total > (uint64_t)ps.max_blocks_per_seq * bs;
    uint32_t limit = bad ? 0 : s_total - ps.l_new + i + 1;
    if (threadIdx.x == 0) bad_s = 0;
    for (uint32_t d = threadIdx.x; d < dh; d += 128) q_s[d] = ld<BF16>(q, q_off + d) * ps.scale;
    __syncthreads();

    float *w = workspace + (uint64_t)row * s_stride;
    const uint32_t *tab = tables + (uint64_t)b * ps.max_blocks_per_seq;
    float mx = -INFINITY;
    for (uint32_t j = threadIdx.x; j < limit; j += 128) {
        uint32_t blk = tab[j / bs];
        if (blk >= ps.num_blocks) {
            bad_s = 1;
            continue;
        }
        uint64_t off = ((uint64_t)blk * bs + j % bs) * e_kv + (uint64_t)kvh * dh;
        float acc = 0.0f;
        for (uint32_t d = 0; d < dh; ++d) acc = __builtin_fmaf(q_s[d], ld<BF16>(k_pool, off + d), acc);
        w[j] = acc;
        mx = fmaxf(mx, acc);
    }
    mx = wave_max(mx);
    __syncthreads();
    if (threadIdx.x % 64 == 0) red[threadIdx.x / 64] = mx;
    __syncthreads();
    mx = fmaxf(red[0], red[1]);
    bad = bad || bad_s != 0;
    float sum = 0.0f;
    if (!bad)
        for (uint32_t j = threadIdx.x; j < limit; j += 128) {
            float e = expf(w[j] - mx);
            w[j] = e;
            sum += e;
        }
    sum = wave_sum(sum);
    __syncthreads();
    if (threadIdx.x % 64 == 0) red[threadIdx.x / 64] = sum;
    __syncthreads();                                 // also orders the w[] writes before the reads below
    sum = red[0] + red[1];
    for (uint32_t d = threadIdx.x; d < dh; d += 128) {
        float o = 0.0f;
        if (bad) {
            o = __uint_as_float(0x7fc00000u);        // violation: NaN, never a silent zero
        } else {
            for (uint32_t j = 0; j < limit; ++j) {
                uint32_t blk = tab[j / bs];
                uint64_t off = ((uint64_t)blk * bs + j % bs) * e_kv + (uint64_t)kvh * dh;
                float p = __fdiv_rn(w[j], sum);
                o = __builtin_fmaf(p, ld<BF16>(v_pool, off + d), o);
            }
        }
        if (BF16)
            ((uint16_t *)out)[q_off + d] = f32_to_bf16(o);
        else
            ((float *)out)[q_off + d] = o;
    }
}

// ------------------------------------------------------- decode fast path
// Work item = (sequence b, kv head, chunk of PPC pages); one wavefront each,
// four per block.  Per page the wavefront
//   1. loads the K slice (16 tokens x 128 dims, 4 KiB) straight into the A
//      operand of v_mfma_f32_16x16x32_bf16 (lane (g, r): token r, dims
//      32*s + 8*g .. +7 for step s) and multiplies by Q^T (B operand, column =
//      query head of the group), giving S^T[token 4g+j][head c] in lane (g, c);
//   2. keeps the scaled, masked scores in registers; after the last page of the
//      chunk takes the chunk maximum per head and the exponentials;
//   3. routes the weights through LDS ([token][head]) and accumulates
//      O[head][8 dims] per lane from V rows loaded 16 bytes per lane
//      (lane (g, c): tokens 4g+j, dims 8c .. 8c+7).
// The chunk's unnormalized O, its maximum and its sum go to the workspace; a
// second kernel merges the chunks of a sequence.  K and V bytes are read once
// for the whole group of query heads.
constexpr int kDh = 128, kPage = 16;

struct DecodeParams {
    const uint16_t *q, *k_pool, *v_pool;
    const uint32_t *tables, *seq_lens;
    float *part_o;      // [items][G_PAD][128]
    float *part_ml;     // [items][2][G_PAD]
    uint32_t num_blocks, e_kv, batch, num_heads, num_kv_heads, group, max_blocks_per_seq, max_chunks;
    float scale;
};

template <int G_PAD, int PPC>
__global__ void __launch_bounds__(256) decode_chunk_kernel(DecodeParams p) {
    constexpr int DEPTH = PPC < 4 ? PPC : 4;            // pages of loads in flight
    __shared__ float p_s[4][PPC * kPage][G_PAD];
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int g = lane / 16, c = lane % 16;
    const uint32_t chunk = blockIdx.x * 4 + wave;
    const uint32_t kvh = blockIdx.y, b = blockIdx.z;
    if (chunk >= p.max_chunks) return;
    uint32_t ctx = p.seq_lens[b];
    bool bad = (uint64_t)ctx > (uint64_t)p.max_blocks_per_seq * kPage;
    if (bad) ctx = p.max_blocks_per_seq * kPage;
    const uint32_t n_pages = (ctx + kPage - 1) / kPage;
    const uint32_t p0 = chunk * PPC;
    if (p0 >= n_pages) return;
    const uint32_t np = n_pages - p0 < (uint32_t)PPC ? n_pages - p0 : (uint32_t)PPC;
    const uint32_t *tab = p.tables + (uint64_t)b * p.max_blocks_per_seq + p0;

    // page ids of the chunk; positions past the end repeat the last page
    // (their scores are masked) so that the loads stay unconditional
    uint32_t ids[PPC];
#pragma unroll
    for (int i = 0; i < PPC; ++i) {
        uint32_t pi = (uint32_t)i < np ? (uint32_t)i : np - 1;
        uint32_t id = tab[pi];
        if (id >= p.num_blocks) {
            bad = true;
            id = 0;
        }
        ids[i] = id;
    }

    // Q^T operand: column c = head of the group (zero beyond the group)
    v8bf qb[4];
    {
        const uint16_t *qrow = p.q + ((uint64_t)b * p.num_heads + (uint64_t)kvh * p.group + c) * kDh + 8 * g;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            v4u t = v4u{0, 0, 0, 0};
            if ((uint32_t)c < p.group) t = *(const v4u *)(qrow + 32 * s);
            qb[s] = __builtin_bit_cast(v8bf, t);
        }
    }

    const uint64_t page_elems = (uint64_t)kPage * p.e_kv;
    const uint64_t k_lane = (uint64_t)c * p.e_kv + (uint64_t)kvh * kDh + 8 * g;       // token c, dims 8g..
    const uint64_t v_lane = (uint64_t)(4 * g) * p.e_kv + (uint64_t)kvh * kDh + 8 * c;  // tokens 4g.., dims 8c..

    // ---- pass 1: scores
    v4u kreg[DEPTH][4];
    auto load_k = [&](int i, v4u *dst) {
        const uint16_t *base = p.k_pool + (uint64_t)ids[i] * page_elems + k_lane;
#pragma unroll
        for (int s = 0; s < 4; ++s) dst[s] = *(const v4u *)(base + 32 * s);
    };
#pragma unroll
    for (int i = 0; i < DEPTH; ++i) load_k(i, kreg[i]);

    float sc[PPC][4];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < PPC; ++i) {
        v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; ++s)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, kreg[i % DEPTH][s]), qb[s], acc, 0,
                                                          0, 0);
        if (i + DEPTH < PPC) load_k(i + DEPTH, kreg[i % DEPTH]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t tok = (p0 + i) * kPage + 4 * g + j;
            float s = (uint32_t)i < np && tok < ctx ? acc[j] * p.scale : -INFINITY;
            sc[i][j] = s;
            mx = fmaxf(mx, s);
        }
    }
    // first V pages are requested before the softmax arithmetic
    v4u vreg[DEPTH][4];
    auto load_v = [&](int i, v4u *dst) {
        const uint16_t *base = p.v_pool + (uint64_t)ids[i] * page_elems + v_lane;
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[j] = *(const v4u *)(base + (uint64_t)j * p.e_kv);
    };
#pragma unroll
    for (int i = 0; i < DEPTH; ++i) load_v(i, vreg[i]);

    // chunk maximum and sum per head: lanes with equal c hold one head
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    float lsum = 0.0f;
#pragma unroll
    for (int i = 0; i < PPC; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float e = expf(sc[i][j] - mx);              // masked scores: exp(-inf) = 0
            sc[i][j] = e;
            lsum += e;
        }
    lsum += __shfl_xor(lsum, 16, 64);
    lsum += __shfl_xor(lsum, 32, 64);
    if (c < G_PAD) {
#pragma unroll
        for (int i = 0; i < PPC; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) p_s[wave][i * kPage + 4 * g + j][c] = sc[i][j];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // ---- pass 2: O[h][8 dims] += p[token][h] * V[token][8 dims]
    float o[G_PAD][8];
#pragma unroll
    for (int h = 0; h < G_PAD; ++h)
#pragma unroll
        for (int d = 0; d < 8; ++d) o[h][d] = 0.0f;
#pragma unroll
    for (int i = 0; i < PPC; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v4u raw = vreg[i % DEPTH][j];
            float vv[8];
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                vv[2 * d] = bf16_lo(raw[d]);
                vv[2 * d + 1] = bf16_hi(raw[d]);
            }
            float pw[G_PAD];
#pragma unroll
            for (int h = 0; h < G_PAD; ++h) pw[h] = p_s[wave][i * kPage + 4 * g + j][h];
#pragma unroll
            for (int h = 0; h < G_PAD; ++h)
#pragma unroll
                for (int d = 0; d < 8; ++d) o[h][d] = __builtin_fmaf(pw[h], vv[d], o[h][d]);
        }
        if (i + DEPTH < PPC) load_v(i + DEPTH, vreg[i % DEPTH]);
    }
    // merge the four token quarters
#pragma unroll
    for (int h = 0; h < G_PAD; ++h)
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            float v = o[h][d];
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            o[h][d] = v;
        }
    const uint64_t item = ((uint64_t)b * p.num_kv_heads + kvh) * p.max_chunks + chunk;
    if (g == 0) {
        float *po = p.part_o + item * (G_PAD * kDh) + 8 * c;
#pragma unroll
        for (int h = 0; h < G_PAD; ++h) {
            *(v4f *)(po + h * kDh) = v4f{o[h][0], o[h][1], o[h][2], o[h][3]};
            *(v4f *)(po + h * kDh + 4) = v4f{o[h][4], o[h][5], o[h][6], o[h][7]};
        }
        if (c < G_PAD) {
            float nanv = __uint_as_float(0x7fc00000u);
            p.part_ml[item * (2 * G_PAD) + c] = bad ? nanv : mx;
            p.part_ml[item * (2 * G_PAD) + G_PAD + c] = bad ? nanv : lsum;
        }
    }
}

// Merges the chunks of one (sequence, query head): block of 128 threads = dims.
template <int G_PAD, int PPC>
__global__ void __launch_bounds__(128) decode_merge_kernel(DecodeParams p, void *__restrict__ out, int out_bf16) {
    const uint32_t h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
    const uint32_t kvh = h / p.group, hg = h % p.group;
    uint32_t ctx = p.seq_lens[b];
    uint32_t max_ctx = p.max_blocks_per_seq * kPage;
    if (ctx > max_ctx) ctx = max_ctx;
    const uint32_t n_pages = (ctx + kPage - 1) / kPage;
    const uint32_t n_chunks = (n_pages + PPC - 1) / PPC;
    const uint64_t item0 = ((uint64_t)b * p.num_kv_heads + kvh) * p.max_chunks;
    float mx = -INFINITY;
    for (uint32_t ch = 0; ch < n_chunks; ++ch) {
        float m = p.part_ml[(item0 + ch) * (2 * G_PAD) + hg];
        mx = (m != m) ? m : fmaxf(mx, m);               // NaN marks a violation and must survive
        if (mx != mx) break;
    }
    float acc = 0.0f, den = 0.0f;
    for (uint32_t ch = 0; ch < n_chunks; ++ch) {
        float m = p.part_ml[(item0 + ch) * (2 * G_PAD) + hg];
        float l = p.part_ml[(item0 + ch) * (2 * G_PAD) + G_PAD + hg];
        float w = expf(m - mx);
        den = __builtin_fmaf(w, l, den);
        acc = __builtin_fmaf(w, p.part_o[(item0 + ch) * (G_PAD * kDh) + hg * kDh + d], acc);
    }
    float r = n_chunks == 0 ? 0.0f : __fdiv_rn(acc, den);
    uint64_t o = ((uint64_t)b * p.num_heads + h) * kDh + d;
    if (out_bf16)
        ((uint16_t *)out)[o] = f32_to_bf16(r);
    else
        ((float *)out)[o] = r;
}

inline int group_pad(uint32_t group) {
    int gp = 1;
    while ((uint32_t)gp < group) gp *= 2;
    return gp;
}

template <int G_PAD, int PPC>
void launch_decode(const DecodeParams &p, void *out, int out_bf16, hipStream_t s) {
    dim3 grid((p.max_chunks + 3) / 4, p.num_kv_heads, p.batch);
    decode_chunk_kernel<G_PAD, PPC><<<grid, 256, 0, s>>>(p);
    dim3 grid2(p.num_heads, p.batch);
    decode_merge_kernel<G_PAD, PPC><<<grid2, 128, 0, s>>>(p, out, out_bf16);
}

template <int G_PAD>
void launch_decode_ppc(const DecodeParams &p, uint32_t ppc, void *out, int out_bf16, hipStream_t s) {
    switch (ppc) {
        case 4: launch_decode<G_PAD, 4>(p, out, out_bf16, s); break;
        case 16: launch_decode<G_PAD, 16>(p, out, out_bf16, s); break;
        default: launch_decode<G_PAD, 8>(p, out, out_bf16, s); break;
    }
}

}  // namespace

void paged_kv_append(const void *k_new, const void *v_new, void *k_pool, void *v_pool, const uint32_t *slots,
                     uint64_t rows, uint64_t e, uint64_t pool_rows, int elem_bytes, hipStream_t s) {
    if (rows == 0 || e == 0) return;
    uint64_t row_bytes = e * (uint64_t)elem_bytes;
    if (row_bytes % 16 == 0)
        append_kernel<v4u><<<(unsigned)rows, 256, 0, s>>>((const v4u *)k_new, (const v4u *)v_new, (v4u *)k_pool,
                                                           (v4u *)v_pool, slots, row_bytes / 16, pool_rows);
    else if (row_bytes % 4 == 0)
        append_kernel<uint32_t><<<(unsigned)rows, 256, 0, s>>>((const uint32_t *)k_new, (const uint32_t *)v_new,
                                                                (uint32_t *)k_pool, (uint32_t *)v_pool, slots,
                                                                row_bytes / 4, pool_rows);
    else
        append_kernel<uint16_t><<<(unsigned)rows, 256, 0, s>>>((const uint16_t *)k_new, (const uint16_t *)v_new,
                                                                (uint16_t *)k_pool, (uint16_t *)v_pool, slots,
                                                                row_bytes / 2, pool_rows);
}

void paged_attention_generic(const void *q, const void *k_pool, const void *v_pool, const uint32_t *tables,
                             const uint32_t *seq_lens, const PagedShape &ps, int is_bf16, float *workspace,
                             uint64_t s_stride, void *out, hipStream_t s) {
    uint64_t rows = (uint64_t)ps.batch * ps.num_heads * ps.l_new;
    if (rows == 0) return;
    size_t smem = (size_t)ps.head_dim * sizeof(float);
    if (is_bf16)
        attention_generic_kernel<true><<<(unsigned)rows, 128, smem, s>>>(q, k_pool, v_pool, tables, seq_lens, ps,
                                                                         workspace, s_stride, out);
    else
        attention_generic_kernel<false><<<(unsigned)rows, 128, smem, s>>>(q, k_pool, v_pool, tables, seq_lens, ps,
                                                                          workspace, s_stride, out);
}

static uint32_t normalize_ppc(uint32_t ppc) { return ppc == 4 || ppc == 16 ? ppc : 8; }

uint64_t paged_decode_workspace_bytes(const PagedShape &ps, uint32_t pages_per_chunk) {
    uint32_t ppc = normalize_ppc(pages_per_chunk);
    uint32_t group = ps.num_heads / ps.num_kv_heads;
    uint64_t gp = (uint64_t)group_pad(group);
    uint64_t max_chunks = ((uint64_t)ps.max_blocks_per_seq + ppc - 1) / ppc;
    uint64_t items = (uint64_t)ps.batch * ps.num_kv_heads * max_chunks;
    return items * (gp * kDh + 2 * gp) * sizeof(float);
}

void paged_attention_decode_bf16(const uint16_t *q, const uint16_t *k_pool, const uint16_t *v_pool,
                                 const uint32_t *tables, const uint32_t *seq_lens, const PagedShape &ps,
                                 uint32_t pages_per_chunk, void *workspace, void *out, int out_bf16, hipStream_t s) {
    if (ps.batch == 0) return;
    uint32_t ppc = normalize_ppc(pages_per_chunk);
    DecodeParams p;
    p.q = q;
    p.k_pool = k_pool;
    p.v_pool = v_pool;
    p.tables = tables;
    p.seq_lens = seq_lens;
    p.num_blocks = ps.num_blocks;
    p.e_kv = ps.e_kv;
    p.batch = ps.batch;
    p.num_heads = ps.num_heads;
    p.num_kv_heads = ps.num_kv_heads;
    p.group = ps.num_heads / ps.num_kv_heads;
    p.max_blocks_per_seq = ps.max_blocks_per_seq;
    p.max_chunks = (ps.max_blocks_per_seq + ppc - 1) / ppc;
    p.scale = ps.scale;
    int gp = group_pad(p.group);
    uint64_t items = (uint64_t)ps.batch * ps.num_kv_heads * p.max_chunks;
    p.part_o = (float *)workspace;
    p.part_ml = p.part_o + items * (uint64_t)gp * kDh;
    switch (gp) {
        case 1: launch_decode_ppc<1>(p, ppc, out, out_bf16, s); break;
        case 2: launch_decode_ppc<2>(p, ppc, out, out_bf16, s); break;
        case 4: launch_decode_ppc<4>(p, ppc, out, out_bf16, s); break;
        default: launch_decode_ppc<8>(p, ppc, out, out_bf16, s); break;
    }
}

}  // namespace k
}  // namespace fa
