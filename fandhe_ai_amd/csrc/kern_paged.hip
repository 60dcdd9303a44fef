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
// four per block.  Both products run on the matrix cores and the K / V bytes
// are read once for the whole group of query heads:
//   1. S^T = K Q^T: the K slice of a page (16 tokens x 128 dims, 4 KiB) is
//      loaded straight into the A operand of v_mfma_f32_16x16x32_bf16 (lane
//      (g, r): token r, dims 32*s + 8*g .. +7 for step s); Q^T is the B operand
//      (column = query head of the group).  Lane (g, c) receives the scores of
//      tokens 4g .. 4g+3 for head c.
//   2. The scaled, masked scores of the whole chunk stay in registers; the
//      chunk maximum per head and the exponentials follow.
//   3. O^T = V^T P^T on v_mfma_f32_16x16x16_bf16: the weights of step 2 are
//      already in B-operand order (k = tokens 4g .. 4g+3, column = head); each
//      f32 weight is split exactly into three bf16 terms (hi + mid + lo) fed
//      to three instructions, so no precision is lost to the bf16 operand.  V^T needs four tokens of one dim per lane, so the
//      V page is staged through LDS (row pitch 272 B: conflict-free both for
//      the 16-byte row writes and for the 4-byte column reads) and every 4-byte
//      read, holding dims (d, d+1) of one token, serves an even / odd pair of
//      output rows after a byte permute.
// The chunk's unnormalized O, its maximum and its sum go to the workspace; a
// second kernel merges the chunks of a sequence.
constexpr int kDh = 128, kPage = 16;
constexpr int kVPitch = 136;            // bf16 elements per staged V row (272 B)

typedef short v4s __attribute__((ext_vector_type(4)));

struct DecodeParams {
    const uint16_t *q, *k_pool, *v_pool;
    const uint32_t *tables, *seq_lens;
    float *part_o;      // [items][g_pad][128]
    float *part_ml;     // [items][2][g_pad]
    uint32_t num_blocks, e_kv, batch, num_heads, num_kv_heads, group, g_pad, max_blocks_per_seq, max_chunks;
    float scale;
};

template <int PPC>
__global__ void __launch_bounds__(256) decode_chunk_kernel(DecodeParams p) {
    constexpr int KD = PPC < 4 ? PPC : 4;               // K pages in flight
    constexpr int VD = PPC < 2 ? PPC : 2;               // V pages in flight
    // one staging tile per wavefront: LDS operations of a wavefront execute in order, so the column
    // reads of page i are done before the row writes of page i + 1 land
    __shared__ __attribute__((aligned(16))) uint16_t v_s[4][kPage * kVPitch];
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int g = lane / 16, c = lane % 16;
    // Work list: item t = (sequence, chunk) pairs that exist, in sequence order, times the kv heads.
    // The wavefront finds its pair with a prefix sum over the chunk counts of the sequences (64 per
    // pass, one per lane).  Consecutive blocks hold consecutive items, so the hardware's round-robin
    // placement of blocks gives every XCD the same share of the bytes whatever the length distribution.
    const uint32_t item_id = blockIdx.x * 4 + wave;
    const uint32_t kvh = item_id % p.num_kv_heads, t = item_id / p.num_kv_heads;
    const uint32_t max_ctx = p.max_blocks_per_seq * kPage;
    uint32_t b = 0, chunk = 0, ctx = 0, base = 0;
    bool found = false, bad = false;
    for (uint32_t b0 = 0; b0 < p.batch && !found; b0 += 64) {
        uint32_t len = b0 + lane < p.batch ? p.seq_lens[b0 + lane] : 0;
        uint32_t len_c = len > max_ctx ? max_ctx : len;
        uint32_t nch = ((len_c + kPage - 1) / kPage + PPC - 1) / PPC;
        uint32_t incl = nch;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            uint32_t up = __shfl_up(incl, off, 64);
            if (lane >= off) incl += up;
        }
        bool hit = t >= base + incl - nch && t < base + incl;
        uint64_t mask = __ballot(hit);
        if (mask != 0) {
            int src = __builtin_ctzll(mask);
            b = b0 + src;
            chunk = t - (base + __shfl(incl - nch, src, 64));
            uint32_t len_src = __shfl(len, src, 64);
            bad = len_src > max_ctx;
            ctx = bad ? max_ctx : len_src;
            found = true;
        }
        base += __shfl(incl, 63, 64);
    }
    if (!found) return;
    b = __builtin_amdgcn_readfirstlane(b);
    chunk = __builtin_amdgcn_readfirstlane(chunk);
    ctx = __builtin_amdgcn_readfirstlane(ctx);
    const uint32_t p0 = chunk * PPC;
    const uint32_t *tab = p.tables + (uint64_t)b * p.max_blocks_per_seq + p0;
    uint32_t raw[PPC];
#pragma unroll
    for (int i = 0; i < PPC; ++i) raw[i] = p0 + i < p.max_blocks_per_seq ? tab[i] : 0xffffffffu;

    // Q^T operand: column c = head of the group (zero beyond the group)
    v8bf qb[4];
    {
        const uint32_t hc = (uint32_t)c < p.group ? (uint32_t)c : 0;
        const uint16_t *qrow = p.q + ((uint64_t)b * p.num_heads + (uint64_t)kvh * p.group + hc) * kDh + 8 * g;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            v4u t = *(const v4u *)(qrow + 32 * s);
            if ((uint32_t)c >= p.group) t = v4u{0, 0, 0, 0};
            qb[s] = __builtin_bit_cast(v8bf, t);
        }
    }

    const uint32_t n_pages = (ctx + kPage - 1) / kPage;
    const uint32_t np = n_pages - p0 < (uint32_t)PPC ? n_pages - p0 : (uint32_t)PPC;
    // positions past the end repeat the last page (their scores are masked): loads stay unconditional
    uint32_t ids[PPC];
    {
        uint32_t cur = 0;
#pragma unroll
        for (int i = 0; i < PPC; ++i) {
            if ((uint32_t)i < np) {
                cur = raw[i];
                if (cur >= p.num_blocks) {
                    bad = true;
                    cur = 0;
                }
            }
            ids[i] = cur;
        }
    }

    const uint64_t page_elems = (uint64_t)kPage * p.e_kv;
    const uint64_t k_lane = (uint64_t)c * p.e_kv + (uint64_t)kvh * kDh + 8 * g;       // token c, dims 8g..
    const uint64_t v_lane = (uint64_t)(4 * g) * p.e_kv + (uint64_t)kvh * kDh + 8 * c;  // tokens 4g.., dims 8c..

    auto load_k = [&](int i, v4u *dst) {
        const uint16_t *base = p.k_pool + (uint64_t)ids[i] * page_elems + k_lane;
#pragma unroll
        for (int s = 0; s < 4; ++s) dst[s] = *(const v4u *)(base + 32 * s);
    };
    auto load_v = [&](int i, v4u *dst) {
        const uint16_t *base = p.v_pool + (uint64_t)ids[i] * page_elems + v_lane;
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[j] = *(const v4u *)(base + (uint64_t)j * p.e_kv);
    };

    // ---- pass 1: scores
    v4u kreg[KD][4];
#pragma unroll
    for (int i = 0; i < KD; ++i) load_k(i, kreg[i]);
    float sc[PPC][4];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < PPC; ++i) {
        v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; ++s)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, kreg[i % KD][s]), qb[s], acc, 0, 0, 0);
        if (i + KD < PPC) load_k(i + KD, kreg[i % KD]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t tok = (p0 + i) * kPage + 4 * g + j;
            float s = (uint32_t)i < np && tok < ctx ? acc[j] * p.scale : -INFINITY;
            sc[i][j] = s;
            mx = fmaxf(mx, s);
        }
    }
    // the first V pages are requested before the softmax arithmetic
    v4u vreg[VD][4];
#pragma unroll
    for (int i = 0; i < VD; ++i) load_v(i, vreg[i]);

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

    // ---- pass 2: O^T[d][head] += V^T[d][token] * P^T[token][head]
    // acc index 2*bp + e covers dims 32*bp + 2*(4g + j) + e, j = 0..3, in lane (g, c)
    v4f o[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) o[t] = v4f{0.f, 0.f, 0.f, 0.f};
    uint16_t *vs = &v_s[wave][0];
#pragma unroll
    for (int i = 0; i < PPC; ++i) {
        // stage the page: lane (g, c) owns tokens 4g + j, dims 8c .. 8c + 7
        // rows of tokens at or past the sequence end are staged as zeros: their weights are zero, but the
        // pool may hold anything there and 0 * NaN must not reach the accumulators
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t tok = (p0 + i) * kPage + 4 * g + j;
            v4u row = (uint32_t)i < np && tok < ctx ? vreg[i % VD][j] : v4u{0, 0, 0, 0};
            *(v4u *)(vs + (4 * g + j) * kVPitch + 8 * c) = row;
        }
        if (i + VD < PPC) load_v(i + VD, vreg[i % VD]);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // each f32 weight as three bf16 operands by repeated truncation: hi + mid + lo == p exactly
        // (3 x 8 significant bits), so the only rounding left is the f32 accumulation
        uint32_t hi[4], mid[4], lo[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float pj = sc[i][j];
            hi[j] = __float_as_uint(pj) & 0xffff0000u;
            float r1 = pj - __uint_as_float(hi[j]);
            mid[j] = __float_as_uint(r1) & 0xffff0000u;
            lo[j] = __float_as_uint(r1 - __uint_as_float(mid[j]));
        }
        v2u ph = v2u{__builtin_amdgcn_perm(hi[1], hi[0], 0x07060302u), __builtin_amdgcn_perm(hi[3], hi[2], 0x07060302u)};
        v2u pm = v2u{__builtin_amdgcn_perm(mid[1], mid[0], 0x07060302u), __builtin_amdgcn_perm(mid[3], mid[2], 0x07060302u)};
        v2u pl = v2u{__builtin_amdgcn_perm(lo[1], lo[0], 0x07060302u), __builtin_amdgcn_perm(lo[3], lo[2], 0x07060302u)};
        v4s b_hi = __builtin_bit_cast(v4s, ph), b_mid = __builtin_bit_cast(v4s, pm), b_lo = __builtin_bit_cast(v4s, pl);
#pragma unroll
        for (int bp = 0; bp < 4; ++bp) {
            // dims (32 bp + 2c, +1) of tokens 4g .. 4g + 3
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = *(const uint32_t *)(vs + (4 * g + j) * kVPitch + 32 * bp + 2 * c);
            v2u ae = v2u{__builtin_amdgcn_perm(w[1], w[0], 0x05040100u), __builtin_amdgcn_perm(w[3], w[2], 0x05040100u)};
            v2u ao = v2u{__builtin_amdgcn_perm(w[1], w[0], 0x07060302u), __builtin_amdgcn_perm(w[3], w[2], 0x07060302u)};
            v4s a_even = __builtin_bit_cast(v4s, ae), a_odd = __builtin_bit_cast(v4s, ao);
            // smallest terms first
            o[2 * bp] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_even, b_lo, o[2 * bp], 0, 0, 0);
            o[2 * bp + 1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_odd, b_lo, o[2 * bp + 1], 0, 0, 0);
            o[2 * bp] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_even, b_mid, o[2 * bp], 0, 0, 0);
            o[2 * bp + 1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_odd, b_mid, o[2 * bp + 1], 0, 0, 0);
            o[2 * bp] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_even, b_hi, o[2 * bp], 0, 0, 0);
            o[2 * bp + 1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_odd, b_hi, o[2 * bp + 1], 0, 0, 0);
        }
    }
    // lane (g, c) holds, for head c: dims 32 bp + 8 g + {0..7} = {o[2bp][0], o[2bp+1][0], o[2bp][1], ...}
    const uint64_t item = ((uint64_t)b * p.num_kv_heads + kvh) * p.max_chunks + chunk;
    if ((uint32_t)c < p.group) {
        float *po = p.part_o + (item * p.g_pad + c) * kDh + 8 * g;
#pragma unroll
        for (int bp = 0; bp < 4; ++bp) {
            *(v4f *)(po + 32 * bp) = v4f{o[2 * bp][0], o[2 * bp + 1][0], o[2 * bp][1], o[2 * bp + 1][1]};
            *(v4f *)(po + 32 * bp + 4) = v4f{o[2 * bp][2], o[2 * bp + 1][2], o[2 * bp][3], o[2 * bp + 1][3]};
        }
        if (g == 0) {
            float nanv = __uint_as_float(0x7fc00000u);
            p.part_ml[item * (2 * p.g_pad) + c] = bad ? nanv : mx;
            p.part_ml[item * (2 * p.g_pad) + p.g_pad + c] = bad ? nanv : lsum;
        }
    }
}

// Merges the chunks of one (sequence, query head).  Block = 256 threads: thread
// (part, d) sums every second chunk for dim d, then the two parts are added.
template <int PPC>
__global__ void __launch_bounds__(256) decode_merge_kernel(DecodeParams p, void *__restrict__ out, int out_bf16,
                                                          float *__restrict__ pmax) {
    __shared__ float s_acc[128], s_den, s_max[2];
    const uint32_t h = blockIdx.x, b = blockIdx.y, d = threadIdx.x % 128, part = threadIdx.x / 128;
    const uint32_t kvh = h / p.group, hg = h % p.group;
    uint32_t ctx = p.seq_lens[b];
    uint32_t max_ctx = p.max_blocks_per_seq * kPage;
    if (ctx > max_ctx) ctx = max_ctx;
    const uint32_t n_pages = (ctx + kPage - 1) / kPage;
    const uint32_t n_chunks = (n_pages + PPC - 1) / PPC;
    const uint64_t item0 = ((uint64_t)b * p.num_kv_heads + kvh) * p.max_chunks;
    const float *ml = p.part_ml + item0 * (2 * p.g_pad) + hg;
    float mx = -INFINITY;
    for (uint32_t ch = 0; ch < n_chunks; ++ch) {
        float m = ml[(uint64_t)ch * (2 * p.g_pad)];
        mx = (m != m || mx != mx) ? __uint_as_float(0x7fc00000u) : fmaxf(mx, m);   // NaN marks a violation
    }
    float acc = 0.0f, den = 0.0f;
    const float *po = p.part_o + (item0 * p.g_pad + hg) * kDh + d;
    for (uint32_t ch = part; ch < n_chunks; ch += 2) {
        float m = ml[(uint64_t)ch * (2 * p.g_pad)];
        float l = ml[(uint64_t)ch * (2 * p.g_pad) + p.g_pad];
        float w = expf(m - mx);
        den = __builtin_fmaf(w, l, den);
        acc = __builtin_fmaf(w, po[(uint64_t)ch * p.g_pad * kDh], acc);
    }
    if (part == 1) {
        s_acc[d] = acc;
        if (d == 0) s_den = den;
    }
    __syncthreads();
    float a = 0.0f;
    if (part == 0) {
        acc += s_acc[d];
        den += s_den;
        float r = n_chunks == 0 ? 0.0f : __fdiv_rn(acc, den);
        uint64_t o = ((uint64_t)b * p.num_heads + h) * kDh + d;
        if (out_bf16) {
            uint16_t rb = f32_to_bf16(r);
            ((uint16_t *)out)[o] = rb;
            r = bf16_to_f32(rb);
        } else {
            ((float *)out)[o] = r;
        }
        a = fabsf(r);
    }
    if (pmax) {                      // absmax of the stored head slice, for the quantizer that follows
        a = wave_max(a);
        if (part == 0 && threadIdx.x % 64 == 0) s_max[threadIdx.x / 64] = a;
        __syncthreads();
        if (threadIdx.x == 0) pmax[(uint64_t)b * p.num_heads + h] = fmaxf(s_max[0], s_max[1]);
    }
}

inline int group_pad(uint32_t group) {
    int gp = 1;
    while ((uint32_t)gp < group) gp *= 2;
    return gp;
}

template <int PPC>
void launch_decode(const DecodeParams &p, void *out, int out_bf16, float *pmax, hipStream_t s) {
    // upper bound of the work list; wavefronts past its real end exit at once
    uint64_t items = (uint64_t)p.batch * p.num_kv_heads * p.max_chunks;
    decode_chunk_kernel<PPC><<<(unsigned)((items + 3) / 4), 256, 0, s>>>(p);
    dim3 grid2(p.num_heads, p.batch);
    decode_merge_kernel<PPC><<<grid2, 256, 0, s>>>(p, out, out_bf16, pmax);
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
                                 uint32_t pages_per_chunk, void *workspace, void *out, int out_bf16, float *pmax,
                                 hipStream_t s) {
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
    p.g_pad = (uint32_t)gp;
    uint64_t items = (uint64_t)ps.batch * ps.num_kv_heads * p.max_chunks;
    p.part_o = (float *)workspace;
    p.part_ml = p.part_o + items * (uint64_t)gp * kDh;
    switch (ppc) {
        case 4: launch_decode<4>(p, out, out_bf16, pmax, s); break;
        case 16: launch_decode<16>(p, out, out_bf16, pmax, s); break;
        default: launch_decode<8>(p, out, out_bf16, pmax, s); break;
    }
}

}  // namespace k
}  // namespace fa
