// Paged KV cache kernels: row scatter (append), a generic attention kernel
// that keeps the reference's per-row summation order, and the decode fast
// path (bf16, head_dim 128, 16-token pages, one query token, grouped-query).
#include "device_utils.hpp"
#include "index_models.hpp"
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
// Both products of the decode attention run on the matrix cores and the K / V
// bytes are read once for the whole group of query heads:
//   1. S^T = K Q^T: the K slice of a page (16 tokens x 128 dims, 4 KiB) is
//      loaded straight into the A operand of v_mfma_f32_16x16x32_bf16 (lane
//      (g, r): token r, dims 32*s + 8*g .. +7 for step s); Q^T is the B operand
//      (column = query head of the group).  Lane (g, c) receives the scores of
//      tokens 4g .. 4g+3 for head c.
//   2. O^T = V^T P^T on v_mfma_f32_16x16x16_bf16: the softmax weights are
//      already in B-operand order (k = tokens 4g .. 4g+3, column = head); each
//      f32 weight is split exactly into three bf16 terms (hi + mid + lo) fed
//      to three instructions, so no precision is lost to the bf16 operand.
//      V^T needs four tokens of one dim per lane, so the V page is staged
//      through LDS (row pitch 272 B: conflict-free both for the 16-byte row
//      writes and for the 4-byte column reads) and every 4-byte read, holding
//      dims (d, d+1) of one token, serves an even / odd pair of output rows
//      after a byte permute.
constexpr int kDh = 128, kPage = 16;
constexpr int kVPitch = 136;            // bf16 elements per staged V row (272 B)

typedef short v4s __attribute__((ext_vector_type(4)));

// The pages of all sequences, laid end to end, are cut into n_ranges equal
// ranges; range r goes to one wavefront per kv head, and the launch is sized so
// that every wavefront is resident at once and all of them carry the same number
// of pages whatever the length distribution.  A range that crosses a sequence
// boundary yields one partial result per sequence it touches; partial (r, b)
// lives in slot r + b, which is unique because r and b never decrease along
// the page axis and one of them grows from one partial to the next.
// Inside a segment the wavefront walks groups of SP pages with a running
// maximum / sum (the accumulators are rescaled when the maximum grows), and the
// K and V loads of later pages are always in flight while a group is being
// multiplied, so the memory pipe never drains between the two products.
struct StreamParams {
    const uint16_t *q, *k_pool, *v_pool;
    const uint32_t *tables, *seq_lens;
    float *part_o;      // [slots * num_kv_heads][g_pad][128]
    float *part_ml;     // [slots * num_kv_heads][2][g_pad]
    uint32_t num_blocks, e_kv, batch, num_heads, num_kv_heads, group, g_pad, max_blocks_per_seq;
    uint32_t n_ranges, min_pages;
    float scale;
    // Prefill (l_new > 1): the 16 columns of the score tile are tpt = 16 / group consecutive new tokens x
    // the heads of the group (column = token-in-tile * group + head), and every such token tile of a
    // sequence is streamed as a sequence of its own ("virtual sequence" b * qt + tile) whose length is the
    // causal limit of its last token; columns are masked individually at their own limit.  A wavefront
    // carries TT token tiles at once (tpv = TT * tpt tokens per virtual sequence), so K / V are read once
    // per tpv new tokens.  One launch covers the new tokens [t0, t0 + qt * tpv) of every sequence.
    // Decode: l_new = tpt = tpv = qt = 1, t0 = 0.
    uint32_t l_new, tpt, tpv, qt, t0, n_vseq;
    // ONE form only (decode_stream_kernel<..., ONE = true>): the finished attention output, f32 values already rounded
    // to bf16 (the operator's output type), [batch][num_heads][128], and the absmax of every head's slice
    float *one_out = nullptr, *one_pmax = nullptr;
};

// Length of (virtual) sequence vs: all cached positions up to the last new token of its tile.  A row whose
// length is below l_new (possible only with unvalidated device tables) streams nothing.
template <bool PF>
__device__ __forceinline__ uint32_t vseq_len(const StreamParams &p, uint32_t vs) {
    if constexpr (!PF) {
        return p.seq_lens[vs];
    } else {
        const uint32_t len = p.seq_lens[vs / p.qt];
        if (len < p.l_new) return 0;
        uint32_t after = p.t0 + (vs % p.qt + 1) * p.tpv;
        if (after > p.l_new) after = p.l_new;
        return len - p.l_new + after;
    }
}
template <bool PF>
__device__ __forceinline__ uint32_t seq_pages(const StreamParams &p, uint32_t vs, uint32_t max_ctx) {
    uint32_t len = vseq_len<PF>(p, vs);
    if (len > max_ctx) len = max_ctx;
    return (len + kPage - 1) / kPage;
}

// pages per range for this launch: the same value in every wavefront of both kernels
__device__ __forceinline__ uint32_t range_pages(const StreamParams &p, uint32_t total) {
    return ixm::stream_range_pages(total, p.n_ranges, p.min_pages);
}

// ONE (decode only): one block per (sequence, kv head) instead of one wavefront per (range, kv head).  The four
// wavefronts of the block take a quarter of the sequence's pages each, their results meet in LDS, and the first
// wavefront normalises and stores the finished output (p.one_out, p.one_pmax): no partial results in memory, no
// merge launch.  For a few short sequences (a compute unit per kv head streams a whole sequence); the arithmetic of
// the meeting is that of the merge kernels.
template <int SP, int KD, int VD, int WPE, bool PF, int TT = 1, bool ONE = false>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) decode_stream_kernel(StreamParams p) {
    static_assert(PF || TT == 1, "several token tiles per wavefront exist only in the prefill form");
    static_assert(!ONE || !PF, "the one-block form is a decode form");
    static_assert(SP % KD == 0 && SP % VD == 0, "static register indices need SP to be a multiple of the depths");
    __shared__ __attribute__((aligned(16))) uint16_t v_s[4][kPage * kVPitch];
    __shared__ float one_o[ONE ? 4 : 1][ONE ? 64 : 1][ONE ? 33 : 1];       // [wavefront][lane][its 32 dims], padded
    __shared__ float one_ml[ONE ? 4 : 1][2][16], one_amax[ONE ? 4 : 1][16];
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int g = lane / 16, c = lane % 16;
    const uint32_t item_id = ONE ? blockIdx.x : blockIdx.x * 4 + wave;
    const uint32_t kvh = item_id % p.num_kv_heads, r = item_id / p.num_kv_heads;   // ONE: r is the sequence
    if (r >= (ONE ? p.batch : p.n_ranges)) return;
    const uint32_t max_ctx = p.max_blocks_per_seq * kPage;
    const uint32_t nv = PF ? p.n_vseq : p.batch;
    uint32_t rlo = 0, rhi = 0;
    if constexpr (!ONE) {
        uint32_t total = 0;
        for (uint32_t b = lane; b < nv; b += 64) total += seq_pages<PF>(p, b, max_ctx);
        total = __builtin_amdgcn_readfirstlane(wave_sum_dpp<uint32_t>(total));
        const uint32_t per = range_pages(p, total);
        const uint64_t rlo64 = (uint64_t)r * per;
        if (rlo64 >= total) return;
        rlo = (uint32_t)rlo64;
        rhi = rlo + per < total ? rlo + per : total;
    }

    const uint64_t page_elems = (uint64_t)kPage * p.e_kv;
    const uint64_t k_lane = (uint64_t)c * p.e_kv + (uint64_t)kvh * kDh + 8 * g;       // token c, dims 8g..
    const uint64_t v_lane = (uint64_t)(4 * g) * p.e_kv + (uint64_t)kvh * kDh + 8 * c;  // tokens 4g.., dims 8c..
    uint16_t *vs = &v_s[wave][0];

    // pages [lo, hi) (hi > lo) of (virtual) sequence vq, whose length is len_b
    auto segment = [&](const uint32_t vq, const uint32_t lo, const uint32_t hi, const uint32_t len_b) {
            const uint32_t b = PF ? vq / p.qt : vq;
            bool bad = len_b > max_ctx;
            if constexpr (PF) bad = p.seq_lens[b] > max_ctx;
            const uint32_t ctx = len_b > max_ctx ? max_ctx : len_b;
            const uint32_t n = hi - lo;                                // pages of this segment (>= 1)
            const uint32_t *tab = p.tables + (uint64_t)b * p.max_blocks_per_seq + lo;

            // Q^T operand: column c = head of the group (zero beyond the group); prefill: column c = new
            // token c / group of the tile, head c % group, masked at that token's own causal limit
            v8bf qb[TT][4];
            uint32_t ctx_l[TT];                                        // this lane's column sees tokens below ctx_l
            if constexpr (!PF) {
                ctx_l[0] = ctx;
                const uint32_t hc = (uint32_t)c < p.group ? (uint32_t)c : 0;
                const uint16_t *qrow = p.q + ((uint64_t)b * p.num_heads + (uint64_t)kvh * p.group + hc) * kDh + 8 * g;
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    v4u t = *(const v4u *)(qrow + 32 * s);
                    if ((uint32_t)c >= p.group) t = v4u{0, 0, 0, 0};
                    qb[0][s] = __builtin_bit_cast(v8bf, t);
                }
            } else {
                const uint32_t tl = (uint32_t)c / p.group, hc = (uint32_t)c % p.group;
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) {
                    const uint32_t t = p.t0 + (vq % p.qt) * p.tpv + tt * p.tpt + tl;
                    const bool valid = tl < p.tpt && t < p.l_new;
                    const uint32_t tc = valid ? t : 0;
                    const uint16_t *qrow =
                        p.q + (((uint64_t)b * p.l_new + tc) * p.num_heads + (uint64_t)kvh * p.group + hc) * kDh + 8 * g;
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        v4u t4 = *(const v4u *)(qrow + 32 * s);
                        if (!valid) t4 = v4u{0, 0, 0, 0};
                        qb[tt][s] = __builtin_bit_cast(v8bf, t4);
                    }
                    // cached positions before the new tokens + new tokens up to and including t; never above
                    // ctx, which is already clamped to what the table can describe
                    const uint32_t lim = p.seq_lens[b] - p.l_new + t + 1;
                    ctx_l[tt] = valid && lim < ctx ? lim : ctx;
                }
            }
            // Block ids of 64 pages at a time, one per lane (idv), with the following 64 (idv_next) already
            // resident.  Everything below is straight-line code per group: loads past the end of the
            // segment repeat its last page and their scores are masked, and the id windows advance by
            // selects, so the compiler can count outstanding loads exactly and never drains them at a join.
            auto tab_at = [&](uint32_t i) -> uint32_t { return tab[i < n ? i : n - 1]; };
            uint32_t idv = tab_at(lane), idv_next = tab_at(64 + lane);
            if (__ballot((uint32_t)lane < n && idv >= p.num_blocks) != 0) bad = true;
            if (idv >= p.num_blocks) idv = 0;
            uint32_t win = 0;                                          // first page of the id window
            auto page_id = [&](uint32_t i) -> uint32_t {               // i uniform, win <= i < win + 128
                const uint32_t ic = i < n ? i : n - 1, rel = ic - win;
                const uint32_t a = __builtin_amdgcn_readlane(idv, (int)(rel & 63));
                const uint32_t bnext = __builtin_amdgcn_readlane(idv_next, (int)(rel & 63));
                uint32_t id = rel < 64 ? a : bnext;
                return id < p.num_blocks ? id : 0;                     // ids of the next window are checked on use too
            };
            auto load_k = [&](uint32_t i, v4u *dst) {
                const uint16_t *src_p = p.k_pool + (uint64_t)page_id(i) * page_elems + k_lane;
#pragma unroll
                for (int s = 0; s < 4; ++s) dst[s] = stream_load<!PF>((const v4u *)(src_p + 32 * s));
            };
            auto load_v = [&](uint32_t i, v4u *dst) {
                const uint16_t *src_p = p.v_pool + (uint64_t)page_id(i) * page_elems + v_lane;
#pragma unroll
                for (int j = 0; j < 4; ++j) dst[j] = stream_load<!PF>((const v4u *)(src_p + (uint64_t)j * p.e_kv));
            };

            // the first requests go out in the order the loop consumes them (oldest first), so that the wait
            // counts at the loop head are as loose on the first pass as on the later ones
            v4u kreg[KD][4], vreg[VD][4];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < KD; ++i) {
                load_k(i, kreg[i]);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < VD; ++i) {
                load_v(i, vreg[i]);
                __builtin_amdgcn_sched_barrier(0);
            }

            float m_run[TT], l_run[TT];
            v4f o[TT][8];
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
                m_run[tt] = -INFINITY;
                l_run[tt] = 0.0f;
#pragma unroll
                for (int t = 0; t < 8; ++t) o[tt][t] = v4f{0.f, 0.f, 0.f, 0.f};
            }

            // 64 is a multiple of SP, so a group never straddles two id windows; the loads issued from a
            // group reach at most max(KD, VD) <= SP pages past it, i.e. at most into the next window
            for (uint32_t p0 = 0; p0 < n; p0 += SP) {
                // ids two windows ahead, requested before this group's K / V loads so that consuming
                // them at the end of the group waits for nothing younger than the loads of the last group
                const uint32_t cand = tab_at(win + 128 + lane);
                __builtin_amdgcn_sched_barrier(0);
                // ---- scores of the group
                float sc[TT][SP][4];
                float mx[TT];
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) mx[tt] = -INFINITY;
#pragma unroll
                for (int i = 0; i < SP; ++i) {
                    const uint32_t pg = p0 + i;
                    v4f acc[TT];
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt) {
                        acc[tt] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int s = 0; s < 4; ++s)
                            acc[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, kreg[i % KD][s]),
                                                                              qb[tt][s], acc[tt], 0, 0, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);                 // keep the request right behind its consumer
                    load_k(pg + KD, kreg[i % KD]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            uint32_t tok = (lo + pg) * kPage + 4 * g + j;
                            float s = pg < n && tok < ctx_l[tt] ? acc[tt][j] * p.scale : -INFINITY;
                            sc[tt][i][j] = s;
                            mx[tt] = fmaxf(mx[tt], s);
                        }
                }
                // ---- running maximum and sum per column (lanes with equal c hold one column)
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) {
                    float m = mx[tt];
                    m = fmaxf(m, __shfl_xor(m, 16, 64));
                    m = fmaxf(m, __shfl_xor(m, 32, 64));
                    const float m_new = fmaxf(m_run[tt], m);
                    // prefill: a column can have every score of a segment masked (the segment lies past its
                    // causal limit); its maximum stays -inf and the exponentials are taken against 0 instead
                    const float m_use = (PF && m_new == -INFINITY) ? 0.0f : m_new;
                    const float alpha = expf(m_run[tt] - m_use);       // first group: exp(-inf) = 0
                    m_run[tt] = m_new;
                    float gsum = 0.0f;
#pragma unroll
                    for (int i = 0; i < SP; ++i)
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            float e = expf(sc[tt][i][j] - m_use);      // masked scores: exp(-inf) = 0
                            sc[tt][i][j] = e;
                            gsum += e;
                        }
                    l_run[tt] = __builtin_fmaf(l_run[tt], alpha, gsum);
#pragma unroll
                    for (int t = 0; t < 8; ++t) o[tt][t] = o[tt][t] * alpha;
                }
                // ---- O^T += V^T P^T
#pragma unroll
                for (int i = 0; i < SP; ++i) {
                    const uint32_t pg = p0 + i;
                    // rows of tokens at or past the sequence end are staged as zeros: their weights are zero,
                    // but the pool may hold anything there and 0 * NaN must not reach the accumulators
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        uint32_t tok = (lo + pg) * kPage + 4 * g + j;
                        v4u row = pg < n && tok < ctx ? vreg[i % VD][j] : v4u{0, 0, 0, 0};
                        *(v4u *)(vs + (4 * g + j) * kVPitch + 8 * c) = row;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    load_v(pg + VD, vreg[i % VD]);
                    __builtin_amdgcn_sched_barrier(0);
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    // each f32 weight as three bf16 operands by repeated truncation: hi + mid + lo == p exactly
                    v4s b_hi[TT], b_mid[TT], b_lo[TT];
#pragma unroll
                    for (int tt = 0; tt < TT; ++tt) {
                        uint32_t whi[4], wmid[4], wlo[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            float pj = sc[tt][i][j];
                            whi[j] = __float_as_uint(pj) & 0xffff0000u;
                            float r1 = pj - __uint_as_float(whi[j]);
                            wmid[j] = __float_as_uint(r1) & 0xffff0000u;
                            wlo[j] = __float_as_uint(r1 - __uint_as_float(wmid[j]));
                        }
                        v2u ph = v2u{__builtin_amdgcn_perm(whi[1], whi[0], 0x07060302u), __builtin_amdgcn_perm(whi[3], whi[2], 0x07060302u)};
                        v2u pm = v2u{__builtin_amdgcn_perm(wmid[1], wmid[0], 0x07060302u), __builtin_amdgcn_perm(wmid[3], wmid[2], 0x07060302u)};
                        v2u pl = v2u{__builtin_amdgcn_perm(wlo[1], wlo[0], 0x07060302u), __builtin_amdgcn_perm(wlo[3], wlo[2], 0x07060302u)};
                        b_hi[tt] = __builtin_bit_cast(v4s, ph);
                        b_mid[tt] = __builtin_bit_cast(v4s, pm);
                        b_lo[tt] = __builtin_bit_cast(v4s, pl);
                    }
#pragma unroll
                    for (int bp = 0; bp < 4; ++bp) {
                        uint32_t w[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) w[j] = *(const uint32_t *)(vs + (4 * g + j) * kVPitch + 32 * bp + 2 * c);
                        v2u ae = v2u{__builtin_amdgcn_perm(w[1], w[0], 0x05040100u), __builtin_amdgcn_perm(w[3], w[2], 0x05040100u)};
                        v2u ao = v2u{__builtin_amdgcn_perm(w[1], w[0], 0x07060302u), __builtin_amdgcn_perm(w[3], w[2], 0x07060302u)};
                        v4s a_even = __builtin_bit_cast(v4s, ae), a_odd = __builtin_bit_cast(v4s, ao);
#pragma unroll
                        for (int tt = 0; tt < TT; ++tt) {
                            // smallest terms first
                            o[tt][2 * bp] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_even, b_lo[tt], o[tt][2 * bp], 0, 0, 0);
                            o[tt][2 * bp + 1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_odd, b_lo[tt], o[tt][2 * bp + 1], 0, 0, 0);
                            o[tt][2 * bp] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_even, b_mid[tt], o[tt][2 * bp], 0, 0, 0);
                            o[tt][2 * bp + 1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_odd, b_mid[tt], o[tt][2 * bp + 1], 0, 0, 0);
                            o[tt][2 * bp] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_even, b_hi[tt], o[tt][2 * bp], 0, 0, 0);
                            o[tt][2 * bp + 1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a_odd, b_hi[tt], o[tt][2 * bp + 1], 0, 0, 0);
                        }
                    }
                }
                // advance the id windows when the next group starts a new one
                const bool adv = p0 + SP >= win + 64;
                if (adv && __ballot(win + 64 + lane < n && idv_next >= p.num_blocks) != 0) bad = true;
                idv = adv ? idv_next : idv;
                idv_next = adv ? cand : idv_next;
                win = adv ? win + 64 : win;
            }
            // lane (g, c) holds, for column c: dims 32 bp + 8 g + {0..7} = {o[2bp][0], o[2bp+1][0], o[2bp][1], ...}
            if constexpr (ONE) {
                float l = l_run[0];
                l += __shfl_xor(l, 16, 64);
                l += __shfl_xor(l, 32, 64);
#pragma unroll
                for (int bp = 0; bp < 4; ++bp) {
                    float *d = &one_o[wave][lane][8 * bp];
                    d[0] = o[0][2 * bp][0], d[1] = o[0][2 * bp + 1][0], d[2] = o[0][2 * bp][1], d[3] = o[0][2 * bp + 1][1];
                    d[4] = o[0][2 * bp][2], d[5] = o[0][2 * bp + 1][2], d[6] = o[0][2 * bp][3], d[7] = o[0][2 * bp + 1][3];
                }
                if (g == 0) {
                    const float nanv = __uint_as_float(0x7fc00000u);
                    one_ml[wave][0][c] = bad ? nanv : m_run[0];
                    one_ml[wave][1][c] = bad ? nanv : l;
                }
                return;
            }
            const uint64_t item = (uint64_t)(r + vq) * p.num_kv_heads + kvh;
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
                float l = l_run[tt];
                l += __shfl_xor(l, 16, 64);
                l += __shfl_xor(l, 32, 64);
                if ((uint32_t)c < (PF ? p.tpt * p.group : p.group)) {
                    float *po = p.part_o + ((item * TT + tt) * p.g_pad + c) * kDh + 8 * g;
#pragma unroll
                    for (int bp = 0; bp < 4; ++bp) {
                        *(v4f *)(po + 32 * bp) = v4f{o[tt][2 * bp][0], o[tt][2 * bp + 1][0], o[tt][2 * bp][1], o[tt][2 * bp + 1][1]};
                        *(v4f *)(po + 32 * bp + 4) = v4f{o[tt][2 * bp][2], o[tt][2 * bp + 1][2], o[tt][2 * bp][3], o[tt][2 * bp + 1][3]};
                    }
                    if (g == 0) {
                        float nanv = __uint_as_float(0x7fc00000u);
                        p.part_ml[(item * TT + tt) * (2 * p.g_pad) + c] = bad ? nanv : m_run[tt];
                        p.part_ml[(item * TT + tt) * (2 * p.g_pad) + p.g_pad + c] = bad ? nanv : l;
                    }
                }
            }
    };
    if constexpr (ONE) {
        const uint32_t len_b = p.seq_lens[r];
        const uint32_t len_c = len_b > max_ctx ? max_ctx : len_b;
        const uint32_t npg = (len_c + kPage - 1) / kPage;
        const uint32_t lo = (uint32_t)((uint64_t)npg * (uint32_t)wave / 4), hi = (uint32_t)((uint64_t)npg * ((uint32_t)wave + 1) / 4);
        if (hi > lo) {
            segment(r, lo, hi, len_b);
        } else {                                                       // no pages for this wavefront: weight zero
#pragma unroll
            for (int j = 0; j < 32; ++j) one_o[wave][lane][j] = 0.0f;
            if (g == 0) {
                one_ml[wave][0][c] = -INFINITY;
                one_ml[wave][1][c] = 0.0f;
            }
        }
        __syncthreads();
        // the meeting, as decode_stream_merge_quantize_kernel does it: maximum (NaN marks a violation), weights,
        // weighted sums in wavefront order, one division, one rounding to bf16; wavefront w finishes dims
        // 32 w + 8 g .. + 7 of every column
        float mx = -INFINITY, den = 0.0f, acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float m = one_ml[w][0][c];
            mx = (m != m || mx != mx) ? __uint_as_float(0x7fc00000u) : fmaxf(mx, m);
        }
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float wt = expf(one_ml[w][0][c] - mx);
            den = __builtin_fmaf(wt, one_ml[w][1][c], den);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(wt, one_o[w][lane][8 * wave + e], acc[e]);
        }
        float amax = 0.0f, v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float res = npg == 0 ? 0.0f : __fdiv_rn(acc[e], den);
            v[e] = bf16_to_f32(f32_to_bf16(res));
            amax = fmaxf(amax, fabsf(v[e]));
        }
        if ((uint32_t)c < p.group) {
            float *dst = p.one_out + ((uint64_t)r * p.num_heads + (uint64_t)kvh * p.group + c) * kDh + 32 * wave + 8 * g;
            *(v4f *)dst = v4f{v[0], v[1], v[2], v[3]};
            *(v4f *)(dst + 4) = v4f{v[4], v[5], v[6], v[7]};
        }
        amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        if (g == 0) one_amax[wave][c] = amax;
        __syncthreads();
        if (wave == 0 && g == 0 && (uint32_t)c < p.group)
            p.one_pmax[(uint64_t)r * p.num_heads + (uint64_t)kvh * p.group + c] =
                fmaxf(fmaxf(one_amax[0][c], one_amax[1][c]), fmaxf(one_amax[2][c], one_amax[3][c]));
    } else {
        uint32_t base = 0;
        for (uint32_t b0 = 0; b0 < nv; b0 += 64) {
            uint32_t len = b0 + lane < nv ? vseq_len<PF>(p, b0 + lane) : 0;
            uint32_t len_c = len > max_ctx ? max_ctx : len;
            uint32_t npg = (len_c + kPage - 1) / kPage;
            uint32_t incl = npg;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                uint32_t up = __shfl_up(incl, off, 64);
                if (lane >= off) incl += up;
            }
            const uint32_t s_b = base + incl - npg, e_b = base + incl;
            uint64_t mask = __ballot(npg != 0 && s_b < rhi && e_b > rlo);
            base += __shfl(incl, 63, 64);
            while (mask != 0) {
                const int src = __builtin_ctzll(mask);
                mask &= mask - 1;
                const uint32_t sb = __builtin_amdgcn_readfirstlane(__shfl(s_b, src, 64));
                const uint32_t eb = __builtin_amdgcn_readfirstlane(__shfl(e_b, src, 64));
                const uint32_t len_b = __builtin_amdgcn_readfirstlane(__shfl(len, src, 64));
                uint32_t lo, hi;                                       // pages [lo, hi) of the sequence: this segment
                ixm::stream_segment(rlo, rhi, sb, eb, &lo, &hi);
                segment(b0 + src, lo, hi, len_b);
            }
        }
    }
}

// Merges the partial results of one (sequence, query head): block = 256 threads,
// thread (part, d) sums every second partial for dim d, then the two parts are added.
__global__ void __launch_bounds__(256) decode_stream_merge_kernel(StreamParams p, void *__restrict__ out, int out_bf16,
                                                                 float *__restrict__ pmax) {
    __shared__ float s_acc[128], s_den, s_max[2];
    __shared__ uint32_t s_tot[4], s_pre[4];
    const uint32_t h = blockIdx.x, d = threadIdx.x % 128, part = threadIdx.x / 128;
    const uint32_t kvh = h / p.group;
    const uint32_t b = blockIdx.y, hg = h % p.group;
    const uint32_t max_ctx = p.max_blocks_per_seq * kPage;
    uint32_t tot = 0, pre = 0;
    for (uint32_t bb = threadIdx.x; bb < p.batch; bb += 256) {
        uint32_t v = seq_pages<false>(p, bb, max_ctx);
        tot += v;
        if (bb < b) pre += v;
    }
    tot = (uint32_t)wave_sum<uint32_t>(tot);
    pre = (uint32_t)wave_sum<uint32_t>(pre);
    if (threadIdx.x % 64 == 0) {
        s_tot[threadIdx.x / 64] = tot;
        s_pre[threadIdx.x / 64] = pre;
    }
    __syncthreads();
    tot = s_tot[0] + s_tot[1] + s_tot[2] + s_tot[3];
    pre = s_pre[0] + s_pre[1] + s_pre[2] + s_pre[3];
    const uint32_t npg = seq_pages<false>(p, b, max_ctx);
    const uint32_t per = range_pages(p, tot);
    uint32_t r_lo, r_hi;
    ixm::stream_merge_ranges(pre, npg, per, &r_lo, &r_hi);   // empty sequence: no partials
    float mx = -INFINITY;
    float acc = 0.0f, den = 0.0f;
    constexpr int kOneTrip = 8;
    const bool one_trip = npg == 0 || r_hi - r_lo < (uint32_t)kOneTrip;
    if (one_trip) {
        // up to eight partial results: all maxima and this thread's every second (l, o) are requested at once,
        // one memory round trip instead of two; the arithmetic and its order are those of the loops below
        float m[kOneTrip], l[kOneTrip / 2], o[kOneTrip / 2];
#pragma unroll
        for (int u = 0; u < kOneTrip; ++u) {
            const uint64_t r = r_lo + u <= r_hi ? r_lo + u : r_hi;
            m[u] = p.part_ml[((r + b) * p.num_kv_heads + kvh) * (2 * p.g_pad) + hg];
        }
#pragma unroll
        for (int u = 0; u < kOneTrip / 2; ++u) {
            const uint64_t r = r_lo + part + 2 * u <= r_hi ? r_lo + part + 2 * u : r_hi;
            const uint64_t item = (r + b) * p.num_kv_heads + kvh;
            l[u] = p.part_ml[item * (2 * p.g_pad) + p.g_pad + hg];
            o[u] = p.part_o[(item * p.g_pad + hg) * kDh + d];
        }
#pragma unroll
        for (int u = 0; u < kOneTrip; ++u)
            if (r_lo + u <= r_hi) mx = (m[u] != m[u] || mx != mx) ? __uint_as_float(0x7fc00000u) : fmaxf(mx, m[u]);
#pragma unroll
        for (int u = 0; u < kOneTrip / 2; ++u) {
            if (r_lo + part + 2 * u <= r_hi) {
                // m of partial part + 2 u: a static index for either value of part
                const float mu = part ? m[2 * u + 1] : m[2 * u];
                const float w = expf(mu - mx);
                den = __builtin_fmaf(w, l[u], den);
                acc = __builtin_fmaf(w, o[u], acc);
            }
        }
    }
    for (uint32_t r = r_lo; !one_trip && r <= r_hi; ++r) {
        float m = p.part_ml[((uint64_t)(r + b) * p.num_kv_heads + kvh) * (2 * p.g_pad) + hg];
        mx = (m != m || mx != mx) ? __uint_as_float(0x7fc00000u) : fmaxf(mx, m);   // NaN marks a violation
    }
    for (uint32_t r = r_lo + part; !one_trip && r <= r_hi; r += 2) {
        const uint64_t item = (uint64_t)(r + b) * p.num_kv_heads + kvh;
        float m = p.part_ml[item * (2 * p.g_pad) + hg];
        float l = p.part_ml[item * (2 * p.g_pad) + p.g_pad + hg];
        float w = expf(m - mx);
        den = __builtin_fmaf(w, l, den);
        acc = __builtin_fmaf(w, p.part_o[(item * p.g_pad + hg) * kDh + d], acc);
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
        float res = npg == 0 ? 0.0f : __fdiv_rn(acc, den);
        uint64_t oi = ((uint64_t)b * p.num_heads + h) * kDh + d;
        if (out_bf16) {
            uint16_t rb = f32_to_bf16(res);
            ((uint16_t *)out)[oi] = rb;
            res = bf16_to_f32(rb);
        } else {
            ((float *)out)[oi] = res;
        }
        a = fabsf(res);
    }
    if (pmax) {                      // absmax of the stored head slice, for the quantizer that follows
        a = wave_max(a);
        if (part == 0 && threadIdx.x % 64 == 0) s_max[threadIdx.x / 64] = a;
        __syncthreads();
        if (threadIdx.x == 0) pmax[(uint64_t)b * p.num_heads + h] = fmaxf(s_max[0], s_max[1]);
    }
}

// Prefill: one block per (kv head, virtual sequence) merges the partial results of all its columns
// (token tiles x tokens of a tile x heads of the group): eight columns at a time, thread = (column slot, dim);
// a column's partials are read one after the other, so the columns are what runs in parallel.
constexpr int kPrefillMergeThreads = 1024;
__global__ void __launch_bounds__(kPrefillMergeThreads)
    prefill_stream_merge_kernel(StreamParams p, void *__restrict__ out, int out_bf16) {
    constexpr int kW = kPrefillMergeThreads / 64, kSlots = kPrefillMergeThreads / 128;
    __shared__ uint32_t s_tot[kW], s_pre[kW];
    const uint32_t kvh = blockIdx.x, vq = blockIdx.y, d = threadIdx.x % 128, part = threadIdx.x / 128;
    const uint32_t max_ctx = p.max_blocks_per_seq * kPage;
    uint32_t tot = 0, pre = 0;
    for (uint32_t bb = threadIdx.x; bb < p.n_vseq; bb += kPrefillMergeThreads) {
        uint32_t v = seq_pages<true>(p, bb, max_ctx);
        tot += v;
        if (bb < vq) pre += v;
    }
    tot = (uint32_t)wave_sum<uint32_t>(tot);
    pre = (uint32_t)wave_sum<uint32_t>(pre);
    if (threadIdx.x % 64 == 0) {
        s_tot[threadIdx.x / 64] = tot;
        s_pre[threadIdx.x / 64] = pre;
    }
    __syncthreads();
    tot = pre = 0;
#pragma unroll
    for (int w = 0; w < kW; ++w) {
        tot += s_tot[w];
        pre += s_pre[w];
    }
    const uint32_t npg = seq_pages<true>(p, vq, max_ctx);
    const uint32_t per = range_pages(p, tot);
    uint32_t r_lo, r_hi;
    ixm::stream_merge_ranges(pre, npg, per, &r_lo, &r_hi);   // nothing streamed: no partials
    const uint32_t seq = vq / p.qt, tiles = p.tpv / p.tpt, cols = p.tpt * p.group;
    const bool violation = p.seq_lens[seq] < p.l_new;              // possible only with unvalidated device tables
    for (uint32_t ci = part; ci < tiles * cols; ci += kSlots) {
        const uint32_t tile = ci / cols, col = ci % cols;
        const uint32_t t = p.t0 + (vq % p.qt) * p.tpv + tile * p.tpt + col / p.group;
        if (t >= p.l_new) continue;
        float mx = -INFINITY;
        for (uint32_t r = r_lo; r <= r_hi; ++r) {
            float m = p.part_ml[(((uint64_t)(r + vq) * p.num_kv_heads + kvh) * tiles + tile) * (2 * p.g_pad) + col];
            mx = (m != m || mx != mx) ? __uint_as_float(0x7fc00000u) : fmaxf(mx, m);   // NaN marks a violation
        }
        float acc = 0.0f, den = 0.0f;
        for (uint32_t r = r_lo; r <= r_hi; ++r) {
            const uint64_t item = ((uint64_t)(r + vq) * p.num_kv_heads + kvh) * tiles + tile;
            float m = p.part_ml[item * (2 * p.g_pad) + col];
            float l = p.part_ml[item * (2 * p.g_pad) + p.g_pad + col];
            float w = expf(m - mx);
            den = __builtin_fmaf(w, l, den);
            acc = __builtin_fmaf(w, p.part_o[(item * p.g_pad + col) * kDh + d], acc);
        }
        float res = npg == 0 ? 0.0f : __fdiv_rn(acc, den);
        if (violation) res = __uint_as_float(0x7fc00000u);
        const uint64_t oi = (((uint64_t)seq * p.l_new + t) * p.num_heads + (uint64_t)kvh * p.group + col % p.group) * kDh + d;
        if (out_bf16)
            ((uint16_t *)out)[oi] = f32_to_bf16(res);
        else
            ((float *)out)[oi] = res;
    }
}

// The merge above for a whole sequence per block, followed by the per-token int8 quantizer of the
// projection that consumes the attention output: thread (head, 4 dims) merges its partial results,
// rounds once to bf16 (the attention output's type), the block takes the row's absmax, and the row
// leaves as int8 activation tiles plus its scale.  Rows at or past the batch are written as zeros.
// QUANT = false: the same merge without the quantizer, the row stored as the operator's output (bf16 or
// f32) with, when asked, the absmax of every head's slice; used whenever the heads fit one block.
template <bool QUANT>
__global__ void __launch_bounds__(1024) decode_stream_merge_quantize_kernel(StreamParams p, int8_t *__restrict__ xq_tiled,
                                                                           float *__restrict__ sx, void *__restrict__ out,
                                                                           int out_bf16, float *__restrict__ pmax,
                                                                           uint32_t row_blocks, WeightPrefetch pull) {
    __shared__ uint32_t s_tot[16], s_pre[16];
    __shared__ float s_max[16];
    if (blockIdx.x >= row_blocks) {                      // appended blocks: weights of the linear that follows
        prefetch_weights(pull, blockIdx.x - row_blocks);
        return;
    }
    const uint32_t b = blockIdx.x;
    const uint32_t e_q = p.num_heads * kDh, k_tiles = e_q / 64;
    const int wave = threadIdx.x / 64, n_waves = blockDim.x / 64;
    if (b >= p.batch) {
        if constexpr (QUANT)
            for (uint32_t c = threadIdx.x; c < e_q / 16; c += blockDim.x)
                *(v4u *)(xq_tiled + tiled_chunk_offset(b, c, k_tiles)) = v4u{0, 0, 0, 0};
        return;
    }
    const uint32_t max_ctx = p.max_blocks_per_seq * kPage;
    uint32_t tot = 0, pre = 0;
    for (uint32_t bb = threadIdx.x; bb < p.batch; bb += blockDim.x) {
        uint32_t v = seq_pages<false>(p, bb, max_ctx);
        tot += v;
        if (bb < b) pre += v;
    }
    tot = wave_sum_dpp<uint32_t>(tot);
    pre = wave_sum_dpp<uint32_t>(pre);
    if (threadIdx.x % 64 == 0) {
        s_tot[wave] = tot;
        s_pre[wave] = pre;
    }
    __syncthreads();
    tot = 0;
    pre = 0;
    for (int w = 0; w < n_waves; ++w) {
        tot += s_tot[w];
        pre += s_pre[w];
    }
    const uint32_t npg = seq_pages<false>(p, b, max_ctx);
    const uint32_t per = range_pages(p, tot);
    uint32_t r_lo, r_hi;
    ixm::stream_merge_ranges(pre, npg, per, &r_lo, &r_hi);   // empty sequence: no partials

    // blockDim.x == num_heads * 32: thread (h, q) owns dims 4 q .. 4 q + 3 of head h
    const uint32_t h = threadIdx.x / 32, d4 = (threadIdx.x % 32) * 4;
    const uint32_t kvh = h / p.group, hg = h % p.group;
    // partial results four at a time, all loads of a batch issued before the first use (the loop is a
    // chain of L2 round trips otherwise); slots past r_hi repeat the last one with weight zero
    const float *ml = p.part_ml + ((uint64_t)b * p.num_kv_heads + kvh) * (2 * p.g_pad) + hg;
    const float *po = p.part_o + (((uint64_t)b * p.num_kv_heads + kvh) * p.g_pad + hg) * kDh + d4;
    const uint64_t ml_step = (uint64_t)p.num_kv_heads * (2 * p.g_pad), po_step = (uint64_t)p.num_kv_heads * p.g_pad * kDh;
    float mx = -INFINITY;
    v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
    float den = 0.0f;
    constexpr int kOneTrip = 8;
    const bool one_trip = npg == 0 || r_hi - r_lo < (uint32_t)kOneTrip;
    if (one_trip) {
        // up to eight partial results: everything is requested at once and the maximum is taken from registers,
        // one memory round trip instead of two; the arithmetic and its order are those of the loops below
        float m[kOneTrip], l[kOneTrip];
        v4f o[kOneTrip];
#pragma unroll
        for (int u = 0; u < kOneTrip; ++u) {
            const uint64_t r = r_lo + u <= r_hi ? r_lo + u : r_hi;
            m[u] = ml[r * ml_step];
            l[u] = ml[r * ml_step + p.g_pad];
            o[u] = *(const v4f *)(po + r * po_step);
        }
#pragma unroll
        for (int u = 0; u < kOneTrip; ++u)
            if (r_lo + u <= r_hi) mx = (m[u] != m[u] || mx != mx) ? __uint_as_float(0x7fc00000u) : fmaxf(mx, m[u]);
#pragma unroll
        for (int u = 0; u < kOneTrip; ++u) {
            if (r_lo + u <= r_hi) {
                const float w = expf(m[u] - mx);
                den = __builtin_fmaf(w, l[u], den);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] = __builtin_fmaf(w, o[u][e], acc[e]);
            }
        }
    }
    for (uint32_t r0 = r_lo; !one_trip && r0 <= r_hi; r0 += 4) {
        float m[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) m[u] = ml[(uint64_t)(r0 + u <= r_hi ? r0 + u : r_hi) * ml_step];
#pragma unroll
        for (int u = 0; u < 4; ++u)
            mx = (m[u] != m[u] || mx != mx) ? __uint_as_float(0x7fc00000u) : fmaxf(mx, m[u]);   // NaN marks a violation
    }
    for (uint32_t r0 = r_lo; !one_trip && r0 <= r_hi; r0 += 4) {
        float m[4], l[4];
        v4f o[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint64_t r = r0 + u <= r_hi ? r0 + u : r_hi;
            m[u] = ml[r * ml_step];
            l[u] = ml[r * ml_step + p.g_pad];
            o[u] = *(const v4f *)(po + r * po_step);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            float w = r0 + u <= r_hi ? expf(m[u] - mx) : 0.0f;
            den = __builtin_fmaf(w, l[u], den);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = __builtin_fmaf(w, o[u][e], acc[e]);
        }
    }
    float v[4], amax = 0.0f;
    if constexpr (!QUANT) {
        const uint64_t oi = ((uint64_t)b * p.num_heads + h) * kDh + d4;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float res = npg == 0 ? 0.0f : __fdiv_rn(acc[e], den);
            if (out_bf16) res = bf16_to_f32(f32_to_bf16(res));
            v[e] = res;
            amax = fmaxf(amax, fabsf(res));
        }
        if (out_bf16) {
            const uint32_t lo = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
            const uint32_t hi = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
            *(v2u *)((uint16_t *)out + oi) = v2u{lo, hi};
        } else {
            *(v4f *)((float *)out + oi) = v4f{v[0], v[1], v[2], v[3]};
        }
        if (pmax) {                                    // absmax of the stored head slice: the 32 threads of a head
#pragma unroll
            for (int off = 1; off < 32; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
            if (threadIdx.x % 32 == 0) pmax[(uint64_t)b * p.num_heads + h] = amax;
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float res = npg == 0 ? 0.0f : __fdiv_rn(acc[e], den);
        v[e] = bf16_to_f32(f32_to_bf16(res));         // the attention output is bf16: round once, then quantize
        amax = fmaxf(amax, fabsf(v[e]));
    }
    amax = wave_max_dpp(amax);
    if (threadIdx.x % 64 == 0) s_max[wave] = amax;
    __syncthreads();
    amax = 0.0f;
    for (int w = 0; w < n_waves; ++w) amax = fmaxf(amax, s_max[w]);
    const float scale = __fdiv_rn(amax, 127.0f);
    if (threadIdx.x == 0) sx[b] = scale;
    uint32_t word = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) word |= ((uint32_t)quant_i8(v[e], scale) & 0xffu) << (8 * e);
    const uint32_t col = h * kDh + d4;
    *(uint32_t *)(xq_tiled + tiled_chunk_offset(b, col / 16, k_tiles) + col % 16) = word;
}

// ------------------------------------------------------- prefill, block form
// Causal attention of many new tokens per row, one block of NW wavefronts per (row, kv head, tile of
// 32 NW / group new tokens).  The block walks the cached positions once, 32 at a time: the K and V rows
// of a step are staged in LDS (two stages; the loads of the next three steps are in flight while this
// one is multiplied) and shared by the wavefronts, so K / V leave the L2 once per tile.  Every
// wavefront owns 32 columns (new token x head of the group, column = token * group + head):
//   S^T = K Q^T on v_mfma_f32_16x16x32_bf16 as in the decode kernel (lane (g, c): positions 4g .. 4g+3
//   of a 16-position tile for column c), two position tiles per step;
//   O^T += V^T P^T on the same instruction with k = the 32 positions of the step: the operand slot
//   8g + i of a lane is position 4g + i of the first tile (i < 4) or of the second (i >= 4), which is
//   where the scores of that lane already are; V^T is read from the staged rows 4 bytes (two dims of
//   one position) at a time and split into an even and an odd operand by byte permutes.  Every f32
//   weight is fed as three bf16 terms that add up to it exactly, as in the decode kernel.
// The running maximum is per column; accumulators are rescaled only on steps where some column's maximum
// grew.  A step wholly past the causal limit of all the columns of a wavefront is skipped by it.  The
// result is normalised and written by the block itself (no partial results, no merge pass).
struct FlashParams {
    const uint16_t *q, *k_pool, *v_pool;
    const uint32_t *tables, *seq_lens;
    void *out;
    int out_bf16;
    uint32_t num_blocks, e_kv, batch, num_heads, num_kv_heads, group, max_blocks_per_seq, l_new, tq, tiles;
    float scale;
    // Split walk (few blocks against a long cache): gridDim.y blocks share a tile, block y walks the steps
    // [y, y + 1) * ceil(steps / gridDim.y) and leaves its unnormalised sums, running maxima and denominators in
    // part_o [tile block][y][column][128] / part_ml [tile block][y][2][columns]; flash_split_merge_kernel adds them.
    uint32_t nsplit;
    float *part_o, *part_ml;
};
constexpr int kFlashNQ = 2, kFlashKeys = 32;

// NQ: column tiles of 16 per wavefront (2: 32 columns; 1: 16 columns, half the multiplies per step and twice the blocks,
// for prompts that leave most compute units without a block).
template <int NW, int NQ = kFlashNQ>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) prefill_flash_kernel(FlashParams p) {
    constexpr int kRows = NW * 4, kPasses = kFlashKeys / kRows;   // staging: rows per pass of the block, passes per step
    __shared__ __attribute__((aligned(16))) uint16_t k_s[2][kFlashKeys * kVPitch];
    __shared__ __attribute__((aligned(16))) uint16_t v_s[2][kFlashKeys * kVPitch];
    __shared__ uint32_t s_bad;
    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int g = lane / 16, c = lane % 16;
    // longest tiles first
    const uint32_t per_tile = p.batch * p.num_kv_heads;
    const uint32_t tile = p.tiles - 1 - blockIdx.x / per_tile;
    const uint32_t b = (blockIdx.x % per_tile) / p.num_kv_heads, kvh = blockIdx.x % p.num_kv_heads;
    const uint32_t max_ctx = p.max_blocks_per_seq * kPage;
    const uint32_t len = p.seq_lens[b];
    const bool violation = len < p.l_new || len > max_ctx;     // possible only with unvalidated device tables
    const uint32_t ctx = len > max_ctx ? max_ctx : len;
    const uint32_t base = violation ? 0 : len - p.l_new;       // cached positions before the new tokens
    const uint32_t t0 = tile * p.tq;
    const uint32_t t_end = t0 + p.tq < p.l_new ? t0 + p.tq : p.l_new;
    uint32_t kmax = violation ? 0 : base + t_end;              // positions the last token of the tile sees
    if (kmax > ctx) kmax = ctx;
    const uint32_t npages = (kmax + kPage - 1) / kPage, n_all = (kmax + kFlashKeys - 1) / kFlashKeys;
    const uint32_t *tab = p.tables + (uint64_t)b * p.max_blocks_per_seq;
    // this block's share of the walk: steps [it_lo, n_it)
    const uint32_t per_split = (n_all + p.nsplit - 1) / p.nsplit;
    const uint32_t it_lo = p.nsplit > 1 ? (blockIdx.y * per_split < n_all ? blockIdx.y * per_split : n_all) : 0;
    const uint32_t n_it = p.nsplit > 1 ? (it_lo + per_split < n_all ? it_lo + per_split : n_all) : n_all;

    // first page of the walk whose id is outside the pool: columns that would read it give NaN
    if (tid == 0) s_bad = 0xffffffffu;
    __syncthreads();
    for (uint32_t i = tid; i < npages; i += NW * 64)
        if (tab[i] >= p.num_blocks) atomicMin(&s_bad, i);
    __syncthreads();
    const uint32_t first_bad_tok = s_bad == 0xffffffffu ? 0xffffffffu : s_bad * kPage;

    // Q^T operands and causal limits of this lane's columns
    v8bf qb[NQ][4];
    uint32_t lim[NQ];
    bool valid[NQ];
    uint64_t out_row[NQ];
#pragma unroll
    for (int qi = 0; qi < NQ; ++qi) {
        const uint32_t col = (uint32_t)wave * (NQ * 16) + qi * 16 + c;
        const uint32_t t = t0 + col / p.group, hc = col % p.group;
        valid[qi] = col < p.tq * p.group && t < p.l_new;        // a group that does not divide the columns leaves some idle
        const uint32_t tc = valid[qi] ? t : 0;
        out_row[qi] = (((uint64_t)b * p.l_new + tc) * p.num_heads + (uint64_t)kvh * p.group + hc) * kDh;
        const uint16_t *qrow = p.q + out_row[qi] + 8 * g;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            v4u t4 = *(const v4u *)(qrow + 32 * s);
            if (!valid[qi]) t4 = v4u{0, 0, 0, 0};
            qb[qi][s] = __builtin_bit_cast(v8bf, t4);
        }
        const uint32_t l = base + t + 1;
        lim[qi] = !valid[qi] || violation ? 0 : (l < ctx ? l : ctx);
    }
    uint32_t wmax = 0, wmin = 0xffffffffu;
#pragma unroll
    for (int qi = 0; qi < NQ; ++qi) {
        wmax = lim[qi] > wmax ? lim[qi] : wmax;
        wmin = lim[qi] < wmin ? lim[qi] : wmin;
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t a = __shfl_xor(wmax, off, 64), i = __shfl_xor(wmin, off, 64);
        wmax = a > wmax ? a : wmax;
        wmin = i < wmin ? i : wmin;
    }
    wmax = __builtin_amdgcn_readfirstlane(wmax);
    wmin = __builtin_amdgcn_readfirstlane(wmin);

    // staging: thread (row r of the step, 16-byte piece c16).  Page ids are requested four steps and K / V
    // rows three steps ahead of the step that multiplies them, so neither the id -> row dependence nor the
    // row loads themselves are waited for; steps past the walk repeat its last page (never used).
    const uint32_t r_st = tid / 16, c16 = tid % 16;           // pass ps stages row r_st + ps * kRows
    auto load_id = [&](uint32_t it, int ps) -> uint32_t {
        uint32_t pg = (it * kFlashKeys + ps * kRows + r_st) / kPage;
        if (pg >= npages) pg = npages - 1;
        return tab[pg];
    };
    auto row_off = [&](uint32_t it, int ps, uint32_t id) -> uint64_t {
        if (id >= p.num_blocks) id = 0;
        return ((uint64_t)id * kPage + (it * kFlashKeys + ps * kRows + r_st) % kPage) * p.e_kv + (uint64_t)kvh * kDh + 8 * c16;
    };
    v4u k_a[kPasses], v_a[kPasses], k_b[kPasses], v_b[kPasses];  // rows of step it + 1 (a) and it + 2 (b)
    uint32_t id_c[kPasses];                                      // page ids of step it + 3
#pragma unroll
    for (int ps = 0; ps < kPasses; ++ps) {
        k_a[ps] = v_a[ps] = k_b[ps] = v_b[ps] = v4u{0, 0, 0, 0};
        id_c[ps] = 0;
    }
    if (n_it > it_lo) {
#pragma unroll
        for (int ps = 0; ps < kPasses; ++ps) {
            const uint32_t id0 = load_id(it_lo, ps), id1 = load_id(it_lo + 1, ps), id2 = load_id(it_lo + 2, ps);
            id_c[ps] = load_id(it_lo + 3, ps);
            const uint64_t off0 = row_off(it_lo, ps, id0), off1 = row_off(it_lo + 1, ps, id1), off2 = row_off(it_lo + 2, ps, id2);
            v4u k0 = *(const v4u *)(p.k_pool + off0), v0 = *(const v4u *)(p.v_pool + off0);
            k_a[ps] = *(const v4u *)(p.k_pool + off1);
            v_a[ps] = *(const v4u *)(p.v_pool + off1);
            k_b[ps] = *(const v4u *)(p.k_pool + off2);
            v_b[ps] = *(const v4u *)(p.v_pool + off2);
            const uint32_t row = ps * kRows + r_st;
            if (it_lo * kFlashKeys + row >= ctx) v0 = v4u{0, 0, 0, 0};   // the pool may hold anything past the sequence end
            *(v4u *)(&k_s[0][row * kVPitch + 8 * c16]) = k0;
            *(v4u *)(&v_s[0][row * kVPitch + 8 * c16]) = v0;
        }
    }
    __syncthreads();

    float m_run[NQ], l_run[NQ];
    v4f o[NQ][8];
#pragma unroll
    for (int qi = 0; qi < NQ; ++qi) {
        m_run[qi] = -INFINITY;
        l_run[qi] = 0.0f;
#pragma unroll
        for (int t = 0; t < 8; ++t) o[qi][t] = v4f{0.f, 0.f, 0.f, 0.f};
    }
    constexpr float kLog2e = 1.4426950408889634f;

    for (uint32_t it = it_lo; it < n_it; ++it) {
        const int st = (it - it_lo) & 1;
        // requests of this step: the rows of step it + 3 (their page id was requested one step ago) and the
        // page id of step it + 4
        v4u k_n[kPasses], v_n[kPasses];
#pragma unroll
        for (int ps = 0; ps < kPasses; ++ps) {
            const uint32_t id_use = id_c[ps];
            id_c[ps] = load_id(it + 4, ps);
            const uint64_t off_n = row_off(it + 3, ps, id_use);
            k_n[ps] = *(const v4u *)(p.k_pool + off_n);
            v_n[ps] = *(const v4u *)(p.v_pool + off_n);
        }
        const uint32_t key0 = it * kFlashKeys;
        if (key0 < wmax) {
            // ---- scores of the step: two tiles of 16 positions
            float sc[NQ][8];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                v4u ka[4];
#pragma unroll
                for (int s = 0; s < 4; ++s) ka[s] = *(const v4u *)(&k_s[st][(kt * 16 + c) * kVPitch + 32 * s + 8 * g]);
#pragma unroll
                for (int qi = 0; qi < NQ; ++qi) {
                    v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < 4; ++s)
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, ka[s]), qb[qi][s], acc, 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < 4; ++j) sc[qi][kt * 4 + j] = acc[j] * p.scale;
                }
            }
            if (key0 + kFlashKeys > wmin) {
#pragma unroll
                for (int qi = 0; qi < NQ; ++qi)
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const uint32_t tok = key0 + (i / 4) * 16 + 4 * g + (i % 4);
                        sc[qi][i] = tok < lim[qi] ? sc[qi][i] : -INFINITY;
                    }
            }
            // ---- running maximum per column (lanes with equal c hold one column)
            float m_new[NQ], m_use[NQ];
            bool grew = false;
#pragma unroll
            for (int qi = 0; qi < NQ; ++qi) {
                float m = sc[qi][0];
#pragma unroll
                for (int i = 1; i < 8; ++i) m = fmaxf(m, sc[qi][i]);
                m = fmaxf(m, __shfl_xor(m, 16, 64));
                m = fmaxf(m, __shfl_xor(m, 32, 64));
                m_new[qi] = fmaxf(m_run[qi], m);
                grew = grew || m_new[qi] > m_run[qi];
                // every score of a column can be masked so far: its maximum stays -inf and the exponentials
                // are taken against 0
                m_use[qi] = m_new[qi] == -INFINITY ? 0.0f : m_new[qi];
            }
            if (__ballot(grew) != 0) {
#pragma unroll
                for (int qi = 0; qi < NQ; ++qi) {
                    const float alpha = __builtin_amdgcn_exp2f((m_run[qi] - m_use[qi]) * kLog2e);   // first step: exp2(-inf) = 0
                    l_run[qi] *= alpha;
#pragma unroll
                    for (int t = 0; t < 8; ++t) o[qi][t] = o[qi][t] * alpha;
                }
            }
            // each f32 weight as three bf16 operands by repeated truncation: hi + mid + lo == weight exactly
            v8bf p_hi[NQ], p_mid[NQ], p_lo[NQ];
#pragma unroll
            for (int qi = 0; qi < NQ; ++qi) {
                m_run[qi] = m_new[qi];
                float sum = 0.0f;
                v4u ph, pm, pl;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float e[2];
                    uint32_t hi[2], mid[2], lo[2];
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        // the difference is exact for scores near the maximum, which carry the weight;
                        // masked scores: exp2(-inf) = 0
                        e[h] = __builtin_amdgcn_exp2f((sc[qi][2 * i + h] - m_use[qi]) * kLog2e);
                        hi[h] = __float_as_uint(e[h]) & 0xffff0000u;
                        const float r1 = e[h] - __uint_as_float(hi[h]);
                        mid[h] = __float_as_uint(r1) & 0xffff0000u;
                        lo[h] = __float_as_uint(r1 - __uint_as_float(mid[h]));
                    }
                    sum += e[0] + e[1];
                    ph[i] = __builtin_amdgcn_perm(hi[1], hi[0], 0x07060302u);
                    pm[i] = __builtin_amdgcn_perm(mid[1], mid[0], 0x07060302u);
                    pl[i] = __builtin_amdgcn_perm(lo[1], lo[0], 0x07060302u);
                }
                l_run[qi] += sum;
                p_hi[qi] = __builtin_bit_cast(v8bf, ph);
                p_mid[qi] = __builtin_bit_cast(v8bf, pm);
                p_lo[qi] = __builtin_bit_cast(v8bf, pl);
            }
            // ---- O^T += V^T P^T
#pragma unroll
            for (int bp = 0; bp < 4; ++bp) {
                uint32_t w[8];
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    w[i] = *(const uint32_t *)(&v_s[st][((i / 4) * 16 + 4 * g + (i % 4)) * kVPitch + 32 * bp + 2 * c]);
                v4u ae, ao;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    ae[i] = __builtin_amdgcn_perm(w[2 * i + 1], w[2 * i], 0x05040100u);
                    ao[i] = __builtin_amdgcn_perm(w[2 * i + 1], w[2 * i], 0x07060302u);
                }
                const v8bf a_even = __builtin_bit_cast(v8bf, ae), a_odd = __builtin_bit_cast(v8bf, ao);
#pragma unroll
                for (int qi = 0; qi < NQ; ++qi) {
                    // smallest terms first
                    o[qi][2 * bp] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_even, p_lo[qi], o[qi][2 * bp], 0, 0, 0);
                    o[qi][2 * bp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_odd, p_lo[qi], o[qi][2 * bp + 1], 0, 0, 0);
                    o[qi][2 * bp] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_even, p_mid[qi], o[qi][2 * bp], 0, 0, 0);
                    o[qi][2 * bp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_odd, p_mid[qi], o[qi][2 * bp + 1], 0, 0, 0);
                    o[qi][2 * bp] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_even, p_hi[qi], o[qi][2 * bp], 0, 0, 0);
                    o[qi][2 * bp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_odd, p_hi[qi], o[qi][2 * bp + 1], 0, 0, 0);
                }
            }
        }
        // rows of step it + 1 go to the other stage (its readers passed the barrier of the last step)
#pragma unroll
        for (int ps = 0; ps < kPasses; ++ps) {
            const uint32_t row = ps * kRows + r_st;
            if ((it + 1) * kFlashKeys + row >= ctx) v_a[ps] = v4u{0, 0, 0, 0};
            *(v4u *)(&k_s[st ^ 1][row * kVPitch + 8 * c16]) = k_a[ps];
            *(v4u *)(&v_s[st ^ 1][row * kVPitch + 8 * c16]) = v_a[ps];
            k_a[ps] = k_b[ps];
            v_a[ps] = v_b[ps];
            k_b[ps] = k_n[ps];
            v_b[ps] = v_n[ps];
        }
        __syncthreads();
    }

    // lane (g, c) holds, for column c: dims 32 bp + 8 g + {0..7} = {o[2bp][0], o[2bp+1][0], o[2bp][1], ...}
#pragma unroll
    for (int qi = 0; qi < NQ; ++qi) {
        float l = l_run[qi];
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);
        if (!valid[qi]) continue;
        const bool nan_out = violation || lim[qi] > first_bad_tok;
        if (p.nsplit > 1) {
            const uint32_t cols = NW * NQ * 16, col = (uint32_t)wave * (NQ * 16) + qi * 16 + c;
            const uint64_t slot = (uint64_t)blockIdx.x * p.nsplit + blockIdx.y;
            float *po = p.part_o + (slot * cols + col) * kDh + 8 * g;
#pragma unroll
            for (int bp = 0; bp < 4; ++bp) {
                *(v4f *)(po + 32 * bp) = v4f{o[qi][2 * bp][0], o[qi][2 * bp + 1][0], o[qi][2 * bp][1], o[qi][2 * bp + 1][1]};
                *(v4f *)(po + 32 * bp + 4) = v4f{o[qi][2 * bp][2], o[qi][2 * bp + 1][2], o[qi][2 * bp][3], o[qi][2 * bp + 1][3]};
            }
            if (g == 0) {
                const float nanv = __uint_as_float(0x7fc00000u);
                p.part_ml[slot * (2 * cols) + col] = nan_out ? nanv : m_run[qi];
                p.part_ml[slot * (2 * cols) + cols + col] = nan_out ? nanv : l;
            }
            continue;
        }
#pragma unroll
        for (int bp = 0; bp < 4; ++bp) {
            float r8[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float acc = o[qi][2 * bp + (e & 1)][e / 2];
                float res = l > 0.0f ? __fdiv_rn(acc, l) : 0.0f;
                r8[e] = nan_out ? __uint_as_float(0x7fc00000u) : res;
            }
            const uint64_t oi = out_row[qi] + 32 * bp + 8 * g;
            if (p.out_bf16) {
                v4u pk;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    pk[e] = (uint32_t)f32_to_bf16(r8[2 * e]) | ((uint32_t)f32_to_bf16(r8[2 * e + 1]) << 16);
                *(v4u *)((uint16_t *)p.out + oi) = pk;
            } else {
                *(v4f *)((float *)p.out + oi) = v4f{r8[0], r8[1], r8[2], r8[3]};
                *(v4f *)((float *)p.out + oi + 4) = v4f{r8[4], r8[5], r8[6], r8[7]};
            }
        }
    }
}

// Adds the shares of a split walk: one block per (tile block, eight columns), thread (column, dim).  The shares
// of a column are read eight at a time, all loads of a batch before the first use (a chain of L2 round trips
// otherwise); slots past the last share repeat it with weight zero.
template <int NW>
__global__ void __launch_bounds__(1024) flash_split_merge_kernel(FlashParams p) {
    constexpr uint32_t kCols = NW * kFlashNQ * 16;
    const uint32_t per_tile = p.batch * p.num_kv_heads;
    const uint32_t tile = p.tiles - 1 - blockIdx.x / per_tile;
    const uint32_t b = (blockIdx.x % per_tile) / p.num_kv_heads, kvh = blockIdx.x % p.num_kv_heads;
    const uint32_t d = threadIdx.x % 128, col = blockIdx.y * 8 + threadIdx.x / 128;
    const uint32_t t = tile * p.tq + col / p.group;
    if (col >= p.tq * p.group || t >= p.l_new) return;
    const float *ml = p.part_ml + (uint64_t)blockIdx.x * p.nsplit * (2 * kCols) + col;
    const float *po = p.part_o + ((uint64_t)blockIdx.x * p.nsplit * kCols + col) * kDh + d;
    const uint32_t last = p.nsplit - 1;
    float mx = -INFINITY;
    for (uint32_t z0 = 0; z0 < p.nsplit; z0 += 8) {
        float m[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) m[u] = ml[(uint64_t)(z0 + u < p.nsplit ? z0 + u : last) * (2 * kCols)];
#pragma unroll
        for (int u = 0; u < 8; ++u) mx = (m[u] != m[u] || mx != mx) ? __uint_as_float(0x7fc00000u) : fmaxf(mx, m[u]);   // NaN marks a violation
    }
    const float m_use = mx == -INFINITY ? 0.0f : mx;
    float acc = 0.0f, den = 0.0f;
    for (uint32_t z0 = 0; z0 < p.nsplit; z0 += 8) {
        float m[8], l[8], o[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const uint64_t z = z0 + u < p.nsplit ? z0 + u : last;
            m[u] = ml[z * (2 * kCols)];
            l[u] = ml[z * (2 * kCols) + kCols];
            o[u] = po[z * kCols * kDh];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float w = z0 + u < p.nsplit ? expf(m[u] - m_use) : 0.0f;           // a share that saw nothing: exp(-inf) = 0
            den = __builtin_fmaf(w, l[u], den);
            acc = __builtin_fmaf(w, o[u], acc);
        }
    }
    float res = den > 0.0f ? __fdiv_rn(acc, den) : 0.0f;
    if (mx != mx) res = mx;
    const uint64_t oi = (((uint64_t)b * p.l_new + t) * p.num_heads + (uint64_t)kvh * p.group + col % p.group) * kDh + d;
    if (p.out_bf16)
        ((uint16_t *)p.out)[oi] = f32_to_bf16(res);
    else
        ((float *)p.out)[oi] = res;
}

inline int group_pad(uint32_t group) {
    int gp = 1;
    while ((uint32_t)gp < group) gp *= 2;
    return gp;
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

}  // namespace k
int g_decode_partials_only = 0;   // profiling: launch only the streaming kernel (the output is not written)
int g_prefill_block_form = 0;     // 0: by shape, 1: never, 2: whenever the group size allows
int g_prefill_block_waves = 0;    // wavefronts per block of the block form: 4 or 8, anything else by shape
int g_prefill_block_split = 0;    // upper bound of the blocks that share one tile's walk (0: by shape)
int g_prefill_block_cols = 0;     // columns per wavefront of the block form: 0 by shape, 1: 16 whenever allowed, 2: always 32
namespace k {

static uint32_t compute_units() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
            cus = v;
        else
            cus = 256;
    }
    return (uint32_t)cus;
}

// Ranges of the streamed kernel: one wavefront per (range, kv head), `waves_per_cu` of them on every
// compute unit, all resident at once.  Four per compute unit (one per SIMD) measured best: longer
// ranges mean fewer partial results, and the loads in flight per wavefront already cover the latency.
static uint32_t stream_ranges(const PagedShape &ps, uint32_t waves_per_cu) {
    if (waves_per_cu == 0) waves_per_cu = 4;
    if (waves_per_cu > 8) waves_per_cu = 8;               // register budget of the kernel: two per SIMD
    uint32_t r = compute_units() * waves_per_cu / ps.num_kv_heads;
    return r ? r : 1;
}

uint64_t paged_decode_workspace_bytes(const PagedShape &ps, uint32_t waves_per_cu) {
    uint32_t group = ps.num_heads / ps.num_kv_heads;
    uint64_t gp = (uint64_t)group_pad(group);
    uint64_t items = ((uint64_t)stream_ranges(ps, waves_per_cu) + ps.batch) * ps.num_kv_heads;
    return items * (gp * kDh + 2 * gp) * sizeof(float);
}

void paged_attention_decode_bf16(const uint16_t *q, const uint16_t *k_pool, const uint16_t *v_pool,
                                 const uint32_t *tables, const uint32_t *seq_lens, const PagedShape &ps,
                                 uint32_t waves_per_cu, void *workspace, void *out, int out_bf16, float *pmax,
                                 hipStream_t s) {
    paged_attention_decode_bf16(q, k_pool, v_pool, tables, seq_lens, ps, waves_per_cu, workspace, out, out_bf16, pmax,
                                nullptr, nullptr, 0, s);
}

void paged_attention_decode_bf16(const uint16_t *q, const uint16_t *k_pool, const uint16_t *v_pool,
                                 const uint32_t *tables, const uint32_t *seq_lens, const PagedShape &ps,
                                 uint32_t waves_per_cu, void *workspace, void *out, int out_bf16, float *pmax,
                                 int8_t *xq_tiled, float *sx, uint32_t m_pad, hipStream_t s, const WeightPrefetch &pull) {
    if (ps.batch == 0) return;
    StreamParams sp;
    sp.q = q;
    sp.k_pool = k_pool;
    sp.v_pool = v_pool;
    sp.tables = tables;
    sp.seq_lens = seq_lens;
    sp.num_blocks = ps.num_blocks;
    sp.e_kv = ps.e_kv;
    sp.batch = ps.batch;
    sp.num_heads = ps.num_heads;
    sp.num_kv_heads = ps.num_kv_heads;
    sp.group = ps.num_heads / ps.num_kv_heads;
    sp.g_pad = (uint32_t)group_pad(sp.group);
    sp.max_blocks_per_seq = ps.max_blocks_per_seq;
    sp.n_ranges = stream_ranges(ps, waves_per_cu);
    sp.min_pages = 4;
    sp.scale = ps.scale;
    sp.l_new = sp.tpt = sp.tpv = sp.qt = 1;
    sp.t0 = 0;
    sp.n_vseq = ps.batch;
    uint64_t items = ((uint64_t)sp.n_ranges + ps.batch) * ps.num_kv_heads;
    sp.part_o = (float *)workspace;
    sp.part_ml = sp.part_o + items * (uint64_t)sp.g_pad * kDh;
    uint64_t waves = (uint64_t)sp.n_ranges * ps.num_kv_heads;
    decode_stream_kernel<4, 4, 2, 2, false><<<(unsigned)((waves + 3) / 4), 256, 0, s>>>(sp);
    if (g_decode_partials_only) return;
    if (xq_tiled != nullptr && ps.num_heads <= 32) {
        // fused merge + per-token quantizer (the bf16 output itself is not written)
        const WeightPrefetch pf = (pull.w && m_pad % 8 == 0) ? pull : WeightPrefetch{};
        decode_stream_merge_quantize_kernel<true><<<m_pad + pf.blocks, ps.num_heads * 32, 0, s>>>(sp, xq_tiled, sx, nullptr, 0, nullptr,
                                                                                                 m_pad, pf);
        return;
    }
    if (ps.num_heads <= 32 && ps.num_heads % 2 == 0) {    // a row per block (whole wavefronts): one launch of batch blocks
        decode_stream_merge_quantize_kernel<false><<<ps.batch, ps.num_heads * 32, 0, s>>>(sp, nullptr, nullptr, out, out_bf16, pmax, ps.batch,
                                                                                         WeightPrefetch{});
        return;
    }
    dim3 grid2(ps.num_heads, ps.batch);
    decode_stream_merge_kernel<<<grid2, 256, 0, s>>>(sp, out, out_bf16, pmax);
}

// Decode attention of a few short sequences with the finished output in one launch (decode_stream_kernel's ONE
// form): out_f32 [batch][num_heads][128] holds the output values rounded to bf16, pmax [batch][num_heads] the absmax
// of every head's slice, which is what a per-token quantizer in front of the next projection needs.  A compute unit
// per (sequence, kv head) streams the whole sequence, so this is for contexts of at most kDecodeOneMaxCtx tokens;
// longer ones go through paged_attention_decode_bf16.
int g_decode_one = 0;
void paged_attention_decode_one_bf16(const uint16_t *q, const uint16_t *k_pool, const uint16_t *v_pool, const uint32_t *tables,
                                     const uint32_t *seq_lens, const PagedShape &ps, float *out_f32, float *pmax, hipStream_t s) {
    if (ps.batch == 0) return;
    StreamParams sp;
    sp.q = q;
    sp.k_pool = k_pool;
    sp.v_pool = v_pool;
    sp.tables = tables;
    sp.seq_lens = seq_lens;
    sp.part_o = sp.part_ml = nullptr;
    sp.num_blocks = ps.num_blocks;
    sp.e_kv = ps.e_kv;
    sp.batch = ps.batch;
    sp.num_heads = ps.num_heads;
    sp.num_kv_heads = ps.num_kv_heads;
    sp.group = ps.num_heads / ps.num_kv_heads;
    sp.g_pad = (uint32_t)group_pad(sp.group);
    sp.max_blocks_per_seq = ps.max_blocks_per_seq;
    sp.n_ranges = ps.batch;
    sp.min_pages = 1;
    sp.scale = ps.scale;
    sp.l_new = sp.tpt = sp.tpv = sp.qt = 1;
    sp.t0 = 0;
    sp.n_vseq = ps.batch;
    sp.one_out = out_f32;
    sp.one_pmax = pmax;
    decode_stream_kernel<4, 4, 2, 2, false, 1, true><<<ps.batch * ps.num_kv_heads, 256, 0, s>>>(sp);
}

// Prefill (l_new > 1) on the same streaming kernel: groups of kPrefillTT token tiles of 16 / group new tokens
// are streamed as sequences of their own, at most kPrefillSeqs of them per launch so that the partial
// results stay within a bounded workspace; the launches for successive token ranges follow each other on
// the stream.  A call whose new tokens fit one tile uses the one-tile form (two wavefronts per SIMD).
constexpr uint32_t kPrefillSeqs = 512, kPrefillTT = 2;

static uint32_t prefill_tt(const PagedShape &ps) {
    uint32_t tpt = 16 / (ps.num_heads / ps.num_kv_heads);
    return ps.l_new > tpt ? kPrefillTT : 1;
}
static uint32_t prefill_seqs_per_row(const PagedShape &ps) {           // virtual sequences of one row per launch
    const uint32_t tpv = 16 / (ps.num_heads / ps.num_kv_heads) * prefill_tt(ps);
    const uint32_t all = (ps.l_new + tpv - 1) / tpv;
    uint32_t cap = kPrefillSeqs / ps.batch;
    if (cap == 0) cap = 1;
    return all < cap ? all : cap;
}

// shares of a split walk that one launch may leave in the workspace (four-wavefront blocks, 128 columns each)
static uint64_t flash_split_slots() { return 2ull * compute_units(); }
constexpr uint64_t kFlashSplitCols = 4 * kFlashNQ * 16;

uint64_t paged_prefill_workspace_bytes(const PagedShape &ps, uint32_t waves_per_cu) {
    uint64_t items = ((uint64_t)stream_ranges(ps, waves_per_cu) + (uint64_t)ps.batch * prefill_seqs_per_row(ps)) *
                     ps.num_kv_heads * prefill_tt(ps);
    const uint64_t streamed = items * (16 * kDh + 2 * 16) * sizeof(float);
    const uint64_t split = flash_split_slots() * kFlashSplitCols * (kDh + 2) * sizeof(float);
    return streamed > split ? streamed : split;
}

// Which prefill form a shape takes.  The block form walks the cache once per tile of new tokens, so its time
// is the longest walk (a lone block does a step of 32 positions in about 1.4 us) or, when blocks queue, the sum
// of the walks over the compute units; the streamed form splits every walk over the whole device but reads
// K / V once per 32 / group new tokens and merges partial results per new token.  The constants are measured
// (32 / 8 heads): they only need to be right where the two forms are far apart, which is where it matters.
struct BlockFormPlan {
    bool use;
    int waves;
    uint32_t nsplit;                    // blocks sharing a tile's walk (1: none)
};
static BlockFormPlan plan_block_form(const PagedShape &ps) {
    const uint32_t group = ps.num_heads / ps.num_kv_heads;
    if (group == 0 || group > 16 || g_prefill_block_form == 1) return {false, 0, 1};
    const uint32_t cus = compute_units();
    const uint32_t bound = ps.max_blocks_per_seq * kPage;
    uint32_t ctx = ps.ctx_hint != 0 && ps.ctx_hint < bound ? ps.ctx_hint : bound;
    if (ctx < ps.l_new) ctx = ps.l_new;
    const double cached = (double)(ctx - ps.l_new), l_new = (double)ps.l_new;
    const uint64_t rows = (uint64_t)ps.batch * ps.num_kv_heads;
    int waves = g_prefill_block_waves == 8 ? 8 : g_prefill_block_waves == 4 ? 4 : 0;
    if (waves == 0) {
        // eight wavefronts halve the K / V traffic of a block pair; they pay once the device is oversubscribed
        const uint32_t tq8 = 256 / group;
        waves = rows * ((ps.l_new + tq8 - 1) / tq8) >= 2ull * cus && ps.l_new >= 1024 ? 8 : 4;
    }
    const uint32_t tq = (uint32_t)waves * kFlashNQ * 16 / group, tiles = (ps.l_new + tq - 1) / tq;
    const double steps_longest = (cached + l_new) / kFlashKeys;
    // few blocks against a long walk over what was cached before (the walks of all tiles are then about equally
    // long): several blocks share a tile's walk (at least eight steps each, at most as many shares as the
    // workspace holds) and a merge pass adds them
    uint32_t nsplit = 1;
    const uint64_t blocks = rows * tiles;
    if (waves == 4 && blocks < cus && cached >= 2.0 * l_new) {
        uint64_t want = flash_split_slots() / blocks, by_steps = (uint64_t)(steps_longest / 8.0);
        if (g_prefill_block_split > 0) want = (uint64_t)g_prefill_block_split < want ? (uint64_t)g_prefill_block_split : want;
        nsplit = (uint32_t)(want < by_steps ? want : by_steps);
        if (nsplit < 1) nsplit = 1;
    }
    if (g_prefill_block_form == 2) return {true, waves, nsplit};
    const double steps_all = (double)blocks * (cached + (tiles > 1 ? 0.5 * l_new : l_new)) / kFlashKeys;
    const double per_cu = waves == 8 ? 2.05 : 1.05;                       // us per step at two wavefronts per SIMD
    const double a = steps_longest / nsplit * 1.4 + (nsplit > 1 ? 9.0 : 0.0), b = steps_all / cus * per_cu;
    const double t_block = (a > b ? a : b) + 8.0;
    const uint32_t tpt = 16 / group, tpv = ps.l_new > tpt ? 2 * tpt : tpt;
    const double bytes = (double)rows * ((ps.l_new + tpv - 1) / tpv) * (cached + 0.5 * l_new) * (2.0 * kDh * 2);
    const double t_stream = 35.0 + bytes / 4.9e6 + 0.035 * l_new * ps.batch;
    return {t_block <= t_stream, waves, nsplit};
}

void paged_attention_prefill_bf16(const uint16_t *q, const uint16_t *k_pool, const uint16_t *v_pool,
                                  const uint32_t *tables, const uint32_t *seq_lens, const PagedShape &ps,
                                  uint32_t waves_per_cu, void *workspace, void *out, int out_bf16, hipStream_t s) {
    if (ps.batch == 0 || ps.l_new == 0) return;
    const BlockFormPlan plan = plan_block_form(ps);
    if (plan.use) {
        FlashParams fp;
        fp.q = q;
        fp.k_pool = k_pool;
        fp.v_pool = v_pool;
        fp.tables = tables;
        fp.seq_lens = seq_lens;
        fp.out = out;
        fp.out_bf16 = out_bf16;
        fp.num_blocks = ps.num_blocks;
        fp.e_kv = ps.e_kv;
        fp.batch = ps.batch;
        fp.num_heads = ps.num_heads;
        fp.num_kv_heads = ps.num_kv_heads;
        fp.group = ps.num_heads / ps.num_kv_heads;
        fp.max_blocks_per_seq = ps.max_blocks_per_seq;
        fp.l_new = ps.l_new;
        fp.tq = (uint32_t)plan.waves * kFlashNQ * 16 / fp.group;
        fp.tiles = (ps.l_new + fp.tq - 1) / fp.tq;
        fp.scale = ps.scale;
        // A short prompt leaves compute units without a block, and a block's time is its walk: with 16 columns per
        // wavefront instead of 32 a step costs half the multiplies and there are twice the blocks (a 300-token prompt:
        // 80 -> 152 blocks; measured through 32 layers: 300 tokens 6.80 -> 6.59 ms, 1024 tokens 16.24 -> 15.72 ms).  Only
        // the unsplit four-wavefront form, and only while the wide blocks would not fill the device more than once.
        const bool narrow = g_prefill_block_cols != 2 && plan.waves == 4 && plan.nsplit == 1 && fp.group <= 16 && 16 % fp.group == 0 &&
                            (g_prefill_block_cols == 1 ||
                             (uint64_t)ps.batch * ps.num_kv_heads * fp.tiles <= (uint64_t)compute_units());
        if (narrow) {
            fp.tq = (uint32_t)plan.waves * 16 / fp.group;
            fp.tiles = (ps.l_new + fp.tq - 1) / fp.tq;
        }
        const uint64_t blocks = (uint64_t)ps.batch * ps.num_kv_heads * fp.tiles;
        fp.nsplit = plan.nsplit;
        fp.part_o = (float *)workspace;
        fp.part_ml = fp.part_o + blocks * fp.nsplit * kFlashSplitCols * kDh;
        if (plan.waves == 8) {
            prefill_flash_kernel<8><<<(unsigned)blocks, 512, 0, s>>>(fp);
        } else if (narrow) {
            prefill_flash_kernel<4, 1><<<(unsigned)blocks, 256, 0, s>>>(fp);
        } else {
            prefill_flash_kernel<4><<<dim3((unsigned)blocks, fp.nsplit), 256, 0, s>>>(fp);
            if (fp.nsplit > 1)
                flash_split_merge_kernel<4><<<dim3((unsigned)blocks, (unsigned)((fp.tq * fp.group + 7) / 8)), 1024, 0, s>>>(fp);
        }
        return;
    }
    StreamParams sp;
    sp.q = q;
    sp.k_pool = k_pool;
    sp.v_pool = v_pool;
    sp.tables = tables;
    sp.seq_lens = seq_lens;
    sp.num_blocks = ps.num_blocks;
    sp.e_kv = ps.e_kv;
    sp.batch = ps.batch;
    sp.num_heads = ps.num_heads;
    sp.num_kv_heads = ps.num_kv_heads;
    sp.group = ps.num_heads / ps.num_kv_heads;
    sp.g_pad = 16;
    sp.max_blocks_per_seq = ps.max_blocks_per_seq;
    sp.min_pages = 4;
    sp.scale = ps.scale;
    sp.l_new = ps.l_new;
    sp.tpt = 16 / sp.group;
    const uint32_t tt = prefill_tt(ps);
    sp.tpv = sp.tpt * tt;
    // the several-tile form keeps one wavefront per SIMD (register budget)
    sp.n_ranges = stream_ranges(ps, tt == 1 ? waves_per_cu : (waves_per_cu && waves_per_cu < 4 ? waves_per_cu : 4));
    const uint32_t vseqs = (ps.l_new + sp.tpv - 1) / sp.tpv;
    const uint32_t qt_max = prefill_seqs_per_row(ps);
    const uint64_t items_max = ((uint64_t)stream_ranges(ps, waves_per_cu) + (uint64_t)ps.batch * qt_max) * ps.num_kv_heads * tt;
    sp.part_o = (float *)workspace;
    sp.part_ml = sp.part_o + items_max * 16 * kDh;
    const uint64_t waves = (uint64_t)sp.n_ranges * ps.num_kv_heads;
    for (uint32_t v0 = 0; v0 < vseqs; v0 += qt_max) {
        sp.qt = vseqs - v0 < qt_max ? vseqs - v0 : qt_max;
        sp.t0 = v0 * sp.tpv;
        sp.n_vseq = ps.batch * sp.qt;
        if (tt == 1)
            decode_stream_kernel<4, 4, 2, 2, true, 1><<<(unsigned)((waves + 3) / 4), 256, 0, s>>>(sp);
        else
            decode_stream_kernel<4, 4, 2, 1, true, kPrefillTT><<<(unsigned)((waves + 3) / 4), 256, 0, s>>>(sp);
        if (g_decode_partials_only) continue;
        dim3 grid2(ps.num_kv_heads, sp.n_vseq);
        prefill_stream_merge_kernel<<<grid2, kPrefillMergeThreads, 0, s>>>(sp, out, out_bf16);
    }
}

}  // namespace k
}  // namespace fa
