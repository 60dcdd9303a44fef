// Decode-shape ("skinny", m <= 64 tokens for int8 activations, m <= 32 for bf16) quantized linears.  Both kernels are
// HBM-bound streams over the tile-ordered int8 weight: every wavefront load
// is one contiguous 1 KiB tile that lands directly in the operand layout of
// the matrix instruction, so the weight never passes through LDS.  The block
// splits K over its wavefronts and reduces their partial tiles in LDS in a
// fixed order (deterministic).
#include <algorithm>

#include <type_traits>

#include "device_utils.hpp"
#include "index_models.hpp"
#include "kernels.hpp"
#include "row_prologue.hpp"

namespace fa {
namespace k {
using namespace fa::dev;

int g_skinny_ntw = 0;      // tuning overrides (0 = heuristic)
int g_skinny_waves = 0;
int g_weight_prefetch = 0;   // 1: row kernels pull nothing for the linear that follows them
int g_rows_rope = 0;         // q | k | v of a prompt pass on the weight-stationary kernel: 0 RoPE and the append in its epilogue, 1 a pass of their own
int g_rows_kernel = 0;      // weight-stationary kernel for a few hundred rows: 0 by shape, 1 never, 2 whenever it can run
int g_skinny_astat = 0;     // activation-stationary kernel: 0 by shape, 1 never, 2 whenever it can run, 3 by shape but not the 33 to 64 row form
int g_skinny_ksplit = 0;    // split k over the blocks of an XCD: 0 by shape, 1 never, 2 whenever it can run (agent-scope
                            // meeting), 3 whenever it can run (meeting in the XCD's L2), 4 by shape but agent scope
int g_skinny_ksplit_s = 0;  // members per group of the split (0 by shape, 2 or 4)
int g_row_fusion = 0;       // row work inside the linears: 0 where it measured faster (norm: two rows, quantizer: one), 1 never, 2 up to the kernels' four / two rows

namespace {

struct EpiI8 {
    const float *sx, *sw, *bias, *residual;
    int32_t *acc_out;
    void *out;
    int out_bf16;
    float *pmax;          // SwiGLU mode: per (row, block) absmax of the activation
    // RoPE mode (fused q/k/v projection of a decode step)
    const float *cos_sin;     // [m][head_dim]: cos of the row's position for i < head_dim/2, then sin
    const uint32_t *slots;    // [m] cache row of the new token
    uint16_t *q_out, *k_pool, *v_pool;
    uint32_t heads, kv_heads, head_dim;
    uint64_t pool_rows;
};

enum { kEpiPlain = 0, kEpiSwiglu = 1, kEpiRope = 2 };


// ------------------------------------------------------------------ W8A8
// acc[m, n] = sum_k xq[m, k] * w[k, n] on v_mfma_i32_16x16x64_i8.
// D layout: lane l holds column l % 16, rows 4 * (l / 16) + j, j = 0..3.
// SWIGLU: the weight holds gate columns [0, n/2) and up columns [n/2, n); the block multiplies the
// gate tile blockIdx.x and the up tile of the same columns and writes act = silu(gate) * up
// ([m, n/2] f32) plus the block's per-row absmax, so that the next quantizer needs no pass over gate|up.
// ROPE (mode 2): the weight is the fused q | k | v projection; the block multiplies tile a and tile
// a + head_dim/32 of one head, i.e. the two halves that the rotation pairs, rotates q and k heads by the
// row's position (products rounded separately, no contraction), rounds once to bf16 and stores q rows
// and the new K / V cache rows directly, so the f32 projection never reaches memory.
// PRO != 0 (at most four rows, eight wavefronts): the block makes its own activation codes from `pro` behind its first
// weight loads (row_prologue.hpp: 1 RMSNorm + quantizer, 2 quantizer from partial maxima) and reads the activation
// operand from LDS; xq_tiled is not read.
template <int MT, int NTW, int NWAVES, int MODE, int PRO = 0>
__global__ void __launch_bounds__(NWAVES * 64)
    w8a8_skinny_kernel(const int8_t *__restrict__ xq_tiled, const int8_t *__restrict__ w_tiles, uint32_t m,
                       uint32_t n, uint32_t n_tiles, uint32_t k_tiles, EpiI8 ep, RowPrologue pro) {
    constexpr bool SWIGLU = MODE == kEpiSwiglu, ROPE = MODE == kEpiRope;
    static_assert(MODE == kEpiPlain || NTW == 2, "the fused epilogues pair two tiles");
    static_assert(PRO == 0 || (MT == 1 && NWAVES * 64 == kPrologueThreads), "row prologues: one row tile, 512 threads");
    constexpr int NACC = MT * NTW * 4;
    __shared__ int red[NWAVES][NACC][64];
    extern __shared__ __attribute__((aligned(16))) int8_t pro_codes[];      // PRO: [m][k] activation codes
    __shared__ float pro_sx[PRO ? kPrologueMaxRows : 1], pro_f[PRO ? 16 : 1];
    __shared__ double pro_d[PRO ? 16 : 1];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const uint32_t half_tiles = ROPE ? ep.head_dim / 32 : 0;
    const uint32_t nt0 = SWIGLU ? blockIdx.x
                         : ROPE ? (blockIdx.x / half_tiles) * 2 * half_tiles + blockIdx.x % half_tiles
                                : blockIdx.x * NTW;
    const uint32_t nt_step = SWIGLU ? n_tiles / 2 : ROPE ? half_tiles : 1;

    v4i acc[MT][NTW];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NTW; ++j) acc[i][j] = v4i{0, 0, 0, 0};

    const int8_t *b_base = w_tiles + (uint64_t)lane * 16;
    // Wavefront w owns the k-tiles w, w + NWAVES, ...: `cnt` of them.  They are streamed through a ring of
    // D register slots (one slot = the weight tiles and the activation tiles of one k-tile): the loads of a
    // whole group of D k-tiles are in flight while the group before it is multiplied, and every multiply
    // is followed at once by the load that refills its slot, so the memory pipe never drains between trips.
    // (A weight tile comes from HBM and takes several times longer than an activation tile from L2; with
    // few loads in flight the whole stream runs at in-flight bytes / HBM latency.)  Loads past the end are
    // clamped to the wavefront's last k-tile instead of predicated, which keeps the number of outstanding
    // loads the same on every path, so the waits the compiler inserts are exact.
    constexpr int D = (MT * NTW >= 6) ? 4 : 8;
    const uint32_t cnt = k_tiles > (uint32_t)wave ? (k_tiles - wave + NWAVES - 1) / NWAVES : 0;
    // lane l holds row l % 16 of a row tile.  The lanes of rows at or past m fetch row 0 of their k-group
    // instead (bytes that its own lane fetches anyway), so a step of one to four rows pulls a quarter of
    // each activation tile; what they hold only reaches accumulator rows that are never stored.  (A load
    // skipped by predicate would make the count of outstanding loads depend on m.)
    uint32_t a_off[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) a_off[i] = ixm::decode_a_lane_byte((uint32_t)i, (uint32_t)lane, m);
    // What the epilogue needs from memory (scales, bias, residual, rotation, cache slot) is requested here,
    // ahead of the weight stream: asked for after the reduction it would cost the kernel one more memory
    // round trip with nothing else in flight.  Item q of this wavefront is accumulator wave + q * NWAVES
    // (plain) or row group wave + q * NWAVES of both tiles (fused epilogues).
    constexpr int NE = ((MODE == kEpiPlain ? NACC : MT * 4) + NWAVES - 1) / NWAVES;
    float p_sx[NE], p_sw0[NE], p_sw1[NE], p_x0[NE], p_x1[NE];
    uint32_t p_slot[NE];
#pragma unroll
    for (int q = 0; q < NE; ++q) {
        p_sx[q] = p_sw0[q] = p_sw1[q] = p_x0[q] = p_x1[q] = 0.0f;
        p_slot[q] = 0xffffffffu;
        const int idx = wave + q * NWAVES;
        if constexpr (MODE == kEpiPlain) {
            const int e = idx % 4, j = (idx / 4) % NTW, i = idx / (4 * NTW);
            const uint32_t row = i * 16 + 4 * (lane / 16) + e, col = (nt0 + j) * 16 + lane % 16;
            if (idx < NACC && row < m && col < n) {
                if constexpr (PRO == 0) p_sx[q] = ep.sx[row];
                p_sw0[q] = ep.sw[col];
                if (ep.bias) p_x0[q] = ep.bias[col];
                if (ep.residual) p_x1[q] = ep.residual[(uint64_t)row * n + col];
            }
        } else {
            const int i = idx / 4, e = idx % 4;
            const uint32_t row = i * 16 + 4 * (lane / 16) + e, col = nt0 * 16 + lane % 16;
            const uint32_t pair = SWIGLU ? n / 2 : ep.head_dim / 2;      // distance to the partner column
            if (idx < MT * 4 && row < m && col + pair < n) {
                if constexpr (PRO == 0) p_sx[q] = ep.sx[row];
                p_sw0[q] = ep.sw[col];
                p_sw1[q] = ep.sw[col + pair];
                if constexpr (ROPE) {
                    const uint32_t h = col / ep.head_dim, d = col % ep.head_dim;
                    if (h < ep.heads + ep.kv_heads) {
                        p_x0[q] = ep.cos_sin[(uint64_t)row * ep.head_dim + d];
                        p_x1[q] = ep.cos_sin[(uint64_t)row * ep.head_dim + pair + d];
                    }
                    if (h >= ep.heads) p_slot[q] = ep.slots[row];
                }
            }
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    v4i a[D][MT], b[D][NTW];
    // PRO: lane (g, r) reads k-group g of row r of the block's own codes; rows at or past m read row 0 (never stored)
    const uint32_t pro_off = ((uint32_t)lane % 16 < m ? (uint32_t)lane % 16 : 0u) * (k_tiles * 64) + ((uint32_t)lane / 16) * 16;
    auto load_b = [&](int s, uint32_t it) {
        const uint32_t kt = wave + (it < cnt ? it : cnt - 1) * NWAVES;
#pragma unroll
        for (int j = 0; j < NTW; ++j) {
            uint32_t nt = nt0 + j * nt_step;
            nt = nt < n_tiles ? nt : n_tiles - 1;            // a tile past the edge is loaded clamped, never stored
            b[s][j] = stream_load<true>((const v4i *)(b_base + ((uint64_t)nt * k_tiles + kt) * 1024));
        }
    };
    auto load_a = [&](int s, uint32_t it) {
        const uint32_t kt = wave + (it < cnt ? it : cnt - 1) * NWAVES;
        if constexpr (PRO != 0) {
            a[s][0] = *(const v4i *)(pro_codes + pro_off + kt * 64);
        } else {
#pragma unroll
            for (int i = 0; i < MT; ++i) a[s][i] = *(const v4i *)(xq_tiled + ((uint64_t)ixm::decode_a_tile((uint32_t)i, m) * k_tiles + kt) * 1024 + a_off[i]);
        }
    };
    auto load_slot = [&](int s, uint32_t it) {
        load_b(s, it);
        load_a(s, it);
    };
    auto mma_slot = [&](int s) {
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NTW; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[s][i], b[s][j], acc[i][j], 0, 0, 0);
    };
    if constexpr (PRO != 0) {
        // the rows are requested first, the first weight tiles behind them: the row work runs while the tiles travel
        typename std::conditional<PRO == 1, NormRows, PmaxRows>::type rows;
        if constexpr (PRO == 1) prologue_norm_load(pro, m, k_tiles * 64, rows);
        else prologue_pmax_load(pro, m, k_tiles * 64, rows);
        __builtin_amdgcn_sched_barrier(0);
        if (cnt != 0) {
#pragma unroll
            for (int s = 0; s < D; ++s) load_b(s, (uint32_t)s);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (PRO == 1) prologue_rmsnorm_quantize(pro, rows, m, k_tiles * 64, pro_codes, pro_sx, pro_d, pro_f);
        else prologue_quantize_from_pmax(pro, rows, m, k_tiles * 64, pro_codes, pro_sx, pro_f);
        prologue_publish(pro, m, k_tiles * 64, pro_codes, pro_sx);
#pragma unroll
        for (int q = 0; q < NE; ++q) {
            const int idx = wave + q * NWAVES;
            const uint32_t row = (uint32_t)(4 * (lane / 16) + idx % 4);      // one row tile: element idx % 4 of the lane
            p_sx[q] = row < m ? pro_sx[row] : 0.0f;
        }
        if (cnt != 0) {
#pragma unroll
            for (int s = 0; s < D; ++s) load_a(s, (uint32_t)s);
        }
    }
    if (cnt != 0) {
        if constexpr (PRO == 0) {
#pragma unroll
            for (int s = 0; s < D; ++s) load_slot(s, (uint32_t)s);
        }
        uint32_t it0 = 0;
        for (; it0 + D < cnt; it0 += D) {                     // a further group exists: refill while multiplying
#pragma unroll
            for (int s = 0; s < D; ++s) {
                mma_slot(s);
                __builtin_amdgcn_sched_barrier(0);            // keep every refill right behind its consumer
                load_slot(s, it0 + D + s);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int s = 0; s < D; ++s)
            if (it0 + s < cnt) mma_slot(s);
    }

#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NTW; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[wave][(i * NTW + j) * 4 + e][lane] = acc[i][j][e];
    __syncthreads();

    if constexpr (SWIGLU) {
        const uint32_t f = n / 2;
#pragma unroll
        for (int pq = 0; pq < NE; ++pq) {
            const int q = wave + pq * NWAVES;
            if (q >= MT * 4) break;
            int i = q / 4, e = q % 4;
            int sg = 0, su = 0;
#pragma unroll
            for (int w = 0; w < NWAVES; ++w) {
                sg += red[w][(i * 2 + 0) * 4 + e][lane];
                su += red[w][(i * 2 + 1) * 4 + e][lane];
            }
            uint32_t row = i * 16 + 4 * (lane / 16) + e;
            uint32_t col = nt0 * 16 + lane % 16;
            float a = 0.0f;
            if (row < m && col < f) {
                float vg = __fmul_rn((float)sg, __fmul_rn(p_sx[pq], p_sw0[pq]));
                float vu = __fmul_rn((float)su, __fmul_rn(p_sx[pq], p_sw1[pq]));
                float act = silu_f32(vg) * vu;
                ((float *)ep.out)[(uint64_t)row * f + col] = act;
                a = fabsf(act);
            }
            // absmax over the 16 columns of the tile (lanes sharing lane / 16)
#pragma unroll
            for (int off = 1; off < 16; off <<= 1) a = fmaxf(a, __shfl_xor(a, off, 64));
            if (lane % 16 == 0 && row < m) ep.pmax[(uint64_t)row * (n_tiles / 2) + nt0] = a;
        }
        return;
    }
    if constexpr (ROPE) {
        const uint32_t half = ep.head_dim / 2;
        const uint32_t eq = ep.heads * ep.head_dim, ekv = ep.kv_heads * ep.head_dim;
#pragma unroll
        for (int pq = 0; pq < NE; ++pq) {
            const int q = wave + pq * NWAVES;
            if (q >= MT * 4) break;
            int i = q / 4, e = q % 4;
            int s0 = 0, s1 = 0;
#pragma unroll
            for (int w = 0; w < NWAVES; ++w) {
                s0 += red[w][(i * 2 + 0) * 4 + e][lane];
                s1 += red[w][(i * 2 + 1) * 4 + e][lane];
            }
            const uint32_t row = i * 16 + 4 * (lane / 16) + e;
            const uint32_t col = nt0 * 16 + lane % 16;             // first half of the head; partner at col + half
            if (row < m && col + half < n) {
                float x0 = __fmul_rn((float)s0, __fmul_rn(p_sx[pq], p_sw0[pq]));
                float x1 = __fmul_rn((float)s1, __fmul_rn(p_sx[pq], p_sw1[pq]));
                const uint32_t h = col / ep.head_dim, d = col % ep.head_dim;
                uint16_t *dst = nullptr;
                if (h < ep.heads) {
                    dst = ep.q_out + (uint64_t)row * eq + (uint64_t)h * ep.head_dim + d;
                } else {
                    const uint64_t slot = p_slot[pq];
                    if (slot < ep.pool_rows) {
                        const uint32_t hk = h - ep.heads;
                        dst = (hk < ep.kv_heads ? ep.k_pool + slot * ekv + (uint64_t)hk * ep.head_dim
                                                : ep.v_pool + slot * ekv + (uint64_t)(hk - ep.kv_heads) * ep.head_dim) + d;
                    }
                }
                if (h < ep.heads + ep.kv_heads) {
                    const float c = p_x0[pq], sn = p_x1[pq];
                    const float r0 = __fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, sn));
                    const float r1 = __fadd_rn(__fmul_rn(x1, c), __fmul_rn(x0, sn));
                    x0 = r0;
                    x1 = r1;
                }
                if (dst) {
                    dst[0] = f32_to_bf16(x0);
                    dst[half] = f32_to_bf16(x1);
                }
            }
        }
        return;
    }
#pragma unroll
    for (int pq = 0; pq < NE; ++pq) {
        const int idx = wave + pq * NWAVES;
        if (idx >= NACC) break;
        int sum = 0;
#pragma unroll
        for (int w = 0; w < NWAVES; ++w) sum += red[w][idx][lane];
        int e = idx % 4, j = (idx / 4) % NTW, i = idx / (4 * NTW);
        uint32_t row = i * 16 + 4 * (lane / 16) + e;
        uint32_t col = (nt0 + j) * 16 + lane % 16;
        if (row < m && col < n) {
            uint64_t o = (uint64_t)row * n + col;
            if (ep.acc_out) ep.acc_out[o] = sum;
            float s = __fmul_rn(p_sx[pq], p_sw0[pq]);
            float v = __fmul_rn((float)sum, s);
            if (ep.bias) v = __fadd_rn(v, p_x0[pq]);
            if (ep.residual) v = __fadd_rn(p_x1[pq], v);
            if (ep.out_bf16)
                ((uint16_t *)ep.out)[o] = f32_to_bf16(v);
            else
                ((float *)ep.out)[o] = v;
        }
    }
}

// Stores that the compiler's wait-count bookkeeping does not see.  On this target loads and stores share one
// counter (vmcnt) but complete out of order with respect to each other, so with a store pending the compiler turns
// every wait for a load into vmcnt(0): in a loop that keeps a ring of loads in flight and stores results once per
// pass, every pass then starts by draining the ring.  Issued like this the stores still raise the hardware counter,
// which only makes a wait for "at most N loads outstanding" stricter than it had to be (loads complete in order
// among themselves), never laxer.  Nothing in the kernels that use them reads the stored locations back through
// the compiler's loads.  POLICY 0: plain, 1: sc0 (workgroup scope), 2: sc1 (agent scope).
template <int POLICY>
__device__ __forceinline__ void store_unseen_b32(void *p, uint32_t v) {
    if constexpr (POLICY == 0) asm volatile("global_store_dword %0, %1, off" : : "v"(p), "v"(v));
    else if constexpr (POLICY == 1) asm volatile("global_store_dword %0, %1, off sc0" : : "v"(p), "v"(v));
    else asm volatile("global_store_dword %0, %1, off sc1" : : "v"(p), "v"(v));
}
// (a store of more than 64 bits must not be followed at once by a write to its data registers; for its own store
// instructions the compiler keeps that distance, for these it cannot know: the s_nop keeps it)
template <int POLICY>
__device__ __forceinline__ void store_unseen_b128(void *p, v4i v) {
    if constexpr (POLICY == 0) asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" : : "v"(p), "v"(v));
    else if constexpr (POLICY == 1) asm volatile("global_store_dwordx4 %0, %1, off sc0\n\ts_nop 1" : : "v"(p), "v"(v));
    else asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v));
}
__device__ __forceinline__ void store_unseen_b16(void *p, uint32_t v) {
    asm volatile("global_store_short %0, %1, off" : : "v"(p), "v"(v));
}

// ------------------------------------------------- W8A8, weight stationary (a few hundred rows)
// Between the decode shapes (at most 64 rows, kernels above) and the tiled GEMMs (which need a few hundred output
// tiles to fill the device): a prompt of 65 to a few hundred tokens against a weight with about one column tile per
// compute unit.  A block owns NTW column tiles for all rows.  Its eight wavefronts divide k as above, but every
// wavefront loads the weight tiles of its k-tiles once and keeps them in registers for the whole kernel; the
// rows then pass by in groups of 64: the wavefront streams the activation tiles of its k-tiles for the group
// (a ring of four k-tiles, refilled behind every multiply, running on into the next group), the eight partial
// tiles meet in LDS and are finished exactly as in the kernel above.  The weight leaves HBM once, an activation
// byte is read from L2 once per block, and once the weights are in, nothing a wavefront loads comes from HBM, so
// no L2 hit waits behind a miss.  k_tiles <= 8 KTW; the tiled activation layout of the decode kernels.
// ROPE (two column tiles): the weight is the fused q | k | v projection and the block's tiles are the two halves of a head
// that the rotation pairs (tile a and tile a + head_dim / 32, as in w8a8_skinny_kernel's mode of that name); the epilogue
// rotates q and k heads by the row's position, rounds once to bf16 and stores q rows and the new K / V cache rows, with
// rope_append's expressions, so the f32 projection never reaches memory and the rotation costs no launch.
template <int KTW, int NTW, bool ROPE = false>
__global__ void __launch_bounds__(512)
    w8a8_wstat_kernel(const int8_t *__restrict__ xq_tiled, const int8_t *__restrict__ w_tiles, uint32_t m, uint32_t n,
                      uint32_t n_tiles, uint32_t k_tiles, EpiI8 ep) {
    constexpr int NW = 8, MT = 4, NACC = MT * NTW * 4, DS = 4;
    static_assert(KTW % DS == 0, "the ring restarts at slot 0 with every row group");
    static_assert(!ROPE || NTW == 2, "the rotation pairs two tiles");
    __shared__ int red[NW][NACC][64];
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const uint32_t half_tiles = ROPE ? ep.head_dim / 32 : 0;
    const uint32_t nt0 = ROPE ? (blockIdx.x / half_tiles) * 2 * half_tiles + blockIdx.x % half_tiles : blockIdx.x * NTW;
    const uint32_t nt_step = ROPE ? half_tiles : 1;
    const uint32_t cnt = k_tiles > (uint32_t)wave ? (k_tiles - wave + NW - 1) / NW : 0;      // k-tiles of this wavefront
    const uint32_t row_tiles = (m + 15) / 16, groups = (row_tiles + MT - 1) / MT;

    // the weights of this wavefront's k-tiles; past its last one zeros, so that every step multiplies and the row
    // loop below is straight-line code (the compiler then counts the loads of the activation ring exactly)
    v4i w[KTW][NTW];
#pragma unroll
    for (int t = 0; t < KTW; ++t) {
        const uint32_t kt = wave + ((uint32_t)t < cnt ? (uint32_t)t : (cnt ? cnt - 1 : 0)) * NW;
#pragma unroll
        for (int j = 0; j < NTW; ++j) {
            uint32_t nt = nt0 + j * nt_step;
            nt = nt < n_tiles ? nt : n_tiles - 1;
            const v4i x = stream_load<true>((const v4i *)(w_tiles + ((uint64_t)nt * k_tiles + (kt < k_tiles ? kt : 0)) * 1024 + (uint64_t)lane * 16));
            w[t][j] = (uint32_t)t < cnt ? x : v4i{0, 0, 0, 0};
        }
    }
    // channel scale and bias of the accumulator elements this wavefront finishes (item q = element wave + 8 q)
    constexpr int NE = NACC / NW;
    float p_sw[NE], p_bias[NE];
#pragma unroll
    for (int q = 0; q < NE; ++q) {
        const int idx = wave + q * NW, j = (idx / 4) % NTW;
        const uint32_t col = (nt0 + j * nt_step) * 16 + lane % 16;
        p_sw[q] = col < n ? ep.sw[col] : 0.0f;
        p_bias[q] = (!ROPE && ep.bias && col < n) ? ep.bias[col] : 0.0f;
    }
    // ROPE: the wavefront finishes pairs instead: pair q = (row tile, element) wave + 8 q of both tiles; the first tile's
    // column, its head and dim, and the channel scales of the two halves
    constexpr int NP = ROPE ? MT * 4 / NW : 1;
    const uint32_t r_col = nt0 * 16 + lane % 16, r_half = ROPE ? ep.head_dim / 2 : 0;
    const uint32_t r_head = ROPE ? r_col / ep.head_dim : 0, r_dim = ROPE ? r_col % ep.head_dim : 0;
    const bool r_live = ROPE && r_col + r_half < n;
    const float r_sw0 = r_live ? ep.sw[r_col] : 0.0f, r_sw1 = r_live ? ep.sw[r_col + r_half] : 0.0f;
    __builtin_amdgcn_sched_barrier(0);

    // step (g, t): the MT activation tiles of k-tile t of this wavefront for row group g; row tiles past the last
    // one repeat it (their sums are never stored)
    v4i a[DS][MT];
    auto load_step = [&](int slot, uint32_t g, int t) {
        const uint32_t kt = wave + ((uint32_t)t < cnt ? (uint32_t)t : (cnt ? cnt - 1 : 0)) * NW;
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            uint32_t rt = g * MT + i;
            rt = rt < row_tiles ? rt : row_tiles - 1;
            a[slot][i] = *(const v4i *)(xq_tiled + ((uint64_t)rt * k_tiles + (kt < k_tiles ? kt : 0)) * 1024 + (uint64_t)lane * 16);
        }
    };
#pragma unroll
    for (int t = 0; t < DS; ++t) load_step(t, 0, t);
    for (uint32_t g = 0; g < groups; ++g) {
        // what the epilogue of this group needs, asked for ahead of its multiplies
        float p_sx[NE], p_res[NE];
        float r_sx[NP], r_cos[NP], r_sin[NP];
        uint32_t r_slot[NP];
        if constexpr (ROPE) {
#pragma unroll
            for (int q = 0; q < NP; ++q) {
                const int idx = wave + q * NW;
                const uint32_t row = (g * MT + idx / 4) * 16 + 4 * (lane / 16) + idx % 4;
                r_sx[q] = r_cos[q] = r_sin[q] = 0.0f;
                r_slot[q] = 0xffffffffu;
                if (row < m && r_live) {
                    r_sx[q] = ep.sx[row];
                    if (r_head < ep.heads + ep.kv_heads) {
                        r_cos[q] = ep.cos_sin[(uint64_t)row * ep.head_dim + r_dim];
                        r_sin[q] = ep.cos_sin[(uint64_t)row * ep.head_dim + r_half + r_dim];
                    }
                    if (r_head >= ep.heads) r_slot[q] = ep.slots[row];
                }
            }
        } else {
#pragma unroll
            for (int q = 0; q < NE; ++q) {
                const int idx = wave + q * NW, e = idx % 4, j = (idx / 4) % NTW, i = idx / (4 * NTW);
                const uint32_t row = (g * MT + i) * 16 + 4 * (lane / 16) + e, col = (nt0 + j) * 16 + lane % 16;
                const bool ok = row < m && col < n;
                p_sx[q] = ok ? ep.sx[row] : 0.0f;
                p_res[q] = (ok && ep.residual) ? ep.residual[(uint64_t)row * n + col] : 0.0f;
            }
        }
        v4i acc[MT][NTW];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NTW; ++j) acc[i][j] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < KTW; ++t) {
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NTW; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[t % DS][i], w[t][j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);                // the refill right behind its consumer
            if (t + DS < KTW) load_step(t % DS, g, t + DS);
            else load_step(t % DS, g + 1 < groups ? g + 1 : g, t + DS - KTW);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();                                      // everybody has read the sums of the group before
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NTW; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) red[wave][(i * NTW + j) * 4 + e][lane] = acc[i][j][e];
        __syncthreads();
        if constexpr (ROPE) {
            const uint32_t eq = ep.heads * ep.head_dim, ekv = ep.kv_heads * ep.head_dim;
#pragma unroll
            for (int q = 0; q < NP; ++q) {
                const int idx = wave + q * NW, i = idx / 4, e = idx % 4;
                int s0 = 0, s1 = 0;
#pragma unroll
                for (int ww = 0; ww < NW; ++ww) {
                    s0 += red[ww][(i * 2 + 0) * 4 + e][lane];
                    s1 += red[ww][(i * 2 + 1) * 4 + e][lane];
                }
                const uint32_t row = (g * MT + i) * 16 + 4 * (lane / 16) + e;
                if (row < m && r_live) {
                    float x0 = __fmul_rn((float)s0, __fmul_rn(r_sx[q], r_sw0));
                    float x1 = __fmul_rn((float)s1, __fmul_rn(r_sx[q], r_sw1));
                    uint16_t *dst = nullptr;
                    if (r_head < ep.heads) {
                        dst = ep.q_out + (uint64_t)row * eq + (uint64_t)r_head * ep.head_dim + r_dim;
                    } else {
                        const uint64_t slot = r_slot[q];
                        if (slot < ep.pool_rows) {
                            const uint32_t hk = r_head - ep.heads;
                            dst = (hk < ep.kv_heads ? ep.k_pool + slot * ekv + (uint64_t)hk * ep.head_dim
                                                    : ep.v_pool + slot * ekv + (uint64_t)(hk - ep.kv_heads) * ep.head_dim) + r_dim;
                        }
                    }
                    if (r_head < ep.heads + ep.kv_heads) {
                        const float r0 = __fsub_rn(__fmul_rn(x0, r_cos[q]), __fmul_rn(x1, r_sin[q]));
                        const float r1 = __fadd_rn(__fmul_rn(x1, r_cos[q]), __fmul_rn(x0, r_sin[q]));
                        x0 = r0;
                        x1 = r1;
                    }
                    if (dst) {
                        store_unseen_b16(dst, f32_to_bf16(x0));
                        store_unseen_b16(dst + r_half, f32_to_bf16(x1));
                    }
                }
            }
            continue;
        }
#pragma unroll
        for (int q = 0; q < NE; ++q) {
            const int idx = wave + q * NW;
            int sum = 0;
#pragma unroll
            for (int ww = 0; ww < NW; ++ww) sum += red[ww][idx][lane];
            const int e = idx % 4, j = (idx / 4) % NTW, i = idx / (4 * NTW);
            const uint32_t row = (g * MT + i) * 16 + 4 * (lane / 16) + e, col = (nt0 + j) * 16 + lane % 16;
            if (row < m && col < n) {
                const uint64_t o = (uint64_t)row * n + col;
                if (ep.acc_out) store_unseen_b32<0>(ep.acc_out + o, (uint32_t)sum);
                float v = __fmul_rn((float)sum, __fmul_rn(p_sx[q], p_sw[q]));
                if (ep.bias) v = __fadd_rn(v, p_bias[q]);
                if (ep.residual) v = __fadd_rn(p_res[q], v);
                if (ep.out_bf16)
                    store_unseen_b16((uint16_t *)ep.out + o, f32_to_bf16(v));
                else
                    store_unseen_b32<0>((float *)ep.out + o, __float_as_uint(v));
            }
        }
    }
}

// ------------------------------------------------- W8A8, activation stationary
// For weights with many more column tiles than the chip has compute units: the
// kernel above re-reads the activation tiles (m x k, twice the bytes of a weight
// tile at m = 32) once per block from L2, and L2 delivers little more than HBM on
// this part, so those re-reads cost as much as the weight stream itself.  Here a
// block of eight wavefronts keeps its activations in registers for its whole life:
// wavefront w owns the k-tiles w, w + 8, ... (at most KTW of them) and walks the
// block's units (pairs of column tiles: b, b + gridDim, ...) streaming only weight
// tiles, one unit ahead in a second register set.  The eight partial tiles of a unit
// meet in LDS (two buffers, one barrier per unit) and wavefront w finishes the rows
// 4 (l / 16) + w % 4 of row tile w / 4 for both tiles of the unit, so SwiGLU has
// gate and up of an element in the same lane.
// PRO == 1 (at most four rows): the block makes its own activation codes (RMSNorm + quantizer of `pro`, see
// row_prologue.hpp) behind the weight loads of its first unit and takes its activation registers from LDS.
template <int MT, int KTW, int MODE, int PRO = 0>
__global__ void __launch_bounds__(512)
    w8a8_astat_kernel(const int8_t *__restrict__ xq_tiled, const int8_t *__restrict__ w_tiles, uint32_t m, uint32_t n,
                      uint32_t n_tiles, uint32_t k_tiles, uint32_t n_units, EpiI8 ep, RowPrologue pro) {
    constexpr bool SWIGLU = MODE == kEpiSwiglu;
    constexpr int NW = 8, NACC = MT * 2 * 4;
    static_assert(PRO == 0 || (PRO == 1 && MT == 1), "row prologue: norm + quantizer, one row tile");
    __shared__ int red[2][NW][NACC][64];
    extern __shared__ __attribute__((aligned(16))) int8_t pro_codes[];      // PRO: [m][k] activation codes
    __shared__ float pro_sx[PRO ? kPrologueMaxRows : 1], pro_f[PRO ? 16 : 1];
    __shared__ double pro_d[PRO ? 16 : 1];
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const uint32_t last_kt = k_tiles - 1, last_tile = n_tiles - 1;

    // activations of this wavefront's k-tiles (clamped repeats past the end are never multiplied)
    v4i a[KTW][MT];
    if constexpr (PRO == 0) {
#pragma unroll
        for (int t = 0; t < KTW; ++t) {
            uint32_t kt = wave + NW * t;
            kt = kt < k_tiles ? kt : last_kt;
#pragma unroll
            for (int i = 0; i < MT; ++i)
                a[t][i] = *(const v4i *)(xq_tiled + ((uint64_t)i * k_tiles + kt) * 1024 + (uint64_t)lane * 16);
        }
    }
    auto tile_of = [&](uint32_t u, int j) -> uint32_t {
        uint32_t nt = SWIGLU ? u + j * (n_tiles / 2) : 2 * u + j;
        return nt < last_tile ? nt : last_tile;
    };
    // What the epilogue of a unit needs from memory travels with the unit's weights (requested first, so it
    // is there before them): asked for after the reduction, these loads would queue behind the next unit's
    // weight tiles, which are already in flight then, and the epilogue would wait for all of them.
    // Wavefront w < 4 MT finishes rows 4 (l / 16) + w % 4 of row tile w / 4: its activation scale is fixed.
    struct UnitEpi {
        float sw[2], bias[2], res[2];
    };
    const uint32_t e_row = (wave / 4) * 16 + 4 * (lane / 16) + wave % 4;
    const bool e_wave = wave < MT * 4 && e_row < m;
    float e_sx = (PRO == 0 && e_wave) ? ep.sx[e_row] : 0.0f;
    auto load_unit = [&](uint32_t u, v4i (&b)[KTW][2], UnitEpi &ue) {
        u = u < n_units ? u : n_units - 1;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            ue.sw[j] = ue.bias[j] = ue.res[j] = 0.0f;
            const uint32_t col = SWIGLU ? u * 16 + lane % 16 + j * (n / 2) : (2 * u + j) * 16 + lane % 16;
            if (e_wave && col < n) {
                ue.sw[j] = ep.sw[col];
                if constexpr (!SWIGLU) {
                    if (ep.bias) ue.bias[j] = ep.bias[col];
                    if (ep.residual) ue.res[j] = ep.residual[(uint64_t)e_row * n + col];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int8_t *base = w_tiles + (uint64_t)tile_of(u, j) * k_tiles * 1024 + (uint64_t)lane * 16;
#pragma unroll
            for (int t = 0; t < KTW; ++t) {
                uint32_t kt = wave + NW * t;
                kt = kt < k_tiles ? kt : last_kt;
                b[t][j] = stream_load<true>((const v4i *)(base + (uint64_t)kt * 1024));
            }
        }
    };
    auto finish_unit = [&](uint32_t u, const v4i (&b)[KTW][2], const UnitEpi &ue, int buf) {
        v4i acc[MT][2];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < KTW; ++t) {
            if ((uint32_t)(wave + NW * t) < k_tiles) {
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[t][i], b[t][j], acc[i][j], 0, 0, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) red[buf][wave][(i * 2 + j) * 4 + e][lane] = acc[i][j][e];
        __syncthreads();
        if (wave < MT * 4) {
            const int i = wave / 4, e = wave % 4;
            int s0 = 0, s1 = 0;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                s0 += red[buf][w][(i * 2 + 0) * 4 + e][lane];
                s1 += red[buf][w][(i * 2 + 1) * 4 + e][lane];
            }
            const uint32_t row = i * 16 + 4 * (lane / 16) + e;
            if constexpr (SWIGLU) {
                const uint32_t f = n / 2, col = u * 16 + lane % 16;
                float av = 0.0f;
                if (row < m && col < f) {
                    float vg = __fmul_rn((float)s0, __fmul_rn(e_sx, ue.sw[0]));
                    float vu = __fmul_rn((float)s1, __fmul_rn(e_sx, ue.sw[1]));
                    float act = silu_f32(vg) * vu;
                    ((float *)ep.out)[(uint64_t)row * f + col] = act;
                    av = fabsf(act);
                }
#pragma unroll
                for (int off = 1; off < 16; off <<= 1) av = fmaxf(av, __shfl_xor(av, off, 64));
                if (lane % 16 == 0 && row < m) ep.pmax[(uint64_t)row * (n_tiles / 2) + u] = av;
            } else {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const uint32_t col = (2 * u + j) * 16 + lane % 16;
                    const int sum = j ? s1 : s0;
                    if (row < m && col < n) {
                        uint64_t o = (uint64_t)row * n + col;
                        if (ep.acc_out) ep.acc_out[o] = sum;
                        float v = __fmul_rn((float)sum, __fmul_rn(e_sx, ue.sw[j]));
                        if (ep.bias) v = __fadd_rn(v, ue.bias[j]);
                        if (ep.residual) v = __fadd_rn(ue.res[j], v);
                        if (ep.out_bf16)
                            ((uint16_t *)ep.out)[o] = f32_to_bf16(v);
                        else
                            ((float *)ep.out)[o] = v;
                    }
                }
            }
        }
    };

    // two units per trip so that the two weight register sets have fixed names; buffer u % 2 of `red` is
    // rewritten two units later, after the barrier of the unit in between
    v4i b0[KTW][2], b1[KTW][2];
    UnitEpi ue0, ue1;
    uint32_t u = blockIdx.x;
    NormRows rows;
    if constexpr (PRO != 0) {
        // the rows are requested first, the first unit's weights behind them: the row work runs while they travel
        prologue_norm_load(pro, m, k_tiles * 64, rows);
        __builtin_amdgcn_sched_barrier(0);
    }
    load_unit(u, b0, ue0);
    if constexpr (PRO != 0) {
        __builtin_amdgcn_sched_barrier(0);
        prologue_rmsnorm_quantize(pro, rows, m, k_tiles * 64, pro_codes, pro_sx, pro_d, pro_f);
        prologue_publish(pro, m, k_tiles * 64, pro_codes, pro_sx);
        e_sx = e_wave ? pro_sx[e_row] : 0.0f;
        const uint32_t off = ((uint32_t)lane % 16 < m ? (uint32_t)lane % 16 : 0u) * (k_tiles * 64) + ((uint32_t)lane / 16) * 16;
#pragma unroll
        for (int t = 0; t < KTW; ++t) {
            uint32_t kt = wave + NW * t;
            kt = kt < k_tiles ? kt : last_kt;
            a[t][0] = *(const v4i *)(pro_codes + off + kt * 64);
        }
    }
    for (; u < n_units; u += 2 * gridDim.x) {
        load_unit(u + gridDim.x, b1, ue1);
        finish_unit(u, b0, ue0, 0);
        if (u + gridDim.x >= n_units) break;
        load_unit(u + 2 * gridDim.x, b0, ue0);
        finish_unit(u + gridDim.x, b1, ue1, 1);
    }
}

// The same for 33 to 64 rows (three or four row tiles).  The activations of four row tiles fill half of a wavefront's
// registers, so the weights have one register set instead of two: every k-tile's pair of weight tiles is multiplied
// and its registers are refilled at once with the same k-tile of the block's next unit, which keeps a whole unit of
// weight loads in flight all the time.  A wavefront finishes two of the 4 MT (row tile, element) items of a unit.
// The partial tiles of two units (2 x 8 wavefronts x 8 MT items x 256 bytes) live in dynamic LDS.
template <int MT, int MODE>
__global__ void __launch_bounds__(512)
    w8a8_astat_wide_kernel(const int8_t *__restrict__ xq_tiled, const int8_t *__restrict__ w_tiles, uint32_t m, uint32_t n,
                           uint32_t n_tiles, uint32_t k_tiles, uint32_t n_units, EpiI8 ep) {
    constexpr bool SWIGLU = MODE == kEpiSwiglu;
    constexpr int NW = 8, KTW = 8, NACC = MT * 2 * 4, NQ = (MT * 4 + NW - 1) / NW;
    static_assert(MT == 3 || MT == 4, "three or four row tiles; fewer take w8a8_astat_kernel");
    extern __shared__ __attribute__((aligned(16))) int red_wide[];          // [2][NW][NACC][64]
    auto red = [&](int buf, int w, int idx) -> int * { return red_wide + (((size_t)buf * NW + w) * NACC + idx) * 64; };
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const uint32_t last_kt = k_tiles - 1, last_tile = n_tiles - 1;

    // activations of this wavefront's k-tiles (clamped repeats past the end are never multiplied)
    v4i a[KTW][MT];
#pragma unroll
    for (int t = 0; t < KTW; ++t) {
        uint32_t kt = wave + NW * t;
        kt = kt < k_tiles ? kt : last_kt;
#pragma unroll
        for (int i = 0; i < MT; ++i)
            a[t][i] = *(const v4i *)(xq_tiled + ((uint64_t)ixm::decode_a_tile((uint32_t)i, m) * k_tiles + kt) * 1024 + (uint64_t)lane * 16);
    }
    auto tile_of = [&](uint32_t u, int j) -> uint32_t {
        uint32_t nt = SWIGLU ? u + j * (n_tiles / 2) : 2 * u + j;
        return nt < last_tile ? nt : last_tile;
    };
    // item q of this wavefront: element idx % 4 of row tile idx / 4, idx = wave + 8 q
    uint32_t e_row[NQ];
    bool e_ok[NQ];
    float e_sx[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        const int idx = wave + NW * q;
        e_row[q] = (uint32_t)(idx / 4) * 16 + 4 * ((uint32_t)lane / 16) + (uint32_t)(idx % 4);
        e_ok[q] = idx < MT * 4 && e_row[q] < m;
        e_sx[q] = e_ok[q] ? ep.sx[e_row[q]] : 0.0f;
    }
    struct UnitEpi {
        float sw[2], bias[2], res[NQ][2];
    };
    auto load_epi = [&](uint32_t u, UnitEpi &ue) {
        u = u < n_units ? u : n_units - 1;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            ue.sw[j] = ue.bias[j] = 0.0f;
            const uint32_t col = SWIGLU ? u * 16 + lane % 16 + j * (n / 2) : (2 * u + j) * 16 + lane % 16;
            if (col < n) {
                ue.sw[j] = ep.sw[col];
                if constexpr (!SWIGLU) {
                    if (ep.bias) ue.bias[j] = ep.bias[col];
                }
            }
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                ue.res[q][j] = 0.0f;
                if constexpr (!SWIGLU) {
                    if (ep.residual && e_ok[q] && col < n) ue.res[q][j] = ep.residual[(uint64_t)e_row[q] * n + col];
                }
            }
        }
    };
    v4i b[KTW][2];
    auto load_w = [&](uint32_t u, int t) {
        u = u < n_units ? u : n_units - 1;
        uint32_t kt = wave + NW * t;
        kt = kt < k_tiles ? kt : last_kt;
#pragma unroll
        for (int j = 0; j < 2; ++j)
            b[t][j] = stream_load<true>((const v4i *)(w_tiles + ((uint64_t)tile_of(u, j) * k_tiles + kt) * 1024 + (uint64_t)lane * 16));
    };

    UnitEpi ue;
    uint32_t u = blockIdx.x;
    load_epi(u, ue);
#pragma unroll
    for (int t = 0; t < KTW; ++t) load_w(u, t);
    for (int it = 0; u < n_units; u += gridDim.x, ++it) {
        const int buf = it & 1;
        UnitEpi ue_next;
        load_epi(u + gridDim.x, ue_next);
        v4i acc[MT][2];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < KTW; ++t) {
            if ((uint32_t)(wave + NW * t) < k_tiles) {
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[t][i], b[t][j], acc[i][j], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);                // the refill right behind its consumer
            load_w(u + gridDim.x, t);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) red(buf, wave, (i * 2 + j) * 4 + e)[lane] = acc[i][j][e];
        __syncthreads();      // buffer buf is rewritten two units later, behind the barrier of the unit in between
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int idx = wave + NW * q;
            if (idx >= MT * 4) break;
            const int i = idx / 4, e = idx % 4;
            int s0 = 0, s1 = 0;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                s0 += red(buf, w, (i * 2 + 0) * 4 + e)[lane];
                s1 += red(buf, w, (i * 2 + 1) * 4 + e)[lane];
            }
            const uint32_t row = e_row[q];
            if constexpr (SWIGLU) {
                const uint32_t f = n / 2, col = u * 16 + lane % 16;
                float av = 0.0f;
                if (row < m && col < f) {
                    float vg = __fmul_rn((float)s0, __fmul_rn(e_sx[q], ue.sw[0]));
                    float vu = __fmul_rn((float)s1, __fmul_rn(e_sx[q], ue.sw[1]));
                    float act = silu_f32(vg) * vu;
                    ((float *)ep.out)[(uint64_t)row * f + col] = act;
                    av = fabsf(act);
                }
#pragma unroll
                for (int off = 1; off < 16; off <<= 1) av = fmaxf(av, __shfl_xor(av, off, 64));
                if (lane % 16 == 0 && row < m) ep.pmax[(uint64_t)row * (n_tiles / 2) + u] = av;
            } else {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const uint32_t col = (2 * u + j) * 16 + lane % 16;
                    const int sum = j ? s1 : s0;
                    if (row < m && col < n) {
                        uint64_t o = (uint64_t)row * n + col;
                        if (ep.acc_out) ep.acc_out[o] = sum;
                        float v = __fmul_rn((float)sum, __fmul_rn(e_sx[q], ue.sw[j]));
                        if (ep.bias) v = __fadd_rn(v, ue.bias[j]);
                        if (ep.residual) v = __fadd_rn(ue.res[q][j], v);
                        if (ep.out_bf16)
                            ((uint16_t *)ep.out)[o] = f32_to_bf16(v);
                        else
                            ((float *)ep.out)[o] = v;
                    }
                }
            }
        }
        ue = ue_next;
    }
}

// ----------------------------------------------------------------- W8A16
// Two exact int8 -> bf16 conversions packed into one dword (low half first).
__device__ __forceinline__ uint32_t pack_i8x2_bf16(int lo, int hi) {
    uint32_t fl = __float_as_uint((float)lo), fh = __float_as_uint((float)hi);
    // upper halves of both floats in one v_perm_b32; |v| <= 128 fits bf16 exactly, so truncation is exact
    return __builtin_amdgcn_perm(fh, fl, 0x07060302u);
}
__device__ __forceinline__ void cvt_i8x8_bf16(uint32_t w0, uint32_t w1, v8bf *out) {
    v4u r;
    r[0] = pack_i8x2_bf16((int)(int8_t)(w0), (int)(int8_t)(w0 >> 8));
    r[1] = pack_i8x2_bf16((int)(int8_t)(w0 >> 16), (int)(int8_t)(w0 >> 24));
    r[2] = pack_i8x2_bf16((int)(int8_t)(w1), (int)(int8_t)(w1 >> 8));
    r[3] = pack_i8x2_bf16((int)(int8_t)(w1 >> 16), (int)(int8_t)(w1 >> 24));
    *out = __builtin_bit_cast(v8bf, r);
}

// out[m, n] = (sum_k a[m, k] * (float)w[k, n]) * sw[n] on v_mfma_f32_16x16x32_bf16.
// A lane's 16 weight bytes are k = 64*kt + 16*g + 0..15; the first eight feed
// one instruction, the last eight the next, and the activation operand uses the
// same split, so the two instructions together cover the tile's 64 k-values.
// RING: the k-tiles go through a ring of register slots (below); otherwise groups of D k-tiles are loaded,
// waited for and multiplied in turn.  The ring is the faster form while a wavefront's share of k fits a few
// groups (k = 4096: 10.4 against 11.2 us at 12288 columns and one row); with a deep k and eight or more rows
// the group form is (k = 11008, 32 rows: 24.1 against 25.6 us), so the launcher picks by k.
template <int MT, int NTW, int NWAVES, bool RING>
__global__ void __launch_bounds__(NWAVES * 64)
    w8a16_skinny_kernel(const uint16_t *__restrict__ a, const int8_t *__restrict__ w_tiles,
                        const float *__restrict__ sw, uint32_t m, uint32_t n, uint32_t n_tiles, uint32_t k_tiles,
                        void *__restrict__ out, int out_bf16) {
    constexpr int NACC = MT * NTW * 4;
    __shared__ float red[NWAVES][NACC][64];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int g = lane / 16, r = lane % 16;
    const uint32_t nt0 = blockIdx.x * NTW;
    const uint64_t k = (uint64_t)k_tiles * 64;

    v4f acc[MT][NTW];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NTW; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    const int8_t *b_base = w_tiles + (uint64_t)lane * 16;
    const uint32_t cnt = k_tiles > (uint32_t)wave ? (k_tiles - wave + NWAVES - 1) / NWAVES : 0;
    // the channel scales of the epilogue are requested ahead of the weight stream (see w8a8_skinny_kernel)
    constexpr int NE = (NACC + NWAVES - 1) / NWAVES;
    float p_sw[NE];
#pragma unroll
    for (int q = 0; q < NE; ++q) {
        const int idx = wave + q * NWAVES;
        const uint32_t col = (nt0 + (idx / 4) % NTW) * 16 + r;
        p_sw[q] = idx < NACC && col < n ? sw[col] : 0.0f;
    }
    __builtin_amdgcn_sched_barrier(0);
    // A ring of D register slots (the weight tiles and the activation tiles of one k-tile each), refilled
    // behind every multiply, as in w8a8_skinny_kernel: the loads of D k-tiles stay in flight throughout.
    // Loads past the wavefront's last k-tile repeat it (never multiplied) and column tiles past the edge repeat
    // the last one (never stored), so the count of outstanding loads is the same on every path; lanes of rows
    // at or past m read row 0 of their k-group, bytes that its own lane fetches anyway.
    // (D = 8 only where the slots leave the kernel at 128 registers, i.e. two blocks per compute unit)
    constexpr int D = (MT * NTW >= 2) ? 4 : 8;
    const uint32_t last_tile = n_tiles - 1;
    uint32_t a_row[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) a_row[i] = (uint32_t)i * 16 + r < m ? (uint32_t)i * 16 + r : 0u;
    v4u braw[D][NTW], lo[D][MT], hi[D][MT];
    auto load_slot = [&](int s_, uint32_t it) {
        const uint32_t kt = wave + (it < cnt ? it : cnt - 1) * NWAVES;
#pragma unroll
        for (int j = 0; j < NTW; ++j) {
            uint32_t nt = nt0 + j;
            nt = nt < last_tile ? nt : last_tile;
            braw[s_][j] = stream_load<true>((const v4u *)(b_base + ((uint64_t)nt * k_tiles + kt) * 1024));
        }
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const v4u *p = (const v4u *)(a + (uint64_t)a_row[i] * k + (uint64_t)kt * 64 + g * 16);
            lo[s_][i] = p[0];
            hi[s_][i] = p[1];
        }
    };
    auto mma_slot = [&](int s_) {
#pragma unroll
        for (int j = 0; j < NTW; ++j) {
            v8bf blo, bhi;
            cvt_i8x8_bf16(braw[s_][j][0], braw[s_][j][1], &blo);
            cvt_i8x8_bf16(braw[s_][j][2], braw[s_][j][3], &bhi);
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, lo[s_][i]), blo, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, hi[s_][i]), bhi, acc[i][j], 0, 0, 0);
            }
        }
    };
    if (cnt != 0 && RING) {
#pragma unroll
        for (int s_ = 0; s_ < D; ++s_) load_slot(s_, (uint32_t)s_);
        uint32_t it0 = 0;
        for (; it0 + D < cnt; it0 += D) {
#pragma unroll
            for (int s_ = 0; s_ < D; ++s_) {
                mma_slot(s_);
                __builtin_amdgcn_sched_barrier(0);
                load_slot(s_, it0 + D + s_);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int s_ = 0; s_ < D; ++s_)
            if (it0 + s_ < cnt) mma_slot(s_);
    } else if (cnt != 0) {
        constexpr int U = (MT * NTW >= 4) ? 2 : 4;
        auto load_group = [&](uint32_t kt, v4u *bw, v4u *l, v4u *h) {
#pragma unroll
            for (int j = 0; j < NTW; ++j) {
                const uint32_t nt = nt0 + j;
                bw[j] = nt < n_tiles ? stream_load<true>((const v4u *)(b_base + ((uint64_t)nt * k_tiles + kt) * 1024)) : v4u{0, 0, 0, 0};
            }
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const uint32_t row = i * 16 + r;
                l[i] = v4u{0, 0, 0, 0};
                h[i] = v4u{0, 0, 0, 0};
                if (row < m) {
                    const v4u *p = (const v4u *)(a + (uint64_t)row * k + (uint64_t)kt * 64 + g * 16);
                    l[i] = p[0];
                    h[i] = p[1];
                }
            }
        };
        auto mma_group = [&](const v4u *l, const v4u *h, const v4u *bw) {
#pragma unroll
            for (int j = 0; j < NTW; ++j) {
                v8bf blo, bhi;
                cvt_i8x8_bf16(bw[j][0], bw[j][1], &blo);
                cvt_i8x8_bf16(bw[j][2], bw[j][3], &bhi);
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, l[i]), blo, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, h[i]), bhi, acc[i][j], 0, 0, 0);
                }
            }
        };
        uint32_t it = 0;
        for (; it + U <= cnt; it += U) {
            v4u bw[U][NTW], l[U][MT], h[U][MT];
#pragma unroll
            for (int u = 0; u < U; ++u) load_group(wave + (it + u) * NWAVES, bw[u], l[u], h[u]);
#pragma unroll
            for (int u = 0; u < U; ++u) mma_group(l[u], h[u], bw[u]);
        }
        for (; it < cnt; ++it) {
            v4u bw[NTW], l[MT], h[MT];
            load_group(wave + it * NWAVES, bw, l, h);
            mma_group(l, h, bw);
        }
    }

#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NTW; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[wave][(i * NTW + j) * 4 + e][lane] = acc[i][j][e];
    __syncthreads();

#pragma unroll
    for (int pq = 0; pq < NE; ++pq) {
        const int idx = wave + pq * NWAVES;
        if (idx >= NACC) break;
        float sum = red[0][idx][lane];
#pragma unroll
        for (int w = 1; w < NWAVES; ++w) sum = __fadd_rn(sum, red[w][idx][lane]);
        int e = idx % 4, j = (idx / 4) % NTW, i = idx / (4 * NTW);
        uint32_t row = i * 16 + 4 * g + e;
        uint32_t col = (nt0 + j) * 16 + r;
        if (row < m && col < n) {
            float v = __fmul_rn(sum, p_sw[pq]);
            uint64_t o = (uint64_t)row * n + col;
            if (out_bf16)
                ((uint16_t *)out)[o] = f32_to_bf16(v);
            else
                ((float *)out)[o] = v;
        }
    }
}

// Activation-stationary form of the kernel above (see w8a8_astat_kernel): the bf16 activations of
// the wavefront's k-tiles stay in registers (at m = 32 they are four times the bytes of a weight tile,
// so re-reading them per column tile through L2 costs far more than the weight stream), the block
// walks the column tiles b, b + gridDim, ... one tile ahead in a second register set, and the eight
// partial tiles are added in LDS in wavefront order, exactly the k-split and summation order of the
// eight-wavefront kernel above.
template <int MT, int KTW>
__global__ void __launch_bounds__(512)
    w8a16_astat_kernel(const uint16_t *__restrict__ a, const int8_t *__restrict__ w_tiles, const float *__restrict__ sw,
                       uint32_t m, uint32_t n, uint32_t n_tiles, uint32_t k_tiles, void *__restrict__ out, int out_bf16) {
    constexpr int NW = 8, NACC = MT * 4;
    __shared__ float red[2][NW][NACC][64];
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int g = lane / 16, r = lane % 16;
    const uint64_t k = (uint64_t)k_tiles * 64;
    const uint32_t last_kt = k_tiles - 1;

    v4u lo[KTW][MT], hi[KTW][MT];
#pragma unroll
    for (int t = 0; t < KTW; ++t) {
        uint32_t kt = wave + NW * t;
        kt = kt < k_tiles ? kt : last_kt;
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            uint32_t row = i * 16 + r;
            row = row < m ? row : m - 1;                   // rows past m are never stored
            const v4u *p = (const v4u *)(a + (uint64_t)row * k + (uint64_t)kt * 64 + g * 16);
            lo[t][i] = p[0];
            hi[t][i] = p[1];
        }
    }
    // the channel scale of a tile travels with its weights (see w8a8_astat_kernel)
    auto load_tile = [&](uint32_t nt, v4u (&b)[KTW], float &scale) {
        nt = nt < n_tiles ? nt : n_tiles - 1;
        scale = wave < NACC && nt * 16 + r < n ? sw[nt * 16 + r] : 0.0f;
        const int8_t *base = w_tiles + (uint64_t)nt * k_tiles * 1024 + (uint64_t)lane * 16;
#pragma unroll
        for (int t = 0; t < KTW; ++t) {
            uint32_t kt = wave + NW * t;
            kt = kt < k_tiles ? kt : last_kt;
            b[t] = stream_load<true>((const v4u *)(base + (uint64_t)kt * 1024));
        }
    };
    auto finish_tile = [&](uint32_t nt, const v4u (&b)[KTW], float scale, int buf) {
        v4f acc[MT];
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < KTW; ++t) {
            if ((uint32_t)(wave + NW * t) < k_tiles) {
                v8bf blo, bhi;
                cvt_i8x8_bf16(b[t][0], b[t][1], &blo);
                cvt_i8x8_bf16(b[t][2], b[t][3], &bhi);
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, lo[t][i]), blo, acc[i], 0, 0, 0);
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, hi[t][i]), bhi, acc[i], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[buf][wave][i * 4 + e][lane] = acc[i][e];
        __syncthreads();
        if (wave < NACC) {
            float sum = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; ++w) sum += red[buf][w][wave][lane];
            const int i = wave / 4, e = wave % 4;
            const uint32_t row = i * 16 + 4 * g + e, col = nt * 16 + r;
            if (row < m && col < n) {
                float v = __fmul_rn(sum, scale);
                uint64_t o = (uint64_t)row * n + col;
                if (out_bf16)
                    ((uint16_t *)out)[o] = f32_to_bf16(v);
                else
                    ((float *)out)[o] = v;
            }
        }
    };
    v4u b0[KTW], b1[KTW];
    float sc0, sc1;
    uint32_t nt = blockIdx.x;
    load_tile(nt, b0, sc0);
    for (; nt < n_tiles; nt += 2 * gridDim.x) {
        load_tile(nt + gridDim.x, b1, sc1);
        finish_tile(nt, b0, sc0, 0);
        if (nt + gridDim.x >= n_tiles) break;
        load_tile(nt + 2 * gridDim.x, b0, sc0);
        finish_tile(nt + gridDim.x, b1, sc1, 1);
    }
}

// ------------------------------------------------- split k across the blocks of one XCD
// With few column tiles (n = 4096: 256 tiles, one per compute unit) every block of the kernels above pulls the whole
// activation matrix through L2: 2 x (int8) or 4 x (bf16) the bytes of its weight tile at 32 rows, and with a deep k
// no register file holds it.  Here a group of S blocks owns S column tiles and each member streams 1 / S of k for
// all of them, so a compute unit fetches 1 / S of the activations.  The members' partial tiles meet in a workspace:
// every member stores its sums, waits until the stores are acknowledged, and takes a ticket from the group's
// counter; the member that draws the last ticket adds the S partial tiles in member order (a fixed order: the f32
// sums do not depend on who arrives last) and runs the epilogue.  Nobody waits for anybody.
// Workgroups are dealt to the eight XCDs round-robin by their linear id, so the members of a group are the blocks
// x + 8 (S q + r), r = 0 .. S - 1: they share one L2.  LOCAL = true relies on that (probed once per context by
// the caller): stores, ticket and loads are ordinary L2 accesses.  LOCAL = false uses agent-scope accesses that
// are coherent between XCDs wherever the blocks run.  The ticket is relaxed; what orders it behind the stores is
// the wait for their acknowledgement, not a fence (an agent-scope release writes back a whole L2).
template <bool LOCAL, typename T>
__device__ __forceinline__ void meet_store(T *p, T v) {
    if constexpr (LOCAL)
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    else
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <bool LOCAL, typename T>
__device__ __forceinline__ T meet_load(const T *p) {
    if constexpr (LOCAL)
        return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    else
        return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Four consecutive words of a partial tile set, requested with the cache policy of meet_load (a wider relaxed atomic
// load does not exist; the words were written by one 16-byte store whose acknowledgement the writer awaited before its
// ticket).  The request is an assembly statement, so the compiler neither waits for it nor knows that `v` is in
// flight: `v` may only be touched after an unseen_wait_all that names it.
template <bool LOCAL>
__device__ __forceinline__ void meet_request_b128(v4i &v, const int32_t *p) {
    if constexpr (LOCAL) asm volatile("global_load_dwordx4 %0, %1, off sc0" : "=&v"(v) : "v"(p));
    else asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=&v"(v) : "v"(p));
}
__device__ __forceinline__ void unseen_wait_all(v4i (&x)[4][4]) {
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(x[0][0]), "+v"(x[0][1]), "+v"(x[0][2]), "+v"(x[0][3]), "+v"(x[1][0]), "+v"(x[1][1]), "+v"(x[1][2]),
                   "+v"(x[1][3]), "+v"(x[2][0]), "+v"(x[2][1]), "+v"(x[2][2]), "+v"(x[2][3]), "+v"(x[3][0]), "+v"(x[3][1]),
                   "+v"(x[3][2]), "+v"(x[3][3]));
}
// Ticket of this block in its group (0 .. S - 1), the same value in every thread.  `slot` is one LDS word that
// nobody else uses between the two barriers.  Call with all of the block's partial stores issued.
template <bool LOCAL>
__device__ __forceinline__ uint32_t meet_ticket(uint32_t *counter, uint32_t *slot) {
    __builtin_amdgcn_s_waitcnt(0);                   // this thread's partial stores are acknowledged by L2 / memory
    __syncthreads();                                 // ... and so are everybody's
    if (threadIdx.x == 0) {
        uint32_t t;
        if constexpr (LOCAL)
            t = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else
            t = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *slot = t;
    }
    __syncthreads();
    return *slot;
}

// LOCAL only: the members of a group must share an XCD, or the partial tiles above were exchanged through two
// different L2s.  Every member notes the XCD it runs on before it takes its ticket; the last arriver compares and
// reports a mismatch in host memory (the context then refuses further work: the launch's results are wrong).
__device__ __forceinline__ uint32_t this_xcc() {
    uint32_t id;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(id));
    return id & 15u;
}
template <int S>
__device__ __forceinline__ void meet_check_xcd(const uint32_t *xcc_seen, uint32_t group, uint32_t *fault) {
    if (threadIdx.x != 0 || !xcc_seen) return;
    const uint32_t mine = this_xcc();
    bool same = true;
#pragma unroll
    for (int r = 0; r < S; ++r) same = same && meet_load<true>(xcc_seen + (uint64_t)group * S + r) == mine + 1u;
    if (!same) __hip_atomic_store(fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// block -> (group, member) of a split-k launch: see above
template <int S>
__device__ __forceinline__ void ksplit_ids(uint32_t *group, uint32_t *member) {
    ixm::ksplit_block(blockIdx.x, S, group, member);
}

// W8A8, plain epilogue.  Item idx = (i * S + j) * 4 + e of a block is accumulator element e of row tile i, column
// tile j of the group; wavefront w finishes the items w, w + 8, ...
template <int MT, int S, int D, bool LOCAL>
__global__ void __launch_bounds__(512)
    w8a8_ksplit_kernel(const int8_t *__restrict__ xq_tiled, const int8_t *__restrict__ w_tiles, uint32_t m, uint32_t n,
                       uint32_t n_tiles, uint32_t k_tiles, uint32_t n_groups, EpiI8 ep, int32_t *partial, uint32_t *counters,
                       uint32_t *xcc_seen, uint32_t *fault) {
    constexpr int NW = 8, NACC = MT * S * 4, NE = NACC / NW;
    static_assert(NACC % NW == 0, "items divide over the wavefronts");
    __shared__ int red[NW][NACC][64];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    uint32_t group, member;
    ksplit_ids<S>(&group, &member);
    if (group >= n_groups) return;                   // the same for every member of the group
    const uint32_t nt0 = group * S;
    uint32_t kt_lo, kt_hi;
    ixm::ksplit_k_range(k_tiles, member, S, &kt_lo, &kt_hi);
    const uint32_t len = kt_hi - kt_lo;
    const uint32_t cnt = len > (uint32_t)wave ? (len - wave + NW - 1) / NW : 0;

    v4i acc[MT][S];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < S; ++j) acc[i][j] = v4i{0, 0, 0, 0};
    // (a row tile that lies wholly at or past m, the fourth one of 33 to 48 rows, need not exist in xq_tiled: its lanes
    // fetch from row tile 0)
    uint32_t a_off[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) a_off[i] = ixm::decode_a_lane_byte((uint32_t)i, (uint32_t)lane, m);
    // epilogue operands, requested ahead of the weight stream by every member (only the last one uses them)
    float p_sx[NE], p_sw[NE], p_bias[NE], p_res[NE];
#pragma unroll
    for (int q = 0; q < NE; ++q) {
        p_sx[q] = p_sw[q] = p_bias[q] = p_res[q] = 0.0f;
        const int idx = wave + q * NW;
        const int e = idx % 4, j = (idx / 4) % S, i = idx / (4 * S);
        const uint32_t row = i * 16 + 4 * (lane / 16) + e, col = (nt0 + j) * 16 + lane % 16;
        if (row < m && col < n) {
            p_sx[q] = ep.sx[row];
            p_sw[q] = ep.sw[col];
            if (ep.bias) p_bias[q] = ep.bias[col];
            if (ep.residual) p_res[q] = ep.residual[(uint64_t)row * n + col];
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    const int8_t *b_base = w_tiles + (uint64_t)lane * 16;
    v4i a[D][MT], b[D][S];
    auto load_slot = [&](int s, uint32_t it) {
        const uint32_t kt = kt_lo + wave + (it < cnt ? it : cnt - 1) * NW;
#pragma unroll
        for (int j = 0; j < S; ++j) {
            uint32_t nt = nt0 + j;
            nt = nt < n_tiles ? nt : n_tiles - 1;            // a tile past the edge is loaded clamped, never stored
            b[s][j] = stream_load<true>((const v4i *)(b_base + ((uint64_t)nt * k_tiles + kt) * 1024));
        }
#pragma unroll
        for (int i = 0; i < MT; ++i) a[s][i] = *(const v4i *)(xq_tiled + ((uint64_t)ixm::decode_a_tile((uint32_t)i, m) * k_tiles + kt) * 1024 + a_off[i]);
    };
    auto mma_slot = [&](int s) {
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < S; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[s][i], b[s][j], acc[i][j], 0, 0, 0);
    };
    if (cnt != 0) {
#pragma unroll
        for (int s = 0; s < D; ++s) load_slot(s, (uint32_t)s);
        uint32_t it0 = 0;
        for (; it0 + D < cnt; it0 += D) {
#pragma unroll
            for (int s = 0; s < D; ++s) {
                mma_slot(s);
                __builtin_amdgcn_sched_barrier(0);
                load_slot(s, it0 + D + s);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int s = 0; s < D; ++s)
            if (it0 + s < cnt) mma_slot(s);
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < S; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[wave][(i * S + j) * 4 + e][lane] = acc[i][j][e];
    __syncthreads();
    int own[NE];
    int32_t *mine = partial + ixm::ksplit_partial_base(group, member, S, NACC);
#pragma unroll
    for (int q = 0; q < NE; ++q) {
        const int idx = wave + q * NW;
        int sum = 0;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += red[w][idx][lane];
        own[q] = sum;
        meet_store<LOCAL>(mine + idx * 64 + lane, sum);
    }
    if (LOCAL && xcc_seen && threadIdx.x == 0) meet_store<true>(xcc_seen + (uint64_t)group * S + member, this_xcc() + 1u);
    const uint32_t ticket = meet_ticket<LOCAL>(counters + group, (uint32_t *)&red[0][0][0]);
    if (ticket != S - 1) return;
    if (threadIdx.x == 0) meet_store<LOCAL>(counters + group, 0u);      // for the next launch
    if constexpr (LOCAL) meet_check_xcd<S>(xcc_seen, group, fault);
    int other[NE][S];
#pragma unroll
    for (int q = 0; q < NE; ++q)
#pragma unroll
        for (int r = 0; r < S; ++r)
            other[q][r] = meet_load<LOCAL>(partial + ixm::ksplit_partial_base(group, r, S, NACC) + (wave + q * NW) * 64 + lane);
#pragma unroll
    for (int q = 0; q < NE; ++q) {
        const int idx = wave + q * NW;
        int sum = 0;
#pragma unroll
        for (int r = 0; r < S; ++r) sum += (uint32_t)r == member ? own[q] : other[q][r];
        const int e = idx % 4, j = (idx / 4) % S, i = idx / (4 * S);
        const uint32_t row = i * 16 + 4 * (lane / 16) + e, col = (nt0 + j) * 16 + lane % 16;
        if (row < m && col < n) {
            const uint64_t o = (uint64_t)row * n + col;
            if (ep.acc_out) ep.acc_out[o] = sum;
            float v = __fmul_rn((float)sum, __fmul_rn(p_sx[q], p_sw[q]));
            if (ep.bias) v = __fadd_rn(v, p_bias[q]);
            if (ep.residual) v = __fadd_rn(p_res[q], v);
            if (ep.out_bf16)
                ((uint16_t *)ep.out)[o] = f32_to_bf16(v);
            else
                ((float *)ep.out)[o] = v;
        }
    }
}

// W8A8, weight stationary, for 65 to a few hundred rows against a deep, narrow weight (k of 8192 and more, about one
// column tile per compute unit): w8a8_wstat_kernel above would pull m x k activation bytes through every compute
// unit.  Here a group of S = 4 same-XCD blocks owns four column tiles and member j keeps the weights of k-range j of
// all four in registers (KTW k-tiles per wavefront x 4 tiles); the rows pass by in groups of 32, every member
// streaming only its quarter of their k.  The sums of a row group over the eight wavefronts meet in LDS and go to
// the workspace as one partial tile set per (member, row group); when the rows are through, the member takes a
// ticket as in w8a8_ksplit_kernel, and the last arriver adds the four partial sets of every row group (int32:
// exact in any order) and runs the epilogue for all rows of the group's 64 columns.  Nobody waits for anybody.
template <int KTW, int DS, bool LOCAL>
__global__ void __launch_bounds__(512)
    w8a8_wstat_ksplit_kernel(const int8_t *__restrict__ xq_tiled, const int8_t *__restrict__ w_tiles, uint32_t m, uint32_t n,
                             uint32_t n_tiles, uint32_t k_tiles, uint32_t n_groups, EpiI8 ep, int32_t *partial,
                             uint32_t *counters, uint32_t *xcc_seen, uint32_t *fault) {
    constexpr int NW = 8, S = 4, MT = 2, NACC = MT * S * 4;
    static_assert(MT * S == NW, "one accumulator tile of a row group per wavefront");
    static_assert(KTW % DS == 0, "the ring restarts at slot 0 with every row group");
    __shared__ v4i red[2][NW][MT * S][64];            // two buffers: one barrier per row group
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    uint32_t group, member;
    ksplit_ids<S>(&group, &member);
    if (group >= n_groups) return;                   // the same for every member of the group
    const uint32_t nt0 = group * S;
    uint32_t kt_lo, kt_hi;
    ixm::ksplit_k_range(k_tiles, member, S, &kt_lo, &kt_hi);
    const uint32_t len = kt_hi - kt_lo;
    const uint32_t cnt = len > (uint32_t)wave ? (len - wave + NW - 1) / NW : 0;       // k-tiles of this wavefront (<= KTW)
    const uint32_t row_tiles = (m + 15) / 16, row_groups = (row_tiles + MT - 1) / MT;
    // k-tile of step t (steps past the wavefront's last k-tile repeat it and multiply it with zeros)
    auto kt_of = [&](int t) -> uint32_t {
        const uint32_t kt = kt_lo + wave + ((uint32_t)t < cnt ? (uint32_t)t : (cnt ? cnt - 1 : 0)) * NW;
        return kt < k_tiles ? kt : k_tiles - 1;
    };

    v4i w[KTW][S];                                   // zeros past the wavefront's last k-tile: every step multiplies
#pragma unroll
    for (int t = 0; t < KTW; ++t) {
        const uint32_t kt = kt_of(t);
#pragma unroll
        for (int j = 0; j < S; ++j) {
            uint32_t nt = nt0 + j;
            nt = nt < n_tiles ? nt : n_tiles - 1;            // a tile past the edge is loaded clamped, never stored
            const v4i x = stream_load<true>((const v4i *)(w_tiles + ((uint64_t)nt * k_tiles + kt) * 1024 + (uint64_t)lane * 16));
            w[t][j] = (uint32_t)t < cnt ? x : v4i{0, 0, 0, 0};
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    v4i a[DS][MT];
    auto load_step = [&](int slot, uint32_t g, int t) {
        const uint32_t kt = kt_of(t);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            uint32_t rt = g * MT + i;
            rt = rt < row_tiles ? rt : row_tiles - 1;
            a[slot][i] = *(const v4i *)(xq_tiled + ((uint64_t)rt * k_tiles + kt) * 1024 + (uint64_t)lane * 16);
        }
    };
#pragma unroll
    for (int t = 0; t < DS; ++t) load_step(t, 0, t);
    for (uint32_t g = 0; g < row_groups; ++g) {
        v4i acc[MT][S];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < S; ++j) acc[i][j] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < KTW; ++t) {
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < S; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[t % DS][i], w[t][j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);                // the refill right behind its consumer
            if (t + DS < KTW) load_step(t % DS, g, t + DS);
            else load_step(t % DS, g + 1 < row_groups ? g + 1 : g, t + DS - KTW);
            __builtin_amdgcn_sched_barrier(0);
        }
        // the sums of row group g - 2 were read from this buffer before the barrier of group g - 1
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < S; ++j) red[g & 1][wave][i * S + j][lane] = acc[i][j];
        __syncthreads();
        // wavefront w adds the eight partial tiles of tile w = (row tile w / S, column tile w % S)
        v4i sum = v4i{0, 0, 0, 0};
#pragma unroll
        for (int ww = 0; ww < NW; ++ww) sum += red[g & 1][ww][wave][lane];
        int32_t *mine = partial + ixm::rows_ksplit_partial_base(group, member, S, row_groups, g, NACC);
        store_unseen_b128<LOCAL ? 1 : 2>(mine + (wave * 64 + lane) * 4, sum);       // the policy meet_store uses
    }
    if (LOCAL && xcc_seen && threadIdx.x == 0) meet_store<true>(xcc_seen + (uint64_t)group * S + member, this_xcc() + 1u);
    const uint32_t ticket = meet_ticket<LOCAL>(counters + group, (uint32_t *)&red[0][0][0][0]);
    if (ticket != S - 1) return;
    if (threadIdx.x == 0) meet_store<LOCAL>(counters + group, 0u);      // for the next launch
    if constexpr (LOCAL) meet_check_xcd<S>(xcc_seen, group, fault);
    // this wavefront's tile of every row group: rows 4 (lane / 16) + e of row tile wave / S, column lane % 16 of
    // column tile wave % S; the four members' sums are added in member order (int32: exact in any order)
    const int ti = wave / S, tj = wave % S;
    const uint32_t col = (nt0 + tj) * 16 + lane % 16;
    const bool col_ok = col < n;
    const float p_sw = col_ok ? ep.sw[col] : 0.0f;
    const float p_bias = (ep.bias && col_ok) ? ep.bias[col] : 0.0f;
    for (uint32_t g0 = 0; g0 < row_groups; g0 += 4) {            // four row groups' partial sets in flight
        v4i part[4][S];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t g = g0 + u < row_groups ? g0 + u : row_groups - 1;
#pragma unroll
            for (int r = 0; r < S; ++r)
                meet_request_b128<LOCAL>(part[u][r], partial + ixm::rows_ksplit_partial_base(group, r, S, row_groups, g, NACC) + (wave * 64 + lane) * 4);
        }
        float p_sx[4][4], p_res[4][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t row0 = ((g0 + u) * MT + ti) * 16 + 4 * (lane / 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const bool ok = row0 + e < m && col_ok;
                p_sx[u][e] = ok ? ep.sx[row0 + e] : 0.0f;
                p_res[u][e] = (ok && ep.residual) ? ep.residual[(uint64_t)(row0 + e) * n + col] : 0.0f;
            }
        }
        unseen_wait_all(part);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t row0 = ((g0 + u) * MT + ti) * 16 + 4 * (lane / 16);
            v4i sum = part[u][0];
#pragma unroll
            for (int r = 1; r < S; ++r) sum += part[u][r];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (row0 + e < m && col_ok) {                     // also false for the row groups past the last one
                    const uint64_t o = (uint64_t)(row0 + e) * n + col;
                    if (ep.acc_out) store_unseen_b32<0>(ep.acc_out + o, (uint32_t)sum[e]);
                    float v = __fmul_rn((float)sum[e], __fmul_rn(p_sx[u][e], p_sw));
                    if (ep.bias) v = __fadd_rn(v, p_bias);
                    if (ep.residual) v = __fadd_rn(p_res[u][e], v);
                    if (ep.out_bf16)
                        store_unseen_b16((uint16_t *)ep.out + o, f32_to_bf16(v));
                    else
                        store_unseen_b32<0>((float *)ep.out + o, __float_as_uint(v));
                }
            }
        }
    }
}

// W8A16: the same with bf16 activations, weights converted in registers, f32 partial tiles added in member order.
template <int MT, int S, int D, bool LOCAL>
__global__ void __launch_bounds__(512)
    w8a16_ksplit_kernel(const uint16_t *__restrict__ a, const int8_t *__restrict__ w_tiles, const float *__restrict__ sw,
                        uint32_t m, uint32_t n, uint32_t n_tiles, uint32_t k_tiles, uint32_t n_groups, void *__restrict__ out,
                        int out_bf16, float *partial, uint32_t *counters, uint32_t *xcc_seen, uint32_t *fault) {
    constexpr int NW = 8, NACC = MT * S * 4, NE = NACC / NW;
    static_assert(NACC % NW == 0, "items divide over the wavefronts");
    __shared__ float red[NW][NACC][64];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int g = lane / 16, r = lane % 16;
    uint32_t group, member;
    ksplit_ids<S>(&group, &member);
    if (group >= n_groups) return;
    const uint32_t nt0 = group * S;
    const uint64_t k = (uint64_t)k_tiles * 64;
    uint32_t kt_lo, kt_hi;
    ixm::ksplit_k_range(k_tiles, member, S, &kt_lo, &kt_hi);
    const uint32_t len = kt_hi - kt_lo;
    const uint32_t cnt = len > (uint32_t)wave ? (len - wave + NW - 1) / NW : 0;

    v4f acc[MT][S];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < S; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
    float p_sw[NE];
#pragma unroll
    for (int q = 0; q < NE; ++q) {
        const int idx = wave + q * NW;
        const uint32_t col = (nt0 + (idx / 4) % S) * 16 + r;
        p_sw[q] = col < n ? sw[col] : 0.0f;
    }
    __builtin_amdgcn_sched_barrier(0);
    const int8_t *b_base = w_tiles + (uint64_t)lane * 16;
    const uint32_t last_tile = n_tiles - 1;
    uint32_t a_row[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) a_row[i] = (uint32_t)i * 16 + r < m ? (uint32_t)i * 16 + r : 0u;
    v4u braw[D][S], lo[D][MT], hi[D][MT];
    auto load_slot = [&](int s_, uint32_t it) {
        const uint32_t kt = kt_lo + wave + (it < cnt ? it : cnt - 1) * NW;
#pragma unroll
        for (int j = 0; j < S; ++j) {
            uint32_t nt = nt0 + j;
            nt = nt < last_tile ? nt : last_tile;
            braw[s_][j] = stream_load<true>((const v4u *)(b_base + ((uint64_t)nt * k_tiles + kt) * 1024));
        }
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const v4u *p = (const v4u *)(a + (uint64_t)a_row[i] * k + (uint64_t)kt * 64 + g * 16);
            lo[s_][i] = p[0];
            hi[s_][i] = p[1];
        }
    };
    auto mma_slot = [&](int s_) {
#pragma unroll
        for (int j = 0; j < S; ++j) {
            v8bf blo, bhi;
            cvt_i8x8_bf16(braw[s_][j][0], braw[s_][j][1], &blo);
            cvt_i8x8_bf16(braw[s_][j][2], braw[s_][j][3], &bhi);
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, lo[s_][i]), blo, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, hi[s_][i]), bhi, acc[i][j], 0, 0, 0);
            }
        }
    };
    if (cnt != 0) {
#pragma unroll
        for (int s_ = 0; s_ < D; ++s_) load_slot(s_, (uint32_t)s_);
        uint32_t it0 = 0;
        for (; it0 + D < cnt; it0 += D) {
#pragma unroll
            for (int s_ = 0; s_ < D; ++s_) {
                mma_slot(s_);
                __builtin_amdgcn_sched_barrier(0);
                load_slot(s_, it0 + D + s_);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int s_ = 0; s_ < D; ++s_)
            if (it0 + s_ < cnt) mma_slot(s_);
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < S; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[wave][(i * S + j) * 4 + e][lane] = acc[i][j][e];
    __syncthreads();
    float own[NE];
    float *mine = partial + ixm::ksplit_partial_base(group, member, S, NACC);
#pragma unroll
    for (int q = 0; q < NE; ++q) {
        const int idx = wave + q * NW;
        float sum = red[0][idx][lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) sum = __fadd_rn(sum, red[w][idx][lane]);
        own[q] = sum;
        meet_store<LOCAL>(mine + idx * 64 + lane, sum);
    }
    if (LOCAL && xcc_seen && threadIdx.x == 0) meet_store<true>(xcc_seen + (uint64_t)group * S + member, this_xcc() + 1u);
    const uint32_t ticket = meet_ticket<LOCAL>(counters + group, (uint32_t *)&red[0][0][0]);
    if (ticket != S - 1) return;
    if (threadIdx.x == 0) meet_store<LOCAL>(counters + group, 0u);
    if constexpr (LOCAL) meet_check_xcd<S>(xcc_seen, group, fault);
    float other[NE][S];
#pragma unroll
    for (int q = 0; q < NE; ++q)
#pragma unroll
        for (int r2 = 0; r2 < S; ++r2)
            other[q][r2] = meet_load<LOCAL>(partial + ixm::ksplit_partial_base(group, r2, S, NACC) + (wave + q * NW) * 64 + lane);
#pragma unroll
    for (int q = 0; q < NE; ++q) {
        const int idx = wave + q * NW;
        float sum = 0.0f;
#pragma unroll
        for (int r2 = 0; r2 < S; ++r2) {
            const float t = (uint32_t)r2 == member ? own[q] : other[q][r2];
            sum = r2 == 0 ? t : __fadd_rn(sum, t);
        }
        const int e = idx % 4, j = (idx / 4) % S, i = idx / (4 * S);
        const uint32_t row = i * 16 + 4 * g + e, col = (nt0 + j) * 16 + r;
        if (row < m && col < n) {
            const float v = __fmul_rn(sum, p_sw[q]);
            const uint64_t o = (uint64_t)row * n + col;
            if (out_bf16)
                ((uint16_t *)out)[o] = f32_to_bf16(v);
            else
                ((float *)out)[o] = v;
        }
    }
}

// ------------------------------------------------------------------ e4m3 x e4m3, decode shape
// out[m, n] = (sum_k a[m, k] * w[k, n]) * (sx[m] * sw[n]) (+ bias[n]) on the scaled 16x16x128 fp8 matrix
// instruction with unit block scales.  The weight is in tiles of 16 columns x 128 k (2 KiB, 32 bytes per lane:
// column l % 16, k-group l / 16); the activations are row-major e4m3 [m, k_pad], and a lane fetches the 32 bytes
// of row l % 16, k-group l / 16 of the k-tile directly (lanes of rows at or past m fetch the row tile's first
// row: their accumulator rows are never stored).  One block per column tile, k split over the wavefronts, the
// k-tiles of a wavefront streamed through a ring of D register slots as in the int8 kernel above; the partial
// tiles are added in LDS in wavefront order.
template <int MT, int NWAVES>
__global__ void __launch_bounds__(NWAVES * 64)
    e4m3_skinny_kernel(const uint8_t *__restrict__ aq, const uint8_t *__restrict__ w_tiles, const float *__restrict__ sx,
                       const float *__restrict__ sw, const float *__restrict__ bias, uint32_t m, uint32_t n,
                       uint32_t k_tiles, void *__restrict__ out, int out_bf16) {
    constexpr int NACC = MT * 4, D = MT >= 3 ? 2 : 4;
    __shared__ float red[NWAVES][NACC][64];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const uint32_t nt = blockIdx.x;
    const uint64_t k_bytes = (uint64_t)k_tiles * 128;
    v4f acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
    const uint8_t *b_base = w_tiles + (uint64_t)nt * k_tiles * 2048 + (uint64_t)lane * 32;
    const uint8_t *a_base[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        uint32_t row = (uint32_t)i * 16 + (uint32_t)lane % 16;
        row = row < m ? row : (uint32_t)i * 16;
        a_base[i] = aq + (uint64_t)row * k_bytes + (uint64_t)(lane / 16) * 32;
    }
    const uint32_t cnt = k_tiles > (uint32_t)wave ? (k_tiles - wave + NWAVES - 1) / NWAVES : 0;
    // scales and bias of the epilogue, requested ahead of the weight stream (see w8a8_skinny_kernel)
    constexpr int NE = (NACC + NWAVES - 1) / NWAVES;
    float p_sx[NE], p_sw[NE], p_bias[NE];
#pragma unroll
    for (int q = 0; q < NE; ++q) {
        const int idx = wave + q * NWAVES;
        const uint32_t row = (idx / 4) * 16 + 4 * (lane / 16) + idx % 4, col = nt * 16 + lane % 16;
        const bool live = idx < NACC && row < m && col < n;
        p_sx[q] = live ? sx[row] : 0.0f;
        p_sw[q] = live ? sw[col] : 0.0f;
        p_bias[q] = live && bias ? bias[col] : 0.0f;
    }
    __builtin_amdgcn_sched_barrier(0);
    v4i a[D][MT][2], b[D][2];
    auto load_slot = [&](int s, uint32_t it) {
        const uint32_t kt = wave + (it < cnt ? it : cnt - 1) * NWAVES;
        const v4i *bp = (const v4i *)(b_base + (uint64_t)kt * 2048);
        b[s][0] = stream_load<true>(bp);
        b[s][1] = stream_load<true>(bp + 1);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const v4i *ap = (const v4i *)(a_base[i] + (uint64_t)kt * 128);
            a[s][i][0] = ap[0];
            a[s][i][1] = ap[1];
        }
    };
    auto mma_slot = [&](int s) {
        const v8i y{b[s][0][0], b[s][0][1], b[s][0][2], b[s][0][3], b[s][1][0], b[s][1][1], b[s][1][2], b[s][1][3]};
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const v8i x{a[s][i][0][0], a[s][i][0][1], a[s][i][0][2], a[s][i][0][3],
                        a[s][i][1][0], a[s][i][1][1], a[s][i][1][2], a[s][i][1][3]};
            acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(x, y, acc[i], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
        }
    };
    if (cnt != 0) {
#pragma unroll
        for (int s = 0; s < D; ++s) load_slot(s, (uint32_t)s);
        uint32_t it0 = 0;
        for (; it0 + D < cnt; it0 += D) {
#pragma unroll
            for (int s = 0; s < D; ++s) {
                mma_slot(s);
                __builtin_amdgcn_sched_barrier(0);
                load_slot(s, it0 + D + s);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int s = 0; s < D; ++s)
            if (it0 + s < cnt) mma_slot(s);
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) red[wave][i * 4 + e][lane] = acc[i][e];
    __syncthreads();
#pragma unroll
    for (int pq = 0; pq < NE; ++pq) {
        const int idx = wave + pq * NWAVES;
        if (idx >= NACC) break;
        float sum = red[0][idx][lane];
#pragma unroll
        for (int w = 1; w < NWAVES; ++w) sum = __fadd_rn(sum, red[w][idx][lane]);
        const int e = idx % 4, i = idx / 4;
        const uint32_t row = i * 16 + 4 * (lane / 16) + e, col = nt * 16 + lane % 16;
        if (row < m && col < n) {
            float v = __fmul_rn(sum, __fmul_rn(p_sx[pq], p_sw[pq]));
            if (bias) v = __fadd_rn(v, p_bias[pq]);
            const uint64_t o = (uint64_t)row * n + col;
            if (out_bf16)
                ((uint16_t *)out)[o] = f32_to_bf16(v);
            else
                ((float *)out)[o] = v;
        }
    }
}

// Picks n-tiles per block and wavefronts per block so that the whole grid is
// resident at once with about 8-16 wavefronts per compute unit.
inline void pick_config(uint64_t n_tiles, uint64_t k_tiles, int num_cus, int *ntw, int *waves) {
    int w = 8, t = 1;
    if (k_tiles < 32) w = 4;
    // blocks = n_tiles / t; resident waves per CU = blocks * w / num_cus
    while (t < 2 && (n_tiles / (uint64_t)t) * (uint64_t)w > (uint64_t)num_cus * 16) t *= 2;
    if ((n_tiles / (uint64_t)t) * (uint64_t)w > (uint64_t)num_cus * 16 && w == 8) w = 4;
    if (g_skinny_ntw) t = g_skinny_ntw;
    if (g_skinny_waves) w = g_skinny_waves;
    *ntw = t;
    *waves = w;
}

// The activation-stationary kernel pays off when every block has several units to amortize its
// activation registers over and the k-tiles fit eight per wavefront.
inline bool astat_applies(uint64_t n_units, uint64_t k_tiles, int num_cus) {
    if (g_skinny_astat == 1) return false;
    if (k_tiles > 64 || k_tiles == 0) return false;
    if (g_skinny_astat == 2) return true;
    return n_units >= 3 * (uint64_t)num_cus;
}

// w8a8_astat_wide_kernel for 33 to 64 rows: as many blocks as compute units (or units), 96 / 128 KiB of dynamic LDS
template <int MODE>
void launch_astat_wide(uint64_t m, unsigned blocks, hipStream_t s, const int8_t *xq_tiled, const int8_t *w_tiles, uint32_t n,
                       uint32_t n_tiles, uint32_t k_tiles, uint32_t n_units, const EpiI8 &e) {
    auto go = [&](auto mt) {
        constexpr int MT = decltype(mt)::value;
        const size_t smem = (size_t)2 * 8 * (MT * 8) * 64 * 4;
        static bool configured = false;
        if (!configured) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&w8a8_astat_wide_kernel<MT, MODE>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
            configured = true;
        }
        w8a8_astat_wide_kernel<MT, MODE><<<blocks, 512, smem, s>>>(xq_tiled, w_tiles, (uint32_t)m, n, n_tiles, k_tiles, n_units, e);
    };
    if (m <= 48)
        go(std::integral_constant<int, 3>{});
    else
        go(std::integral_constant<int, 4>{});
}
inline bool astat_wide_applies(uint64_t m, uint64_t n_units, uint64_t k_tiles, int num_cus) {
    return g_skinny_astat != 3 && m > 32 && m <= 64 && astat_applies(n_units, k_tiles, num_cus);
}

// Row tiles per block by the number of rows (16 each, at most 64 rows), 4 or 8 wavefronts.
template <int NTW, int MODE, typename... A>
void launch_w8a8_rows(uint64_t m, int waves, unsigned grid, hipStream_t s, A... args) {
    auto go = [&](auto mt) {
        constexpr int MT = decltype(mt)::value;
        if (waves == 8)
            w8a8_skinny_kernel<MT, NTW, 8, MODE><<<grid, 512, 0, s>>>(args..., RowPrologue{});
        else
            w8a8_skinny_kernel<MT, NTW, 4, MODE><<<grid, 256, 0, s>>>(args..., RowPrologue{});
    };
    if (m <= 16)
        go(std::integral_constant<int, 1>{});
    else if (m <= 32)
        go(std::integral_constant<int, 2>{});
    else if (m <= 48)
        go(std::integral_constant<int, 3>{});
    else
        go(std::integral_constant<int, 4>{});
}

template <int MT, bool RING>
void launch_w8a16_form(const uint16_t *a, const int8_t *wt, const float *sw, uint32_t m, uint32_t n, uint32_t n_tiles,
                       uint32_t k_tiles, void *out, int out_bf16, int ntw, int waves, hipStream_t s) {
    unsigned grid = (n_tiles + ntw - 1) / ntw;
    if (ntw == 1 && waves == 8)
        w8a16_skinny_kernel<MT, 1, 8, RING><<<grid, 512, 0, s>>>(a, wt, sw, m, n, n_tiles, k_tiles, out, out_bf16);
    else if (ntw == 1)
        w8a16_skinny_kernel<MT, 1, 4, RING><<<grid, 256, 0, s>>>(a, wt, sw, m, n, n_tiles, k_tiles, out, out_bf16);
    else if (waves == 8)
        w8a16_skinny_kernel<MT, 2, 8, RING><<<grid, 512, 0, s>>>(a, wt, sw, m, n, n_tiles, k_tiles, out, out_bf16);
    else
        w8a16_skinny_kernel<MT, 2, 4, RING><<<grid, 256, 0, s>>>(a, wt, sw, m, n, n_tiles, k_tiles, out, out_bf16);
}

template <int MT>
void launch_w8a16(const uint16_t *a, const int8_t *wt, const float *sw, uint32_t m, uint32_t n, uint32_t n_tiles,
                  uint32_t k_tiles, void *out, int out_bf16, int ntw, int waves, hipStream_t s) {
    if (k_tiles <= 64 || m == 1)
        launch_w8a16_form<MT, true>(a, wt, sw, m, n, n_tiles, k_tiles, out, out_bf16, ntw, waves, s);
    else
        launch_w8a16_form<MT, false>(a, wt, sw, m, n, n_tiles, k_tiles, out, out_bf16, ntw, waves, s);
}


// Whether a decode-shape linear goes out in the split-k form (w8a8_ksplit_kernel), and how: members per group,
// depth of the register ring, where the partial tiles meet.
struct KsplitPlan {
    int s, d;
    bool local;
    uint32_t n_groups, blocks;
};
inline bool ksplit_plan(uint64_t m, uint32_t n_tiles, uint32_t k_tiles, int num_cus, const SplitKArea *sk, int act_bytes,
                        KsplitPlan *p) {
    // int8 activations: up to four row tiles (64 rows), in pairs of blocks; bf16 activations: up to two
    const uint64_t m_max = act_bytes == 1 ? 64 : 32;
    if (!sk || !sk->partial || !sk->counters || g_skinny_ksplit == 1 || m == 0 || m > m_max || n_tiles == 0) return false;
    const bool forced = g_skinny_ksplit == 2 || g_skinny_ksplit == 3;
    // By shape: the projections with about one column tile per compute unit whose blocks would each pull 256 KiB of
    // activations or more (measured in a decode step's kernel trace at 32 rows: 14336 -> 4096 int8 17.3 -> 14.6 us,
    // while 4096 -> 4096 int8, 128 KiB per block, loses 0.7 us to the meeting); wider weights keep their activations
    // in registers (w8a8_astat_kernel).
    const int mt = m <= 16 ? 1 : m <= 32 ? 2 : 4;
    const uint64_t a_bytes = (uint64_t)(16 * mt) * k_tiles * 64 * (uint64_t)act_bytes;
    // (with four row tiles a pair of blocks halves the bytes: worth it from 512 KiB on; in a 64-row step's trace
    // 4096 -> 4096 at 256 KiB went from 6 to 7.4 us, 14336 -> 4096 from 24 to 21.7 us)
    if (!forced && ((uint64_t)n_tiles > 2 * (uint64_t)num_cus || a_bytes < ((mt == 4 ? 512u : 256u) << 10))) return false;
    int s = g_skinny_ksplit_s ? g_skinny_ksplit_s : (k_tiles >= 128 ? 4 : 2);
    if (mt == 4) s = 2;                                        // the partial tiles of four row tiles x four members do not fit LDS
    if (s != 2 && s != 4) return false;
    if (k_tiles / (uint32_t)s < 16) return false;              // two k-tiles per wavefront at least
    const uint32_t n_groups = (n_tiles + s - 1) / s;
    const uint64_t bytes = (uint64_t)n_groups * s * ((uint64_t)mt * s * 4 * 64 * 4);
    if (n_groups > sk->n_counters || bytes > sk->partial_bytes) return false;
    p->s = s;
    p->d = k_tiles / (uint32_t)s >= 32 ? 4 : 2;
    p->local = g_skinny_ksplit == 3 || ((g_skinny_ksplit == 0) && sk->xcd_local);
    p->n_groups = n_groups;
    p->blocks = 8u * (uint32_t)s * ((n_groups + 7) / 8);       // whole groups on every XCD; surplus groups return at once
    return true;
}

// the XCD notes of a launch, when the area has room for one word per block and a place to report to
inline uint32_t *xcc_seen_for(const SplitKArea *sk, const KsplitPlan &p) {
    return (sk->xcc_seen && sk->fault && (uint64_t)p.n_groups * p.s <= sk->n_xcc_seen) ? sk->xcc_seen : nullptr;
}

// Calls go(MT, S, D, LOCAL) with the plan's values as integral constants.
template <typename F>
void ksplit_dispatch(uint64_t m, const KsplitPlan &p, F &&go) {
    auto with_local = [&](auto mt, auto s, auto d) {
        if (p.local)
            go(mt, s, d, std::true_type{});
        else
            go(mt, s, d, std::false_type{});
    };
    auto with_d = [&](auto mt, auto s) {
        if (p.d == 4)
            with_local(mt, s, std::integral_constant<int, 4>{});
        else
            with_local(mt, s, std::integral_constant<int, 2>{});
    };
    auto with_s = [&](auto mt) {
        if (p.s == 4)
            with_d(mt, std::integral_constant<int, 4>{});
        else
            with_d(mt, std::integral_constant<int, 2>{});
    };
    if (m <= 16)
        with_s(std::integral_constant<int, 1>{});
    else if (m <= 32)
        with_s(std::integral_constant<int, 2>{});
    else
        with_d(std::integral_constant<int, 4>{}, std::integral_constant<int, 2>{});      // 33 .. 64 rows: pairs only
}

}  // namespace

// out[b] = id of the XCD that workgroup b of this launch runs on (what ksplit_ids assumes is b % 8 up to a
// renaming of the XCDs; the caller checks)
namespace {
__global__ void __launch_bounds__(64) xcc_id_probe_kernel(uint32_t *out) {
    uint32_t id;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(id));
    if (threadIdx.x == 0) out[blockIdx.x] = id & 15u;
}
}  // namespace
void xcc_id_probe(uint32_t *out, uint32_t blocks, hipStream_t s) { xcc_id_probe_kernel<<<blocks, 64, 0, s>>>(out); }

// Which weight bytes the blocks of the launches below read first, for the row kernel in front of them to pull
// (WeightPrefetch): the block -> tile mapping of every form is restated here beside the launch that uses it.
// `budget` bounds the bytes of one pull (what HBM delivers while a row kernel waits on its own round trips).
namespace {
WeightPrefetch make_prefetch(const int8_t *w_tiles, uint32_t blocks, uint32_t n_tiles, uint32_t k_tiles, uint32_t half_tiles,
                             uint32_t tile_stride, uint32_t pair_step, uint64_t budget) {
    WeightPrefetch pf;
    if (g_weight_prefetch == 1 || blocks == 0 || k_tiles == 0 || n_tiles == 0) return pf;
    const uint64_t regions = (uint64_t)blocks * (pair_step ? 2 : 1);
    uint64_t per = budget / regions / 1024 * 1024;
    if (per > (uint64_t)k_tiles * 1024) per = (uint64_t)k_tiles * 1024;
    if (per == 0) return pf;
    pf.w = w_tiles;
    pf.blocks = blocks;
    pf.n_tiles = n_tiles;
    pf.k_tiles = k_tiles;
    pf.half_tiles = half_tiles;
    pf.tile_stride = tile_stride;
    pf.pair_step = pair_step;
    pf.bytes = (uint32_t)per;
    return pf;
}
}  // namespace

WeightPrefetch prefetch_for_linear_w8a8_skinny(const int8_t *w_tiles, uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus,
                                               uint64_t budget, const SplitKArea *sk) {
    const uint32_t n_tiles = (uint32_t)(n_pad / 16), k_tiles = (uint32_t)(k_pad / 64);
    if (m == 0 || n_tiles == 0) return WeightPrefetch{};
    KsplitPlan kp;
    if (ksplit_plan(m, n_tiles, k_tiles, num_cus, sk, 1, &kp)) {     // block -> (group, member) as in ksplit_ids
        if (g_weight_prefetch == 1 || k_tiles == 0) return WeightPrefetch{};
        WeightPrefetch pf;
        uint64_t per = budget / ((uint64_t)kp.blocks * kp.s) / 1024 * 1024;
        per = std::min<uint64_t>(per, (uint64_t)(k_tiles / kp.s) * 1024);
        if (per == 0) return pf;
        pf.w = w_tiles;
        pf.blocks = kp.blocks;
        pf.n_tiles = n_tiles;
        pf.k_tiles = k_tiles;
        pf.bytes = (uint32_t)per;
        pf.ksplit = (uint32_t)kp.s;
        return pf;
    }
    if ((m <= 32 && astat_applies((n_tiles + 1) / 2, k_tiles, num_cus)) ||
        astat_wide_applies(m, (n_tiles + 1) / 2, k_tiles, num_cus)) {           // block b starts with unit b = tiles 2 b, 2 b + 1
        const uint32_t n_units = (n_tiles + 1) / 2;
        return make_prefetch(w_tiles, (uint32_t)std::min<uint64_t>(n_units, (uint64_t)num_cus), n_tiles, k_tiles, 0, 2, n_tiles > 1 ? 1 : 0, budget);
    }
    int ntw, waves;
    pick_config(n_tiles, k_tiles, num_cus, &ntw, &waves);
    const uint32_t grid = (n_tiles + ntw - 1) / ntw;
    return make_prefetch(w_tiles, grid, n_tiles, k_tiles, 0, (uint32_t)ntw, ntw == 2 && n_tiles > 1 ? 1 : 0, budget);
}

WeightPrefetch prefetch_for_linear_w8a8_qkv_rope_skinny(const int8_t *w_tiles, uint64_t m, uint64_t n_pad, uint64_t k_pad,
                                                        const QkvRopeTargets &t, uint64_t budget) {
    if (m == 0) return WeightPrefetch{};
    const uint32_t n = (t.heads + 2 * t.kv_heads) * t.head_dim, half_tiles = t.head_dim / 32;
    // block b: tile (b / half) * 2 * half + b % half and the tile half_tiles further on
    return make_prefetch(w_tiles, n / 32, (uint32_t)(n_pad / 16), (uint32_t)(k_pad / 64), half_tiles, 1, half_tiles, budget);
}

namespace {
// bytes of LDS a block needs for its own activation codes
inline size_t prologue_lds_bytes(uint64_t m, uint64_t k_pad) { return (size_t)((m * k_pad + 15) / 16 * 16); }
inline bool norm_prologue_shape(uint64_t m, uint64_t k_pad) {
    // the stand-alone kernel whose f64 association the prologue reproduces is the 1024-thread, one-group-per-thread form
    // by measurement one or two rows (whole steps of 1 / 2 / 3 / 4 rows through 32 layers, contexts 100-200: 2.10 / 2.22 / 2.35 /
    // 2.47 ms with the row work in here against 2.30 / 2.34 / 2.29 / 2.30 ms with the row kernels); the kernels take four
    const uint64_t rows = g_row_fusion == 2 ? 4 : 2;
    return g_row_fusion != 1 && m >= 1 && m <= rows && k_pad > 1024 && k_pad <= 4096 && k_pad % 64 == 0;
}
}  // namespace

bool qkv_rope_fuses_norm(uint64_t m, uint64_t k_pad) { return norm_prologue_shape(m, k_pad) && !g_skinny_waves; }
bool swiglu_fuses_norm(uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus) {
    return norm_prologue_shape(m, k_pad) && astat_applies(n_pad / 32, k_pad / 64, num_cus);
}
bool plain_fuses_pmax_quantizer(uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus) {
    // by measurement one row (two rows: 2.22 ms a step without, 2.34 ms with); the kernel takes two
    const uint64_t rows = g_row_fusion == 2 ? 2 : 1;
    if (g_row_fusion == 1 || m == 0 || m > rows || k_pad % 64 != 0 || k_pad > 16384) return false;     // PmaxRows
    if (k_pad / 16 > 1024) return false;                     // partial maxima per row the prologue reads
    const uint64_t n_tiles = n_pad / 16, k_tiles = k_pad / 64;
    if (astat_applies((n_tiles + 1) / 2, k_tiles, num_cus)) return false;
    int ntw, waves;
    pick_config(n_tiles, k_tiles, num_cus, &ntw, &waves);
    return ntw == 1 && waves == 8;                          // the form the fused kernel is built in
}

void linear_w8a8_skinny(const int8_t *xq_tiled, const int8_t *w_tiles, uint64_t m, uint64_t n, uint64_t n_pad,
                        uint64_t k_pad, const EpilogueI8 &ep, int num_cus, hipStream_t s, const SplitKArea *sk,
                        const RowPrologue *pro) {
    if (m == 0 || n == 0) return;
    uint32_t n_tiles = (uint32_t)(n_pad / 16), k_tiles = (uint32_t)(k_pad / 64);
    if (pro) {                                              // the caller asked plain_fuses_pmax_quantizer first
        EpiI8 e{};
        e.sw = ep.sw;
        e.bias = ep.bias;
        e.residual = ep.residual;
        e.acc_out = ep.acc_out;
        e.out = ep.out;
        e.out_bf16 = ep.out_bf16;
        w8a8_skinny_kernel<1, 1, 8, kEpiPlain, 2><<<n_tiles, 512, prologue_lds_bytes(m, k_pad), s>>>(
            nullptr, w_tiles, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, e, *pro);
        return;
    }
    EpiI8 e{};
    e.sx = ep.sx;
    e.sw = ep.sw;
    e.bias = ep.bias;
    e.residual = ep.residual;
    e.acc_out = ep.acc_out;
    e.out = ep.out;
    e.out_bf16 = ep.out_bf16;
    KsplitPlan kp;
    if (ksplit_plan(m, n_tiles, k_tiles, num_cus, sk, 1, &kp)) {
        ksplit_dispatch(m, kp, [&](auto mt, auto ss, auto d, auto local) {
            w8a8_ksplit_kernel<decltype(mt)::value, decltype(ss)::value, decltype(d)::value, decltype(local)::value>
                <<<kp.blocks, 512, 0, s>>>(xq_tiled, w_tiles, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, kp.n_groups, e,
                                           (int32_t *)sk->partial, sk->counters, xcc_seen_for(sk, kp), sk->fault);
        });
        return;
    }
    if (m <= 32 && astat_applies((n_tiles + 1) / 2, k_tiles, num_cus)) {
        unsigned n_units = (n_tiles + 1) / 2;
        unsigned blocks = (unsigned)std::min<uint64_t>(n_units, (uint64_t)num_cus);
        if (m <= 16)
            w8a8_astat_kernel<1, 8, kEpiPlain><<<blocks, 512, 0, s>>>(xq_tiled, w_tiles, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, n_units, e, RowPrologue{});
        else
            w8a8_astat_kernel<2, 8, kEpiPlain><<<blocks, 512, 0, s>>>(xq_tiled, w_tiles, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, n_units, e, RowPrologue{});
        return;
    }
    if (astat_wide_applies(m, (n_tiles + 1) / 2, k_tiles, num_cus)) {
        const unsigned n_units = (n_tiles + 1) / 2;
        launch_astat_wide<kEpiPlain>(m, (unsigned)std::min<uint64_t>(n_units, (uint64_t)num_cus), s, xq_tiled, w_tiles, (uint32_t)n, n_tiles,
                                     k_tiles, n_units, e);
        return;
    }
    int ntw, waves;
    pick_config(n_tiles, k_tiles, num_cus, &ntw, &waves);
    const unsigned grid = (n_tiles + ntw - 1) / ntw;
    if (ntw == 1)
        launch_w8a8_rows<1, kEpiPlain>(m, waves, grid, s, xq_tiled, w_tiles, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, e);
    else
        launch_w8a8_rows<2, kEpiPlain>(m, waves, grid, s, xq_tiled, w_tiles, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, e);
}

// The split-k form of the weight-stationary kernel (w8a8_wstat_ksplit_kernel): deep, narrow weights (k from 8192 up to
// what four members x eight wavefronts x eight k-tiles hold, about one column tile per compute unit), more rows than
// the decode kernels take, and a quarter of the activations (m x k / 4 bytes per block) within what a compute unit
// pulls from L2 in the time of the tiled GEMM.
namespace {
struct RowsKsplitPlan {
    uint32_t n_groups, blocks, row_groups;
    uint64_t workspace_bytes;
    bool local;
};
inline bool rows_ksplit_plan(uint64_t m, uint32_t n_tiles, uint32_t k_tiles, int num_cus, const SplitKArea *sk, RowsKsplitPlan *p) {
    if (!sk || !sk->counters || g_rows_kernel == 1 || g_rows_kernel == 2 || g_skinny_ksplit == 1) return false;
    // (k up to what the kernel without the split holds as well, so that a caller without a workspace still has a form)
    if (m <= 64 || n_tiles == 0 || k_tiles < 128 || k_tiles > 224) return false;
    // measured against the tiled GEMM with its k split and the kernel without the split (us incl. the row quantizer, 65 / 128 /
    // 200 / 300 / 512 rows): 14336 -> 4096 27.7 / 31.6 / 45.4 / 57.8 / 79.3 against 37.6 / 41.8 / 49.3 / 67.7 / 90.7 and 32.7 /
    // 36.6 / 53.8 / 69.1 / 102; 11008 -> 4096 26.0 / 29.7 / 43.8 / 53.9 / 71.6 against 34.6 / 39.9 / 43.5 / 56.0 / 76.3; at
    // 8192 -> 4096 the kernel without the split is the faster one while its rule admits it and the three are level above
    if (g_rows_kernel != 3 && k_tiles < 160) return false;
    if (g_rows_kernel != 3 && (m > 512 || (uint64_t)n_tiles > 2 * (uint64_t)num_cus)) return false;
    const uint32_t n_groups = (n_tiles + 3) / 4;
    if (n_groups > sk->n_counters) return false;
    p->n_groups = n_groups;
    p->blocks = 32u * ((n_groups + 7) / 8);                    // whole groups on every XCD; surplus groups return at once
    p->row_groups = (uint32_t)((m + 31) / 32);
    p->workspace_bytes = (uint64_t)n_groups * 4 * p->row_groups * (2 * 4 * 4 * 64 * 4);
    p->local = g_skinny_ksplit == 3 || ((g_skinny_ksplit == 0) && sk->xcd_local);
    return true;
}
}  // namespace

// Whether a linear of m rows takes a weight-stationary kernel: more rows than the decode kernels hold, a weight
// with at most about two column tiles per compute unit, k within what a wavefront keeps in registers, and a block's
// activation bytes (m x k, read from L2 once per block) below what the tiled GEMM with its k split costs.  With a
// split-k area given, deep weights take the form that splits k over four blocks of an XCD.
bool linear_w8a8_rows_applies(uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus, const SplitKArea *sk) {
    if (g_rows_kernel == 1) return false;
    const uint64_t n_tiles = n_pad / 16, k_tiles = k_pad / 64;
    RowsKsplitPlan kp;
    if (rows_ksplit_plan(m, (uint32_t)n_tiles, (uint32_t)k_tiles, num_cus, sk, &kp)) return true;
    if (m <= 64 || n_tiles == 0 || k_tiles == 0 || k_tiles > 224) return false;
    if (g_rows_kernel == 2) return true;
    // measured against the tiled GEMM with its k split (both with their row quantizer, us): 4096 -> 4096 at 65 / 128 / 300 /
    // 512 rows 13.9 / 14.8 / 25.7 / 37.1 against 24.3 / 27.5 / 33.2 / 41.1; 14336 -> 4096 at 128 rows 36.9 against 41.5, at 200
    // rows 54.9 against 48.7: what it costs is the m x k bytes of activations every block pulls from L2
    return n_tiles <= 2 * (uint64_t)num_cus && m * k_pad <= (2ull << 20);
}

uint64_t linear_w8a8_rows_workspace_bytes(uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus, const SplitKArea *sk) {
    RowsKsplitPlan kp;
    return rows_ksplit_plan(m, (uint32_t)(n_pad / 16), (uint32_t)(k_pad / 64), num_cus, sk, &kp) ? kp.workspace_bytes : 0;
}

void linear_w8a8_rows(const int8_t *xq_tiled, const int8_t *w_tiles, uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad,
                      const EpilogueI8 &ep, int num_cus, hipStream_t s, const SplitKArea *sk, void *workspace,
                      uint64_t workspace_bytes) {
    if (m == 0 || n == 0) return;
    EpiI8 e{};
    e.sx = ep.sx;
    e.sw = ep.sw;
    e.bias = ep.bias;
    e.residual = ep.residual;
    e.acc_out = ep.acc_out;
    e.out = ep.out;
    e.out_bf16 = ep.out_bf16;
    const uint32_t n_tiles = (uint32_t)(n_pad / 16), k_tiles = (uint32_t)(k_pad / 64);
    RowsKsplitPlan kp;
    if (workspace && rows_ksplit_plan(m, n_tiles, k_tiles, num_cus, sk, &kp) && workspace_bytes >= kp.workspace_bytes) {
        KsplitPlan as_ks{};
        as_ks.s = 4;
        as_ks.n_groups = kp.n_groups;
        uint32_t *seen = xcc_seen_for(sk, as_ks);
        auto go = [&](auto ktw, auto ds, auto local) {
            w8a8_wstat_ksplit_kernel<decltype(ktw)::value, decltype(ds)::value, decltype(local)::value><<<kp.blocks, 512, 0, s>>>(
                xq_tiled, w_tiles, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, kp.n_groups, e, (int32_t *)workspace, sk->counters, seen,
                sk->fault);
        };
        using std::integral_constant;
        auto with_local = [&](auto ktw, auto ds) {
            if (kp.local) go(ktw, ds, std::true_type{});
            else go(ktw, ds, std::false_type{});
        };
        // k-tiles of a wavefront: a quarter of k over eight wavefronts, rounded up
        const uint32_t per_wave = ((k_tiles + 3) / 4 + 7) / 8;
        if (per_wave <= 4) with_local(integral_constant<int, 4>{}, integral_constant<int, 4>{});
        else with_local(integral_constant<int, 7>{}, integral_constant<int, 7>{});      // k_tiles <= 224
        return;
    }
    // two column tiles per block once there are more tiles than compute units (every activation tile then feeds two
    // multiplies), where the registers allow it
    const bool two = n_tiles > (uint32_t)num_cus && k_tiles <= 64;
    const unsigned grid = two ? (n_tiles + 1) / 2 : n_tiles;
    auto go = [&](auto ktw, auto ntw) {
        w8a8_wstat_kernel<decltype(ktw)::value, decltype(ntw)::value><<<grid, 512, 0, s>>>(xq_tiled, w_tiles, (uint32_t)m, (uint32_t)n,
                                                                                           n_tiles, k_tiles, e);
    };
    using std::integral_constant;
    if (two) {
        go(integral_constant<int, 8>{}, integral_constant<int, 2>{});
    } else {
        if (k_tiles <= 64) go(integral_constant<int, 8>{}, integral_constant<int, 1>{});
        else if (k_tiles <= 128) go(integral_constant<int, 16>{}, integral_constant<int, 1>{});
        else go(integral_constant<int, 28>{}, integral_constant<int, 1>{});
    }
}

// The q | k | v projection of a prompt pass of 65 to a few hundred rows on the weight-stationary kernel with RoPE, the
// bf16 rounding and the K / V append in its epilogue (w8a8_wstat_kernel<8, 2, true>: a block per pair of tiles that the
// rotation pairs).  Applies where linear_w8a8_rows would take the unsplit kernel and a wavefront holds its k-tiles.
bool linear_w8a8_qkv_rope_rows_applies(uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus, const SplitKArea *sk,
                                       const QkvRopeTargets &t) {
    if (g_rows_rope == 1 || k_pad == 0 || k_pad / 64 > 64 || t.head_dim == 0 || t.head_dim % 32 != 0) return false;
    const uint64_t n = (uint64_t)(t.heads + 2 * t.kv_heads) * t.head_dim;
    if (n == 0 || n != n_pad) return false;
    RowsKsplitPlan kp;
    if (rows_ksplit_plan(m, (uint32_t)(n_pad / 16), (uint32_t)(k_pad / 64), num_cus, sk, &kp)) return false;
    return linear_w8a8_rows_applies(m, n_pad, k_pad, num_cus, sk);
}
void linear_w8a8_qkv_rope_rows(const int8_t *xq_tiled, const int8_t *w_tiles, const float *sx, const float *sw, uint64_t m,
                               uint64_t n_pad, uint64_t k_pad, const QkvRopeTargets &t, hipStream_t s) {
    if (m == 0) return;
    const uint32_t n = (t.heads + 2 * t.kv_heads) * t.head_dim;
    EpiI8 e{};
    e.sx = sx;
    e.sw = sw;
    e.cos_sin = t.cos_sin;
    e.slots = t.slots;
    e.q_out = t.q_out;
    e.k_pool = t.k_pool;
    e.v_pool = t.v_pool;
    e.heads = t.heads;
    e.kv_heads = t.kv_heads;
    e.head_dim = t.head_dim;
    e.pool_rows = t.pool_rows;
    w8a8_wstat_kernel<8, 2, true><<<n / 32, 512, 0, s>>>(xq_tiled, w_tiles, (uint32_t)m, n, (uint32_t)(n_pad / 16),
                                                       (uint32_t)(k_pad / 64), e);
}

void linear_w8a8_swiglu_skinny(const int8_t *xq_tiled, const int8_t *w_tiles, const float *sx, const float *sw,
                               uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad, float *act, float *pmax,
                               int waves, int num_cus, hipStream_t s, const RowPrologue *pro) {
    if (m == 0 || n == 0) return;
    uint32_t n_tiles = (uint32_t)(n_pad / 16), k_tiles = (uint32_t)(k_pad / 64);
    if (g_skinny_waves) waves = g_skinny_waves;
    EpiI8 e{};
    e.sx = sx;
    e.sw = sw;
    e.out = act;
    e.pmax = pmax;
    if (pro) {                                              // the caller asked swiglu_fuses_norm first
        unsigned blocks = (unsigned)std::min<uint64_t>(n_tiles / 2, (uint64_t)num_cus);
        w8a8_astat_kernel<1, 8, kEpiSwiglu, 1><<<blocks, 512, prologue_lds_bytes(m, k_pad), s>>>(
            nullptr, w_tiles, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, n_tiles / 2, e, *pro);
        return;
    }
    if (m <= 32 && astat_applies(n_tiles / 2, k_tiles, num_cus)) {
        unsigned blocks = (unsigned)std::min<uint64_t>(n_tiles / 2, (uint64_t)num_cus);
        if (m <= 16)
            w8a8_astat_kernel<1, 8, kEpiSwiglu><<<blocks, 512, 0, s>>>(xq_tiled, w_tiles, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, n_tiles / 2, e, RowPrologue{});
        else
            w8a8_astat_kernel<2, 8, kEpiSwiglu><<<blocks, 512, 0, s>>>(xq_tiled, w_tiles, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, n_tiles / 2, e, RowPrologue{});
        return;
    }
    if (astat_wide_applies(m, n_tiles / 2, k_tiles, num_cus)) {
        launch_astat_wide<kEpiSwiglu>(m, (unsigned)std::min<uint64_t>(n_tiles / 2, (uint64_t)num_cus), s, xq_tiled, w_tiles, (uint32_t)n,
                                      n_tiles, k_tiles, n_tiles / 2, e);
        return;
    }
    launch_w8a8_rows<2, kEpiSwiglu>(m, waves, n_tiles / 2, s, xq_tiled, w_tiles, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, e);
}

void linear_w8a8_qkv_rope_skinny(const int8_t *xq_tiled, const int8_t *w_tiles, const float *sx, const float *sw,
                                 uint64_t m, uint64_t n_pad, uint64_t k_pad, const QkvRopeTargets &t, hipStream_t s,
                                 const RowPrologue *pro) {
    if (m == 0) return;
    uint32_t n = (t.heads + 2 * t.kv_heads) * t.head_dim;
    uint32_t n_tiles = (uint32_t)(n_pad / 16), k_tiles = (uint32_t)(k_pad / 64);
    EpiI8 e{};
    e.sx = sx;
    e.sw = sw;
    e.cos_sin = t.cos_sin;
    e.slots = t.slots;
    e.q_out = t.q_out;
    e.k_pool = t.k_pool;
    e.v_pool = t.v_pool;
    e.heads = t.heads;
    e.kv_heads = t.kv_heads;
    e.head_dim = t.head_dim;
    e.pool_rows = t.pool_rows;
    unsigned grid = n / 32;                                  // one block per pair of 16-column tiles
    if (pro) {                                               // the caller asked qkv_rope_fuses_norm first
        w8a8_skinny_kernel<1, 2, 8, kEpiRope, 1><<<grid, 512, prologue_lds_bytes(m, k_pad), s>>>(nullptr, w_tiles, (uint32_t)m, n, n_tiles,
                                                                                              k_tiles, e, *pro);
        return;
    }
    int waves = g_skinny_waves ? g_skinny_waves : 8;
    launch_w8a8_rows<2, kEpiRope>(m, waves, grid, s, xq_tiled, w_tiles, (uint32_t)m, n, n_tiles, k_tiles, e);
}

void linear_e4m3_skinny(const uint8_t *aq, const uint8_t *w_tiles, const float *sx, const float *sw, const float *bias,
                        uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad, void *out, int out_bf16, hipStream_t s) {
    if (m == 0 || n == 0) return;
    const uint32_t n_tiles = (uint32_t)(n_pad / 16), k_tiles = (uint32_t)(k_pad / 128);
    auto go = [&](auto mt) {
        constexpr int MT = decltype(mt)::value;
        if (k_tiles >= 16)
            e4m3_skinny_kernel<MT, 8><<<n_tiles, 512, 0, s>>>(aq, w_tiles, sx, sw, bias, (uint32_t)m, (uint32_t)n, k_tiles, out, out_bf16);
        else
            e4m3_skinny_kernel<MT, 4><<<n_tiles, 256, 0, s>>>(aq, w_tiles, sx, sw, bias, (uint32_t)m, (uint32_t)n, k_tiles, out, out_bf16);
    };
    if (m <= 16)
        go(std::integral_constant<int, 1>{});
    else if (m <= 32)
        go(std::integral_constant<int, 2>{});
    else if (m <= 48)
        go(std::integral_constant<int, 3>{});
    else
        go(std::integral_constant<int, 4>{});
}

void linear_w8a16_skinny(const uint16_t *a, const int8_t *w_tiles, const float *sw, uint64_t m, uint64_t n,
                         uint64_t n_pad, uint64_t k_pad, void *out, int out_bf16, int num_cus, hipStream_t s,
                         const SplitKArea *sk) {
    if (m == 0 || n == 0) return;
    uint32_t n_tiles = (uint32_t)(n_pad / 16), k_tiles = (uint32_t)(k_pad / 64);
    KsplitPlan kp;
    if (m > 4 && ksplit_plan(m, n_tiles, k_tiles, num_cus, sk, 2, &kp)) {
        ksplit_dispatch(m, kp, [&](auto mt, auto ss, auto d, auto local) {
            w8a16_ksplit_kernel<decltype(mt)::value, decltype(ss)::value, decltype(d)::value, decltype(local)::value>
                <<<kp.blocks, 512, 0, s>>>(a, w_tiles, sw, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, kp.n_groups, out, out_bf16,
                                           (float *)sk->partial, sk->counters, xcc_seen_for(sk, kp), sk->fault);
        });
        return;
    }
    // by shape only above 16 rows: with one row tile the activations are as small as the weight tile
    // and the block-per-tile kernel, which spreads over more wavefronts, measured faster
    if (astat_applies(n_tiles, k_tiles, num_cus) && !(g_skinny_ntw || g_skinny_waves) && (m > 16 || g_skinny_astat == 2)) {
        unsigned blocks = (unsigned)std::min<uint64_t>(n_tiles, (uint64_t)num_cus);
        if (m <= 16)
            w8a16_astat_kernel<1, 8><<<blocks, 512, 0, s>>>(a, w_tiles, sw, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, out, out_bf16);
        else
            w8a16_astat_kernel<2, 8><<<blocks, 512, 0, s>>>(a, w_tiles, sw, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, out, out_bf16);
        return;
    }
    int ntw, waves;
    pick_config(n_tiles, k_tiles, num_cus, &ntw, &waves);
    if (m <= 16)
        launch_w8a16<1>(a, w_tiles, sw, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, out, out_bf16, ntw, waves, s);
    else
        launch_w8a16<2>(a, w_tiles, sw, (uint32_t)m, (uint32_t)n, n_tiles, k_tiles, out, out_bf16, ntw, waves, s);
}

}  // namespace k
}  // namespace fa
