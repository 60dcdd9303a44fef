// Prefill-shape quantized GEMMs on the CDNA4 matrix cores:
//   int8 : v_mfma_i32_16x16x64_i8, int32 accumulators, dequant epilogue
//   e4m3 : v_mfma_scale_f32_16x16x128_f8f6f4 (unit block scales), f32 accumulators
// The weight arrives in tile order (kernels.hpp), i.e. already in the byte
// order a wavefront needs for the B operand; activations are row-major and
// are re-ordered into the same tile order on their way into LDS.  Both operand
// tiles are double-buffered in LDS; every LDS read is a conflict-free 16-byte
// read at lane * 16.
#include <algorithm>
#include <type_traits>
#include <utility>

#include "device_utils.hpp"
#include "index_models.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {
using namespace fa::dev;

int g_gemm_small_tiles = 0;   // tuning: nonzero keeps the 128 x 128 kernel for every shape
extern int g_skinny_ksplit;   // kern_qlinear.hip
int g_gemm_pair = 0;          // tuning, 256 x 128 tiles of the large-tile kernel: 1 keeps one block per tile, 2 shares a tile
                              // only where the tiles alone would cover half the device
int g_gemm_swiglu = 0;        // tuning, prompt passes: bit 0 keeps SwiGLU out of the gate | up GEMM's epilogue, bit 1 RoPE
                              // and the K / V append out of the q | k | v GEMM's
int g_gemm_waves = 0;
int g_gemm_split_fill = 0;    // tuning: blocks per compute unit a split-k launch aims for (default 2)
int g_gemm_ntb = 0;           // tuning: 14 or 16 fixes the column tiles per large-tile block         // tuning: 4 = four wavefronts per large-tile block instead of eight

namespace {

struct EpiI8 {
    const float *sx, *sw, *bias, *residual;
    int32_t *acc_out;
    void *out;
    int out_bf16;
    // Large-tile kernel, k split over split_s = 2 or 4 blocks (split_partial != null): blocks b, b + 8, ... of a launch
    // (one XCD) own one output tile and a share of k each; all leave their raw sums in split_partial, wait for their
    // stores and take a ticket from the tile's counter, and the one that draws the last ticket adds the others' sums
    // (int32: exact in any order) and runs the epilogue.  split_local: the exchange stays in the XCD's L2.
    int32_t *split_partial = nullptr;
    uint32_t *split_counters = nullptr;
    int split_local = 0;
    uint32_t split_s = 2;
};
// int8, large-tile kernel only: the weight is gate | up (f columns each) and the kernel leaves silu(gate) * up, f32 [m, f]
struct EpiI8Swiglu {
    const float *sx, *sw;
    float *out;
    uint32_t f;
};
// int8, large-tile kernel only: the weight is q | k | v (heads of 128 dims) and the kernel leaves what the plain GEMM followed
// by the RoPE + append pass leaves: q rotated, bf16 [m, heads * 128]; K rotated and V as they are, bf16, in pool row slots[r]
struct EpiI8QkvRope {
    const float *sx, *sw, *cos_sin;
    const uint32_t *slots;
    uint16_t *q_out, *k_pool, *v_pool;
    uint32_t heads, kv_heads;
    uint64_t pool_rows;
};
struct EpiF8 {
    const float *a_scale, *w_scale;   // one scale each (per-tensor form) ...
    void *out;
    int out_bf16;
    const float *sx, *sw, *bias;      // ... or, when sx is set, one per row and one per column (+ optional bias)
};

constexpr int BM = 128, BN = 128;      // block tile; 4 wavefronts in 2 x 2, 64 x 64 each
constexpr int MT = BM / 16, NT = BN / 16;

// FP8 = false: k-tile of 64 int8 (1 KiB operand tiles, 16 B per lane)
// FP8 = true : k-tile of 128 e4m3 (2 KiB operand tiles, 32 B per lane)
template <bool FP8>
struct Cfg {
    static constexpr int TK = FP8 ? 128 : 64;
    static constexpr int CH = TK / 4;              // bytes per lane per operand tile
    static constexpr int TILE = 64 * CH;           // bytes per operand tile
};

template <bool FP8, typename Epi>
__global__ void __launch_bounds__(256)
    gemm_mfma_kernel(const uint8_t *__restrict__ aq, const uint8_t *__restrict__ w_tiles, uint32_t m, uint32_t n,
                     uint32_t n_tiles, uint32_t k_tiles, Epi ep, int32_t *__restrict__ partial) {
    using C = Cfg<FP8>;
    constexpr int TK = C::TK, CH = C::CH, TILE = C::TILE;
    constexpr int VPL = CH / 16;                    // 16-byte vectors per lane chunk
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][MT * TILE];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[2][NT * TILE];

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int wm = wave / 2, wn = wave % 2;
    const uint32_t m0 = blockIdx.y * BM, nt0 = blockIdx.x * NT;
    const uint64_t k_bytes = (uint64_t)k_tiles * TK;
    // split k: block z of gridDim.z covers k tiles [kt_lo, kt_hi) and leaves raw int32 sums in its own
    // slice of `partial`; a second kernel adds the slices (exactly) and applies the epilogue
    const uint32_t kt_lo = (uint32_t)((uint64_t)k_tiles * blockIdx.z / gridDim.z);
    const uint32_t kt_hi = (uint32_t)((uint64_t)k_tiles * (blockIdx.z + 1) / gridDim.z);

    // global -> register staging: A has BM rows x TK bytes = MT*TILE bytes,
    // i.e. MT*64 lane chunks of CH bytes; thread t moves chunks t, t+256, ...
    constexpr int A_CHUNKS = MT * 64 / 256;         // chunks per thread (2)
    constexpr int B_CHUNKS = NT * 64 / 256;
    v4u a_stage[A_CHUNKS][VPL], b_stage[B_CHUNKS][VPL];

    auto load_stage = [&](uint32_t kt) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            int chunk = tid + i * 256;                // = mt*64 + g*16 + r
            int mt = chunk / 64, g = (chunk / 16) % 4, r = chunk % 16;
            uint32_t row = m0 + mt * 16 + r;
#pragma unroll
            for (int v = 0; v < VPL; ++v) a_stage[i][v] = v4u{0, 0, 0, 0};
            if (row < m) {
                const v4u *src = (const v4u *)(aq + (uint64_t)row * k_bytes + (uint64_t)kt * TK + g * CH);
#pragma unroll
                for (int v = 0; v < VPL; ++v) a_stage[i][v] = src[v];
            }
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i) {
            int chunk = tid + i * 256;                // = nt*64 + lane chunk
            int nt = chunk / 64, lc = chunk % 64;
#pragma unroll
            for (int v = 0; v < VPL; ++v) b_stage[i][v] = v4u{0, 0, 0, 0};
            if (nt0 + nt < n_tiles) {
                const v4u *src = (const v4u *)(w_tiles + ((uint64_t)(nt0 + nt) * k_tiles + kt) * TILE + lc * CH);
#pragma unroll
                for (int v = 0; v < VPL; ++v) b_stage[i][v] = src[v];
            }
        }
    };
    auto store_stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            int chunk = tid + i * 256;
#pragma unroll
            for (int v = 0; v < VPL; ++v) *(v4u *)(&lds_a[buf][chunk * CH + v * 16]) = a_stage[i][v];
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i) {
            int chunk = tid + i * 256;
#pragma unroll
            for (int v = 0; v < VPL; ++v) *(v4u *)(&lds_b[buf][chunk * CH + v * 16]) = b_stage[i][v];
        }
    };

    typedef typename std::conditional<FP8, v4f, v4i>::type acc_t;
    acc_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (FP8) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
            else acc[i][j] = v4i{0, 0, 0, 0};
        }

    if (kt_lo < kt_hi) {
        load_stage(kt_lo);
        store_stage(0);
    }
    __syncthreads();
    for (uint32_t kt = kt_lo; kt < kt_hi; ++kt) {
        int buf = (kt - kt_lo) & 1;
        if (kt + 1 < kt_hi) load_stage(kt + 1);
        if constexpr (FP8) {
            v8i a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = *(const v8i *)(&lds_a[buf][(wm * 4 + i) * TILE + lane * CH]);
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = *(const v8i *)(&lds_b[buf][(wn * 4 + j) * TILE + lane * CH]);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i], b[j], acc[i][j], 0, 0, 0,
                                                                                 0x7f7f7f7f, 0, 0x7f7f7f7f);
        } else {
            v4i a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = *(const v4i *)(&lds_a[buf][(wm * 4 + i) * TILE + lane * CH]);
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = *(const v4i *)(&lds_b[buf][(wn * 4 + j) * TILE + lane * CH]);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < kt_hi) store_stage(buf ^ 1);     // the other buffer was last read one iteration ago
        __syncthreads();
    }

    // epilogue: lane l holds column l % 16 and rows 4 * (l / 16) + e of each 16 x 16 tile
    const int g = lane / 16, c = lane % 16;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                uint32_t row = m0 + (wm * 4 + i) * 16 + 4 * g + e;
                uint32_t col = (nt0 + wn * 4 + j) * 16 + c;
                if (row >= m || col >= n) continue;
                uint64_t o = (uint64_t)row * n + col;
                float v;
                if constexpr (!FP8) {
                    if (partial) {
                        partial[(uint64_t)blockIdx.z * m * n + o] = acc[i][j][e];
                        continue;
                    }
                }
                if constexpr (FP8) {
                    if (ep.sx) {
                        v = __fmul_rn(acc[i][j][e], __fmul_rn(ep.sx[row], ep.sw[col]));
                        if (ep.bias) v = __fadd_rn(v, ep.bias[col]);
                    } else {
                        v = __fmul_rn(acc[i][j][e], __fmul_rn(*ep.a_scale, *ep.w_scale));
                    }
                } else {
                    if (ep.acc_out) ep.acc_out[o] = acc[i][j][e];
                    v = __fmul_rn((float)acc[i][j][e], __fmul_rn(ep.sx[row], ep.sw[col]));
                    if (ep.bias) v = __fadd_rn(v, ep.bias[col]);
                    if (ep.residual) v = __fadd_rn(ep.residual[o], v);
                }
                if (ep.out_bf16)
                    ((uint16_t *)ep.out)[o] = f32_to_bf16(v);
                else
                    ((float *)ep.out)[o] = v;
            }
}

// Second half of a split-k int8 GEMM: adds the `splits` slices of raw sums (int32, exact in any order) and
// applies the same epilogue arithmetic as the kernel above.  One thread per four consecutive columns.
__global__ void __launch_bounds__(256)
    splitk_epilogue_i8_kernel(const int32_t *__restrict__ partial, uint32_t splits, uint32_t m, uint32_t n, EpiI8 ep) {
    const uint64_t quads_per_row = (n + 3) / 4, total = (uint64_t)m * quads_per_row;
    for (uint64_t q = (uint64_t)blockIdx.x * 256 + threadIdx.x; q < total; q += (uint64_t)gridDim.x * 256) {
        const uint32_t row = (uint32_t)(q / quads_per_row), c0 = (uint32_t)(q % quads_per_row) * 4;
        const uint64_t o0 = (uint64_t)row * n + c0;
        int32_t acc[4] = {0, 0, 0, 0};
        const bool vec = (n % 4 == 0);                       // then o0 is a multiple of 4: 16-byte loads
        for (uint32_t z = 0; z < splits; ++z) {
            const int32_t *src = partial + (uint64_t)z * m * n + o0;
            if (vec) {
                v4i v = *(const v4i *)src;
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] += v[e];
            } else {
                for (int e = 0; e < 4 && c0 + e < n; ++e) acc[e] += src[e];
            }
        }
        const float sx = ep.sx[row];
        for (int e = 0; e < 4 && c0 + e < n; ++e) {
            const uint32_t col = c0 + e;
            const uint64_t o = o0 + e;
            if (ep.acc_out) ep.acc_out[o] = acc[e];
            float v = __fmul_rn((float)acc[e], __fmul_rn(sx, ep.sw[col]));
            if (ep.bias) v = __fadd_rn(v, ep.bias[col]);
            if (ep.residual) v = __fadd_rn(ep.residual[o], v);
            if (ep.out_bf16)
                ((uint16_t *)ep.out)[o] = f32_to_bf16(v);
            else
                ((float *)ep.out)[o] = v;
        }
    }
}

// Matrix instructions with the accumulator pinned to the accumulation registers ("+a"): with 256
// accumulator registers per lane the register allocator otherwise shuffles tiles between the two
// register files around every instruction.  Same instructions as the builtins emit.  volatile keeps
// them in program order, ahead of the drain that precedes the epilogue.
__device__ __forceinline__ void mfma_acc(v4i &c, const v4i &a, const v4i &b) {
    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_acc(v4f &c, const v8i &a, const v8i &b) {
    const int unit = 0x7f7f7f7f;                      // block scales 2^0
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0]"
                 : "+a"(c)
                 : "v"(a), "v"(b), "v"(unit));
}

// Waits until the matrix pipeline has retired everything issued before, and ties the accumulators of one
// row of tiles to that point (they are in/out operands, so no read of them can be placed ahead of it).
template <typename T>
__device__ __forceinline__ void drain_row(T (&r)[7]) {
    asm volatile("s_nop 15\n\ts_nop 15"
                 : "+a"(r[0]), "+a"(r[1]), "+a"(r[2]), "+a"(r[3]), "+a"(r[4]), "+a"(r[5]), "+a"(r[6]));
}
template <typename T>
__device__ __forceinline__ void drain_row(T (&r)[4]) {
    asm volatile("s_nop 15\n\ts_nop 15" : "+a"(r[0]), "+a"(r[1]), "+a"(r[2]), "+a"(r[3]));
}
template <typename T>
__device__ __forceinline__ void drain_row(T (&r)[8]) {
    asm volatile("s_nop 15\n\ts_nop 15"
                 : "+a"(r[0]), "+a"(r[1]), "+a"(r[2]), "+a"(r[3]), "+a"(r[4]), "+a"(r[5]), "+a"(r[6]), "+a"(r[7]));
}

// LDS fragment reads and the waits for them, as assembly, for the large-tile kernel's main loop.  A read's result
// may only be touched after an lds_wait that names it: the wait takes the registers as in/out operands, so every
// use the compiler sees comes after it.  addr is an LDS byte address, OFF an immediate offset below 65536.
template <int OFF>
__device__ __forceinline__ void lds_read16(v4i &dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
// At most N LDS reads issued before this point are still outstanding afterwards (N = 0 emits no instruction: the
// caller has just waited for all of them).
template <int N>
__device__ __forceinline__ void lds_wait(v4i &x, v4i &y) {
    if constexpr (N == 0) asm volatile("" : "+v"(x), "+v"(y));
    else asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(x), "+v"(y) : "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_wait_all_a(v4i (&a)[2][2], v4i (&b)[2]) {
    asm volatile("s_waitcnt lgkmcnt(%6)"
                 : "+v"(a[0][0]), "+v"(a[0][1]), "+v"(a[1][0]), "+v"(a[1][1]), "+v"(b[0]), "+v"(b[1])
                 : "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_wait_all_a(v4i (&a)[4][2], v4i (&b)[2]) {
    asm volatile("s_waitcnt lgkmcnt(%10)"
                 : "+v"(a[0][0]), "+v"(a[0][1]), "+v"(a[1][0]), "+v"(a[1][1]), "+v"(a[2][0]), "+v"(a[2][1]), "+v"(a[3][0]),
                   "+v"(a[3][1]), "+v"(b[0]), "+v"(b[1])
                 : "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_wait_all_a(v4i (&a)[8][2], v4i (&b)[2]) {
    asm volatile("s_waitcnt lgkmcnt(%18)"
                 : "+v"(a[0][0]), "+v"(a[0][1]), "+v"(a[1][0]), "+v"(a[1][1]), "+v"(a[2][0]), "+v"(a[2][1]), "+v"(a[3][0]),
                   "+v"(a[3][1]), "+v"(a[4][0]), "+v"(a[4][1]), "+v"(a[5][0]), "+v"(a[5][1]), "+v"(a[6][0]), "+v"(a[6][1]),
                   "+v"(a[7][0]), "+v"(a[7][1]), "+v"(b[0]), "+v"(b[1])
                 : "n"(N));
}
template <int... I, typename F>
__device__ __forceinline__ void static_for_seq(std::integer_sequence<int, I...>, F &&f) {
    (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant expression
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_seq(std::make_integer_sequence<int, N>{}, f);
}

// ------------------------------------------------------------ large tiles
// Block tile 256 rows x NTB * 16 columns, four wavefronts in 2 x 2, one per
// SIMD, each owning 128 rows x NTB / 2 column tiles of accumulators (up to 256
// registers).  Per k-step a wavefront reads 8 A fragments once and streams its
// B fragments past them, so the LDS traffic per matrix instruction is a quarter
// of the 64 x 64 wavefront tile above, which is what lets the matrix cores run
// instead of waiting on LDS.  Rows / tiles past the edge are loaded from a
// clamped address (never stored), so the main loop has no predicated loads.
// The block index is remapped so that the blocks that land on one XCD (the
// hardware deals consecutive block ids round-robin over the 8 XCDs) are
// consecutive tiles, m fastest: they share one B panel and walk k together,
// which keeps the panel in that XCD's L2.
template <bool FP8, int NTB, int WM, typename Epi>
__global__ void __launch_bounds__(128 * WM) __attribute__((amdgpu_waves_per_eu(WM / 2, WM / 2)))
    gemm_mfma_big_kernel(const uint8_t *__restrict__ aq, const uint8_t *__restrict__ w_tiles, uint32_t m, uint32_t n,
                         uint32_t n_tiles, uint32_t k_steps, uint32_t m_blocks, uint32_t n_blocks, Epi ep) {
    // One stage is 128 bytes of k for both types: one e4m3 instruction step, or two int8 steps (two
    // adjacent 1 KiB weight tiles).  Fewer, larger stages halve the per-stage fixed cost (barrier, load
    // issue, first fragment reads) for int8 and let its A rows be fetched as whole 128-byte lines.
    constexpr int TK = 128, TILE = 2048;             // bytes of k per stage; bytes per operand tile and stage
    constexpr int WNT = NTB / 2;                     // column tiles per wavefront
    constexpr int NWAVES = 2 * WM;                   // WM wavefronts along m, 2 along n
    constexpr int AI = 16 / WM;                      // row tiles per wavefront
    constexpr int TPW = 16 / NWAVES;                 // operand tiles each wavefront moves per stage
    constexpr int A_STAGE = 16 * TILE, B_STAGE = NTB * TILE;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];   // [3][A_STAGE] then [2][B_STAGE]

    constexpr bool SWI = std::is_same<Epi, EpiI8Swiglu>::value, ROPE = std::is_same<Epi, EpiI8QkvRope>::value;
    static_assert(!SWI || (!FP8 && NTB % 4 == 0), "the SwiGLU form pairs gate and up tiles inside a wavefront");
    static_assert(!ROPE || (!FP8 && NTB == 16), "the RoPE form: a head of 128 dims is the eight column tiles of one wavefront");
    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int wm = wave / 2, wn = wave % 2;
    uint32_t mb, nb;
    uint32_t tile_id = blockIdx.x, half = 0, ks_lo = 0, ks_n = k_steps;
    [[maybe_unused]] bool split = false;
    if constexpr (std::is_same<Epi, EpiI8>::value) {
        if (ep.split_partial) {
            split = true;
            ixm::ksplit_block(blockIdx.x, ep.split_s, &tile_id, &half);      // partners b, b + 8, ...: one XCD
            if (tile_id >= m_blocks * n_blocks) return;               // the same for all partners
            uint32_t ks_hi;
            ixm::ksplit_k_range(k_steps, half, ep.split_s, &ks_lo, &ks_hi);
            ks_n = ks_hi - ks_lo;
        }
    }
    ixm::big_block_tile(tile_id, m_blocks, n_blocks, &mb, &nb);
    const uint32_t m0 = mb * 256, nt0 = nb * NTB;
    const uint64_t k_bytes = (uint64_t)k_steps * TK;

    // Global -> LDS without passing through registers: one load instruction moves 16 bytes per lane to
    // LDS base + lane * 16, i.e. one 1 KiB slice of an operand tile in the matrix instruction's lane
    // order; a tile of a stage is two slices h = 0, 1.  e4m3: slice h holds bytes 16 h .. 16 h + 15 of every
    // lane's 32-byte chunk.  int8: slice h is the operand tile of k-step h of the stage.
    // Wavefront w moves tiles w, w + 4, w + 8, w + 12 of A and of B.  Rows / tiles past the edge are loaded
    // from a clamped address and never stored.
    // A rows are row-major in memory: a row's 128 bytes of a stage are eight 16-byte pieces q.  Load
    // instruction x takes the pieces with q % 2 == x, four consecutive lanes sharing one row, so every
    // lane quad touches one whole cache line per instruction (the L1 fetches it once; the second
    // instruction hits) instead of one line per lane.  Lane 4 r + p fills LDS slot 4 r + p of slice x; which
    // piece that is rotates with the row, so that the fragment reads spread over the LDS banks: e4m3's k-group g
    // of the matrix instruction is pieces 2 g, 2 g + 1, kept in slot 4 r + (g + r / 2) mod 4 of both slices; int8's
    // k-group g of k-step s is the single piece 4 s + g in slice g % 2, kept in slot 4 r + (g + s + r / 2) mod 4
    // (the LDS serves sixteen lanes of a 16-byte read per cycle, the lanes of two neighbouring k-groups together:
    // their slots have to differ by an odd number, or the read runs at half rate).
    constexpr int B_H = FP8 ? 16 : 1024;             // byte offset of slice h in a stage's weight tile in memory
    static_assert(ixm::big_b_src_byte<FP8>(0, 1) == B_H && ixm::kBigTk == TK && ixm::kBigTile == TILE, "index model out of step");
    const uint8_t *a_src[TPW][2];
    const uint8_t *b_src[TPW];
    // (the index expressions live in index_models.hpp, where a host program checks them for every instantiation)
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
        uint32_t row = m0 + ixm::big_a_tile<NWAVES>(wave, i) * 16 + ixm::big_a_row(lane);
        row = row < m ? row : m - 1;
#pragma unroll
        for (int x = 0; x < 2; ++x) a_src[i][x] = aq + (uint64_t)row * k_bytes + (uint64_t)ks_lo * TK + ixm::big_a_src_byte<FP8>(lane, x);
        // a block of NTB = 14 has no tiles 14, 15: the wavefronts that would move them repeat tiles
        // 0, 1 instead (same bytes to the same place, served by the L1), which keeps the main loop
        // free of branches
        uint32_t t = nt0 + ixm::big_b_tile<NTB, NWAVES>(wave, i);
        if constexpr (SWI) t = ixm::big_swiglu_tile<NTB>(nb, ixm::big_b_tile<NTB, NWAVES>(wave, i), ep.f / 16);
        t = t < n_tiles ? t : n_tiles - 1;
        b_src[i] = w_tiles + ((uint64_t)t * k_steps + ks_lo) * TILE + ixm::big_b_src_byte<FP8>(lane, 0);
    }
    // byte offsets of this lane's two A operand reads inside a tile
    const int a_off[2] = {ixm::big_a_frag_off<FP8>(lane, 0), ixm::big_a_frag_off<FP8>(lane, 1)};
    // LDS holds three stages of A and two of B: A runs two stages ahead of the multiplies, B one, so that
    // requests stay in flight across the wait at the top of a stage (with both operands one stage ahead
    // the path from L2 runs dry there; a third stage of both does not fit).
    constexpr int NSA = 3, NSB = 2;
    // Load instruction `idx` of a stage: tile wave + NWAVES (idx / 2), slice idx % 2.  They are spread over
    // the multiply groups of the stage before, which keeps a steady stream of requests going to the L2
    // instead of one burst per stage.
    typedef __attribute__((address_space(1))) const void *gptr;
    typedef __attribute__((address_space(3))) void *lptr;
    auto issue_a = [&](uint32_t ks, int slot, int idx) {
        const int i = idx / 2, h = idx % 2;
        __builtin_amdgcn_global_load_lds((gptr)(a_src[i][h] + (uint64_t)ks * TK),
                                         (lptr)(lds + ixm::big_a_lds_slice<NTB>(slot, ixm::big_a_tile<NWAVES>(wave, i), h)), 16, 0, 0);
    };
    auto issue_b = [&](uint32_t ks, int slot, int idx) {
        const int i = idx / 2, h = idx % 2;
        __builtin_amdgcn_global_load_lds((gptr)(b_src[i] + (uint64_t)ks * TILE + h * B_H),
                                         (lptr)(lds + ixm::big_b_lds_slice<NTB>(slot, ixm::big_b_tile<NTB, NWAVES>(wave, i), h)), 16, 0, 0);
    };

    typedef typename std::conditional<FP8, v4f, v4i>::type acc_t;
    acc_t acc[AI][WNT];
#pragma unroll
    for (int i = 0; i < AI; ++i)
#pragma unroll
        for (int j = 0; j < WNT; ++j) {
            if constexpr (FP8) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
            else acc[i][j] = v4i{0, 0, 0, 0};
        }
    // the per-tensor scales of the e4m3 epilogue are fetched here, not after the last stage, where the two dependent
    // scalar loads would be a memory round trip that nothing overlaps
    [[maybe_unused]] float fscale = 0.0f;
    if constexpr (FP8) {
        if (ep.sx == nullptr) fscale = __fmul_rn(*ep.a_scale, *ep.w_scale);
    }

    // Per stage a wavefront issues its B loads of stage ks + 1 first and its A loads of stage ks + 2 after
    // them, so the wait at the top of stage ks + 1 can leave exactly those 2 TPW A loads outstanding.  Past
    // the end the loads are repeated from the last stage into slots nobody reads again, which keeps the
    // count of outstanding loads the same in every pass.
    constexpr int NLD = 2 * TPW;                     // A load instructions per wavefront and stage
    const uint32_t last = ks_n - 1;                  // stages are counted from the block's first one
#pragma unroll
    for (int idx = 0; idx < NLD; ++idx) issue_a(0, 0, idx);
#pragma unroll
    for (int idx = 0; idx < NLD; ++idx) issue_b(0, 0, idx);
#pragma unroll
    for (int idx = 0; idx < NLD; ++idx) issue_a(last < 1 ? last : 1, 1, idx);
    // The barrier that opens stage ks + 1 sits before the last multiply group of stage ks, and the first
    // fragments of stage ks + 1 (all of A, the first of B) are read under that group: with the barrier
    // at the top of a stage every wavefront of the block would wait there for its first fragments at
    // the same time, with the matrix cores idle.  Per stage:
    //   groups 0 .. WNT - 2: loads of B (stage ks + 1) and A (stage ks + 2), B fragment j + 1, multiplies j
    //   group WNT - 1: own reads of stage ks complete and own loads of stage ks + 1 landed, barrier,
    //                  multiplies interleaved with the A fragment reads of stage ks + 1, then its first B
    // The loads overwrite the buffers of stage ks - 1; they are issued after the barrier that opened
    // stage ks, which a wavefront reaches only after all its reads of stage ks - 1 have completed.
    int slot_a = 0;
    // Fragment reads are written as assembly with their own lgkmcnt waits (lds_read16 / lds_wait above): left to
    // the compiler, every wait for a fragment becomes lgkmcnt(0), which also waits for the fragment of the NEXT
    // group that was issued a moment earlier, and the read-ahead is lost.  Addresses are LDS byte offsets.
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr)lds;
    const uint32_t la_lane[2] = {lds0 + (wm * AI) * TILE + a_off[0], lds0 + (wm * AI) * TILE + a_off[1]};
    const uint32_t lb_lane = lds0 + NSA * A_STAGE + ixm::big_b_frag_off<NTB>(wn, 0, 0, lane);
    uint32_t la[2] = {la_lane[0], la_lane[1]};        // A fragment (i, sub) at la[sub] + i * TILE
    uint32_t lb = lb_lane;                            // B fragment j, slice h at lb + j * TILE + h * 1024
    __builtin_amdgcn_s_waitcnt(0x0F70 | NLD);         // stage 0 of this wavefront has landed (A of stage 1 may not)
    __builtin_amdgcn_s_barrier();                     // a bare barrier: __syncthreads would add a fence on top
    // B fragments go through three registers sets: group 0 of a stage multiplies from set 2, group j >= 1 from set
    // (j - 1) % 2.  Fragment j + 1 is read under the multiplies of group j, and fragment 0 of the next stage is read
    // into set 2 right behind the barrier that makes that stage visible, ahead of the last group's multiplies, so
    // no stage begins by waiting for an LDS read it has only just issued.  LDS reads complete in the order they were
    // issued, so with the two reads of fragment j + 1 the only younger ones, lgkmcnt(2) says fragment j (and, in
    // group 0, every A fragment) has arrived.
    v4i a[AI][2], b[3][2];                            // [..][slice]
    static_for<AI>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        lds_read16<i * TILE>(a[i][0], la[0]);
        lds_read16<i * TILE>(a[i][1], la[1]);
    });
    lds_read16<0>(b[2][0], lb);
    lds_read16<1024>(b[2][1], lb);
    uint32_t ks = 0;
    do {                                              // ks_n >= 1: the launcher sees to it
        const int buf = ks % NSB;
        const uint32_t ks_b = ks + 1 < last ? ks + 1 : last, ks_a = ks + 2 < last ? ks + 2 : last;
        const int slot_a2 = slot_a == 0 ? 2 : slot_a - 1;             // (slot_a + 2) % 3
        static_for<WNT>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            {
                // 2 NLD load instructions over the first multiply groups, B before A
                constexpr int PER = (2 * NLD + WNT - 3) / (WNT - 2);
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    const int idx = j * PER + q;
                    if (idx < NLD) issue_b(ks_b, buf ^ 1, idx);
                    else if (idx < 2 * NLD) issue_a(ks_a, slot_a2, idx - NLD);
                }
            }
            constexpr int cur = j == 0 ? 2 : (j - 1) % 2, nxt = j % 2;   // sets of group j and of group j + 1
            constexpr bool tail = j + 1 == WNT;
            if constexpr (!tail) {                    // next fragment under the multiplies
                lds_read16<(j + 1) * TILE>(b[nxt][0], lb);
                lds_read16<(j + 1) * TILE + 1024>(b[nxt][1], lb);
                if constexpr (j == 0) lds_wait_all_a<2>(a, b[cur]);
                else lds_wait<2>(b[cur][0], b[cur][1]);
            } else {
                // lgkmcnt(0), vmcnt(NLD): every read of stage ks by this wavefront is complete and its
                // loads of stage ks + 1 have landed (the A loads of stage ks + 2 may be outstanding)
                __builtin_amdgcn_s_waitcnt(0x0070 | NLD);
                lds_wait<0>(b[cur][0], b[cur][1]);    // no instruction: ties the fragment to the wait above
                __builtin_amdgcn_s_barrier();         // stage ks + 1 visible to all; stage ks no longer read
                slot_a = slot_a == 2 ? 0 : slot_a + 1;
                la[0] = la_lane[0] + slot_a * A_STAGE;
                la[1] = la_lane[1] + slot_a * A_STAGE;
                lb = lb_lane + (buf ^ 1) * B_STAGE;
                lds_read16<0>(b[2][0], lb);           // fragment 0 of the next stage (set 2 was last used by group 0)
                lds_read16<1024>(b[2][1], lb);
            }
            // past the last stage the tail's reads fetch stale, unused data
            if constexpr (FP8) {
                static_for<AI>([&](auto ic) {
                    constexpr int i = decltype(ic)::value;
                    const v4i &x0 = a[i][0], &x1 = a[i][1], &y0 = b[cur][0], &y1 = b[cur][1];
                    // weight fragment first: the accumulator tile comes out transposed (see the epilogue)
                    mfma_acc(acc[i][j], v8i{y0[0], y0[1], y0[2], y0[3], y1[0], y1[1], y1[2], y1[3]},
                             v8i{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]});
                    if constexpr (tail) {
                        lds_read16<i * TILE>(a[i][0], la[0]);
                        lds_read16<i * TILE>(a[i][1], la[1]);
                    }
                });
            } else {
                // the two k-steps of a tile are eight instructions apart, so no instruction waits for the
                // accumulator of the one before it
                static_for<2>([&](auto hc) {
                    constexpr int h = decltype(hc)::value;
                    static_for<AI>([&](auto ic) {
                        constexpr int i = decltype(ic)::value;
                        mfma_acc(acc[i][j], b[cur][h], a[i][h]);
                        if constexpr (tail) lds_read16<i * TILE>(a[i][h], la[h]);
                    });
                });
            }
        });
    } while (++ks < ks_n);
    // the reads the last pass issued for a stage that does not exist are still on their way to registers that are
    // dead from here on: hold those registers until the reads have written them
    lds_wait_all_a<0>(a, b[2]);
    // The compiler cannot see that the asm statements are matrix instructions, so it does not insert the
    // wait states their results need before other instructions read the accumulators (it may even peel
    // the last pass and start copying accumulators between its multiplies).  Every accumulator therefore
    // passes through a statement that waits out the matrix pipeline before anything else may read it.
#pragma unroll
    for (int i = 0; i < AI; ++i) drain_row(acc[i]);
    __builtin_amdgcn_s_waitcnt(0x0F70);               // the repeated loads of the tail have landed too

    if constexpr (std::is_same<Epi, EpiI8>::value) {
        if (split) {
            // raw sums of this half of k: word (i, j, e) of thread t at [(i * WNT + j) * 4 + e][t], 2 KiB per store
            constexpr int WORDS = AI * WNT * 4;
            const uint32_t S = ep.split_s;
            int32_t *mine = ep.split_partial + ((uint64_t)tile_id * S + half) * ((uint64_t)WORDS * 128 * WM);
            const bool local = ep.split_local != 0;
#pragma unroll
            for (int i = 0; i < AI; ++i)
#pragma unroll
                for (int j = 0; j < WNT; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        int32_t *p = mine + ((i * WNT + j) * 4 + e) * (128 * WM) + tid;
                        if (local) __hip_atomic_store(p, (int32_t)acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        else __hip_atomic_store(p, (int32_t)acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
            __builtin_amdgcn_s_waitcnt(0);            // this thread's stores are acknowledged
            __syncthreads();                          // ... and everybody's; nobody reads the stages any more
            uint32_t *slot = (uint32_t *)lds;
            if (tid == 0) {
                uint32_t *ctr = ep.split_counters + tile_id;
                const uint32_t t = local ? __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)
                                         : __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (t == S - 1) {                     // all are in: the counter returns to zero for the next launch
                    if (local) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    else __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                *slot = t;
            }
            __syncthreads();
            if (*slot != S - 1) return;               // a partner finishes the tile
            for (uint32_t r = 0; r < S; ++r) {
                if (r == half) continue;
                const int32_t *other = ep.split_partial + ((uint64_t)tile_id * S + r) * ((uint64_t)WORDS * 128 * WM);
#pragma unroll
                for (int i = 0; i < AI; ++i)
#pragma unroll
                    for (int j = 0; j < WNT; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int32_t *p = other + ((i * WNT + j) * 4 + e) * (128 * WM) + tid;
                            acc[i][j][e] += local ? __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)
                                                  : __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
            }
        }
    }

    // Epilogue.  The matrix instructions took the weight fragment as their first operand, so an accumulator tile is
    // the transpose of the usual one: lane l holds row l % 16 of the output tile and its columns 4 (l / 16) + e,
    // e = 0 .. 3: four consecutive outputs of one row, which leave as one 8-byte (bf16) or 16-byte (f32) store
    // without passing through LDS, the activation scale is one value per lane and row tile, and the channel scales
    // of a tile are one 16-byte load.  Two bf16 roundings are one v_cvt_pk_bf16_f32.
    int row_l0, col_l0;                               // block-local row of this lane in row tile 0, first column in tile 0
    ixm::big_out_elem<NTB, WM>(wm, wn, 0, 0, 0, lane, &row_l0, &col_l0);
    const int g = lane / 16;
    if constexpr (ROPE) {
        // The eight column tiles of this wavefront are head hd = 2 nb + wn of q | k | v; tiles j and j + 4 hold dims d
        // and d + 64 of the rotate-half pairs (four consecutive d per lane).  The arithmetic is rope_append's: dequantize,
        // x0 c - x1 s and x1 c + x0 s with explicit roundings, one rounding to bf16.
        const uint32_t hd = nb * 2 + wn, heads = ep.heads, kv = ep.kv_heads;
        const uint64_t eq = (uint64_t)heads * 128, ekv = (uint64_t)kv * 128;
        const uint32_t c0 = hd * 128 + 4 * g;                              // this lane's first column in tile 0
        v4f sw0[4], sw1[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            sw0[j] = *(const v4f *)(ep.sw + c0 + j * 16);
            sw1[j] = *(const v4f *)(ep.sw + c0 + 64 + j * 16);
        }
#pragma unroll
        for (int i = 0; i < AI; ++i) {
            const uint32_t row = m0 + row_l0 + i * 16;
            const bool row_ok = row < m;
            const uint32_t rc = row_ok ? row : m - 1;
            const float sxr = ep.sx[rc];
            uint16_t *dst = nullptr;
            if (hd < heads) {
                dst = ep.q_out + (uint64_t)rc * eq + (uint64_t)hd * 128;
            } else {
                const uint64_t slot = ep.slots[rc];
                if (slot < ep.pool_rows)
                    dst = hd < heads + kv ? ep.k_pool + slot * ekv + (uint64_t)(hd - heads) * 128
                                          : ep.v_pool + slot * ekv + (uint64_t)(hd - heads - kv) * 128;
            }
            const bool rotate = hd < heads + kv;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v4f cs = v4f{0.f, 0.f, 0.f, 0.f}, sn = cs;
                if (rotate) {
                    cs = *(const v4f *)(ep.cos_sin + (uint64_t)rc * 128 + j * 16 + 4 * g);
                    sn = *(const v4f *)(ep.cos_sin + (uint64_t)rc * 128 + 64 + j * 16 + 4 * g);
                }
                float y0[4], y1[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float x0 = __fmul_rn((float)acc[i][j][e], __fmul_rn(sxr, sw0[j][e]));
                    float x1 = __fmul_rn((float)acc[i][j + 4][e], __fmul_rn(sxr, sw1[j][e]));
                    if (rotate) {
                        const float r0 = __fsub_rn(__fmul_rn(x0, cs[e]), __fmul_rn(x1, sn[e]));
                        const float r1 = __fadd_rn(__fmul_rn(x1, cs[e]), __fmul_rn(x0, sn[e]));
                        x0 = r0;
                        x1 = r1;
                    }
                    y0[e] = x0;
                    y1[e] = x1;
                }
                if (row_ok && dst) {
                    *(v2u *)(dst + j * 16 + 4 * g) = v2u{f32x2_to_bf16x2(y0[0], y0[1]), f32x2_to_bf16x2(y0[2], y0[3])};
                    *(v2u *)(dst + 64 + j * 16 + 4 * g) = v2u{f32x2_to_bf16x2(y1[0], y1[1]), f32x2_to_bf16x2(y1[2], y1[3])};
                }
            }
        }
        return;
    } else if constexpr (SWI) {
        // accumulator tiles j and j + WNT / 2 hold gate and up of product tile nb * NTB / 2 + wn * WNT / 2 + j: the
        // decode step's expressions (dequantize both, silu(gate) * up), four consecutive columns per lane
        constexpr int HT = WNT / 2;
        const uint32_t f = ep.f;
        const uint32_t hc0 = (nb * (NTB / 2) + wn * HT) * 16 + 4 * g;      // this lane's first product column
        v4f swg[HT], swu[HT];
#pragma unroll
        for (int j = 0; j < HT; ++j) {
            swg[j] = *(const v4f *)(ep.sw + hc0 + j * 16);
            swu[j] = *(const v4f *)(ep.sw + f + hc0 + j * 16);
        }
#pragma unroll
        for (int i = 0; i < AI; ++i) {
            const uint32_t row = m0 + row_l0 + i * 16;
            const bool row_ok = row < m;
            const float sxr = ep.sx[row_ok ? row : m - 1];
            float *orow = ep.out + (uint64_t)(row_ok ? row : m - 1) * f + hc0;
#pragma unroll
            for (int j = 0; j < HT; ++j) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float vg = __fmul_rn((float)acc[i][j][e], __fmul_rn(sxr, swg[j][e]));
                    const float vu = __fmul_rn((float)acc[i][j + HT][e], __fmul_rn(sxr, swu[j][e]));
                    v[e] = silu_f32(vg) * vu;
                }
                if (row_ok) *(v4f *)(orow + j * 16) = v4f{v[0], v[1], v[2], v[3]};
            }
        }
        return;
    } else {
    bool extras = false, raw_out = false;
    const bool out_bf16 = ep.out_bf16 != 0;
    bool f8_rows = false;
    const float *bias = nullptr, *residual = nullptr;
    if constexpr (FP8) {
        f8_rows = ep.sx != nullptr;
        extras = f8_rows && ep.bias != nullptr;
        if (extras) bias = ep.bias;
    } else {
        extras = ep.acc_out != nullptr || ep.bias != nullptr || ep.residual != nullptr;
        raw_out = ep.acc_out != nullptr;
        bias = ep.bias;
        residual = ep.residual;
    }
    const uint32_t col0 = (nt0 + wn * WNT) * 16;      // first column of this wavefront
    const bool full_cols = nt0 + wn * WNT + WNT <= n_tiles && col0 + WNT * 16 <= n;
    const bool row_scales = !FP8 || f8_rows;
    if (!raw_out && full_cols && n % 8 == 0) {
        // bias and residual are added in the order of the general form below: (product + bias), then residual + that
        v4f swc[WNT], bc[WNT];
#pragma unroll
        for (int j = 0; j < WNT; ++j) {
            if (row_scales) swc[j] = *(const v4f *)(ep.sw + col0 + j * 16 + 4 * g);
            if (bias) bc[j] = *(const v4f *)(bias + col0 + j * 16 + 4 * g);
        }
#pragma unroll
        for (int i = 0; i < AI; ++i) {
            const uint32_t row = m0 + row_l0 + i * 16;
            const bool row_ok = row < m;
            const float sxr = row_scales ? ep.sx[row_ok ? row : m - 1] : 0.0f;
            const uint64_t o0 = (uint64_t)(row_ok ? row : m - 1) * n + nt0 * 16 + col_l0;
            uint8_t *orow = (uint8_t *)ep.out + o0 * (out_bf16 ? 2 : 4);
            v4f res[WNT];
            if (residual) {
#pragma unroll
                for (int j = 0; j < WNT; ++j) res[j] = *(const v4f *)(residual + o0 + j * 16);
            }
            v2u pk[WNT];                              // bf16 output: the four columns of tile j, packed
#pragma unroll
            for (int j = 0; j < WNT; ++j) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if constexpr (FP8) v[e] = __fmul_rn(acc[i][j][e], f8_rows ? __fmul_rn(sxr, swc[j][e]) : fscale);
                    else v[e] = __fmul_rn((float)acc[i][j][e], __fmul_rn(sxr, swc[j][e]));
                    if (bias) v[e] = __fadd_rn(v[e], bc[j][e]);
                    if (residual) v[e] = __fadd_rn(res[j][e], v[e]);
                }
                if (out_bf16) pk[j] = v2u{f32x2_to_bf16x2(v[0], v[1]), f32x2_to_bf16x2(v[2], v[3])};
                else if (row_ok) *(v4f *)(orow + j * 64) = v4f{v[0], v[1], v[2], v[3]};
            }
            if (out_bf16) {
                // Two tiles at a time, the lanes of column groups g = 1, 3 trade their four columns of the first tile
                // for the four columns that groups g - 1 hold of the second (v_permlane16_swap: rows of sixteen lanes
                // 1, 3 of one register against rows 0, 2 of the other).  Then g = 0, 2 hold columns 0 .. 7 and 8 .. 15
                // of the first tile and g = 1, 3 those of the second: one 16-byte store per lane, 64 contiguous bytes
                // per output row and instruction instead of 32.
#pragma unroll
                for (int j = 0; j + 1 < WNT; j += 2) {
                    const auto lo = __builtin_amdgcn_permlane16_swap(pk[j][0], pk[j + 1][0], false, false);
                    const auto hi = __builtin_amdgcn_permlane16_swap(pk[j][1], pk[j + 1][1], false, false);
                    if (row_ok) *(v4u *)(orow - 8 * g + (j + (g & 1)) * 32 + (g >> 1) * 16) = v4u{lo[0], hi[0], lo[1], hi[1]};
                }
                if (WNT % 2 == 1 && row_ok) *(v2u *)(orow + (WNT - 1) * 32) = pk[WNT - 1];
            }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < WNT; ++j) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t col = (nt0 + wn * WNT + j) * 16 + 4 * g + e;
            const bool col_ok = col < n && nt0 + wn * WNT + j < n_tiles;
            float swc = 0.0f;
            if (row_scales) swc = col_ok ? ep.sw[col] : 0.0f;
#pragma unroll
            for (int i = 0; i < AI; ++i) {
                const uint32_t row = m0 + row_l0 + i * 16;
                if (col_ok && row < m) {
                    const uint64_t o = (uint64_t)row * n + col;
                    float v;
                    if constexpr (FP8) {
                        v = __fmul_rn(acc[i][j][e], f8_rows ? __fmul_rn(ep.sx[row], swc) : fscale);
                        if (extras) v = __fadd_rn(v, ep.bias[col]);
                    } else {
                        v = __fmul_rn((float)acc[i][j][e], __fmul_rn(ep.sx[row], swc));
                        if (extras) {                  // uniform: raw accumulators, bias, residual
                            if (ep.acc_out) ep.acc_out[o] = acc[i][j][e];
                            if (ep.bias) v = __fadd_rn(v, ep.bias[col]);
                            if (ep.residual) v = __fadd_rn(ep.residual[o], v);
                        }
                    }
                    if (out_bf16)
                        ((uint16_t *)ep.out)[o] = f32_to_bf16(v);
                    else
                        ((float *)ep.out)[o] = v;
                }
            }
        }
    }
    }                                                 // !SWI
}

// Column tiles per block for the large-tile kernel: the width that leaves the fewest idle block slots
// in the last round over the compute units (0: the matrix is too small for it).
inline int pick_big_ntb(uint64_t m, uint64_t n_tiles, int num_cus) {
    if (m < 256 || n_tiles < 14) return 0;
    if (g_gemm_ntb == 14 || g_gemm_ntb == 16) return g_gemm_ntb;
    uint64_t mb = (m + 255) / 256;
    // a few hundred rows against a narrow weight: too few large tiles to keep the compute units' L2 ports
    // busy (each pulls operands at a fixed rate), the 128 x 128 kernel spreads the same bytes over more of them
    if (mb * ((n_tiles + 13) / 14) * 2 <= (uint64_t)num_cus) return 0;
    int best = 0;
    double best_cost = 0;
    for (int ntb : {16, 14}) {
        uint64_t blocks = mb * ((n_tiles + ntb - 1) / ntb);
        uint64_t rounds = (blocks + num_cus - 1) / num_cus;
        double cost = (double)rounds * ntb;           // time ~ rounds x tile width
        if (best == 0 || cost < best_cost) {
            best = ntb;
            best_cost = cost;
        }
    }
    return best;
}

template <bool FP8, int NTB, int WM, typename Epi>
void launch_big_wm(const uint8_t *aq, const uint8_t *w_tiles, uint64_t m, uint64_t n, uint64_t n_tiles, uint64_t k_steps,
                const Epi &e, hipStream_t s) {
    const size_t smem = (3 * 16 + 2 * (size_t)NTB) * 2048;          // three stages of A, two of B
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mfma_big_kernel<FP8, NTB, WM, Epi>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        configured = true;
    }
    uint32_t mb = (uint32_t)((m + 255) / 256), nb = (uint32_t)((n_tiles + NTB - 1) / NTB);
    gemm_mfma_big_kernel<FP8, NTB, WM, Epi><<<mb * nb, 128 * WM, smem, s>>>(aq, w_tiles, (uint32_t)m, (uint32_t)n, (uint32_t)n_tiles,
                                                                  (uint32_t)k_steps, mb, nb, e);
}

template <bool FP8, int NTB, typename Epi>
void launch_big(const uint8_t *aq, const uint8_t *w_tiles, uint64_t m, uint64_t n, uint64_t n_tiles, uint64_t k_steps,
                const Epi &e, hipStream_t s) {
    if (g_gemm_waves == 4)
        launch_big_wm<FP8, NTB, 2, Epi>(aq, w_tiles, m, n, n_tiles, k_steps, e, s);
    else if (g_gemm_waves == 16)
        launch_big_wm<FP8, NTB, 8, Epi>(aq, w_tiles, m, n, n_tiles, k_steps, e, s);
    else
        launch_big_wm<FP8, NTB, 4, Epi>(aq, w_tiles, m, n, n_tiles, k_steps, e, s);
}

}  // namespace

// How an int8 GEMM is launched.  ntb != 0: the large-tile kernel with that many column tiles per block,
// ntb == 0: the 128 x 128 kernel; splits > 1 (128 x 128 kernel only): k is divided over that many blocks
// per output tile, which leave int32 partial sums in a workspace that a second kernel adds (exactly) before
// the epilogue.  A matrix with few output tiles (a prompt of a few hundred rows against a 4096-column
// weight) occupies only a fraction of the compute units otherwise, and each of them pulls operands at a
// fixed rate.  (The same split on the large-tile kernel measured no faster.)
struct W8a8Plan {
    int ntb;
    uint32_t splits;
    uint32_t share = 1;    // large-tile kernel on 256 x 128 tiles: same-XCD blocks that share a tile, a part of k each
};

static W8a8Plan plan_w8a8(uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus, bool may_share = true) {
    const uint64_t n_tiles = n_pad / 16;
    const uint64_t fill = (uint64_t)num_cus * (g_gemm_split_fill > 0 ? g_gemm_split_fill : 2);
    const bool big_ok = !(g_gemm_small_tiles || k_pad % 128 || k_pad == 0) && n_tiles >= 14;
    if (big_ok && m >= 256) {
        if (int ntb = pick_big_ntb(m, n_tiles, num_cus)) return {ntb, 1};
        // Too few 256 x 224 tiles for the device, but 256 x 128 tiles for at least half of it (about a thousand rows
        // against a 4096- or 6144-column weight): the large-tile kernel on the narrower tile keeps its rate per compute
        // unit, where the 128 x 128 kernel with its k split and second pass ran at a third of it (1024 rows, us: q | k | v
        // 65 + 18 -> 40, o 65 + 18 -> 37)
        const uint64_t blocks8 = ((m + 255) / 256) * ((n_tiles + 7) / 8), k_steps = k_pad / 128;
        // ... and when those tiles cover a quarter to a half of it, two blocks share a tile, half of k each (one prompt
        // of 1024 tokens through 32 layers: 14.0 -> 12.4 ms; 600 / 767 rows, us incl. the row quantizer: 4096 -> 4096
        // 46 / 53 -> 41 / 41, 14336 -> 4096 105 / 133 -> 93 / 95), at least sixteen stages of k per block.  Four blocks a
        // tile measured slower than every other form (14336 -> 4096 at 257 .. 512 rows: 82 - 87 us against 55 - 78 us).
        if (g_gemm_ntb == 0 && blocks8 * 2 >= (uint64_t)num_cus)
            return {8, 1, (may_share && g_gemm_pair != 1 && blocks8 * 2 <= (uint64_t)num_cus && k_steps >= 32) ? 2u : 1u};
        if (may_share && g_gemm_ntb == 0 && g_gemm_pair != 1 && g_gemm_pair != 2) {
            if (blocks8 * 4 >= (uint64_t)num_cus && blocks8 * 2 <= (uint64_t)num_cus && k_steps >= 32) return {8, 1, 2};
        }
    }
    const uint64_t blocks = ((n_tiles + NT - 1) / NT) * ((m + BM - 1) / BM);
    if (blocks == 0 || blocks * 2 > fill) return {0, 1};
    uint64_t s = std::min<uint64_t>(std::min<uint64_t>(16, fill / blocks), (k_pad / 64) / 4);
    return {0, (uint32_t)std::max<uint64_t>(s, 1)};
}

GemmPlan gemm_plan(bool fp8, uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus) {
    GemmPlan out{0, 4, 1};
    if (fp8) {
        out.big_ntb = (g_gemm_small_tiles || k_pad == 0) ? 0 : pick_big_ntb(m, n_pad / 16, num_cus);
    } else {
        const W8a8Plan p = plan_w8a8(m, n_pad, k_pad, num_cus);
        out.big_ntb = p.ntb;
        out.splits = p.splits;
    }
    if (out.big_ntb) out.waves = g_gemm_waves == 4 ? 4 : g_gemm_waves == 16 ? 16 : 8;
    return out;
}

uint64_t gemm_w8a8_workspace_bytes(uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad, int num_cus) {
    const W8a8Plan p = plan_w8a8(m, n_pad, k_pad, num_cus);
    if (p.share > 1) return ((m + 255) / 256) * ((n_pad / 16 + 7) / 8) * p.share * (uint64_t)(256 * 128 * 4);
    return p.splits > 1 ? (uint64_t)p.splits * m * n * 4 : 0;
}

void gemm_w8a8_mfma(const int8_t *aq, const int8_t *w_tiles, uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad,
                    const EpilogueI8 &ep, int num_cus, hipStream_t s, void *workspace, uint64_t workspace_bytes,
                    const SplitKArea *sk) {
    if (m == 0 || n == 0) return;
    EpiI8 e{ep.sx, ep.sw, ep.bias, ep.residual, ep.acc_out, ep.out, ep.out_bf16};
    W8a8Plan p = plan_w8a8(m, n_pad, k_pad, num_cus);
    if (p.share > 1) {
        const uint64_t tiles = ((m + 255) / 256) * ((n_pad / 16 + 7) / 8), need = tiles * p.share * (uint64_t)(256 * 128 * 4);
        if (sk && sk->counters && tiles <= sk->n_counters && workspace && workspace_bytes >= need && g_gemm_waves != 4 && g_gemm_waves != 16) {
            e.split_partial = (int32_t *)workspace;
            e.split_counters = sk->counters;
            // (the scope knob of the split-k decode linears forces either form here as well: 2 agent scope, 3 the XCD's L2)
            e.split_local = g_skinny_ksplit == 2 ? 0 : g_skinny_ksplit == 3 ? 1 : sk->xcd_local;
            e.split_s = p.share;
            constexpr int NTB = 8;
            const size_t smem = (3 * 16 + 2 * (size_t)NTB) * 2048;
            static bool configured = false;
            if (!configured) {
                (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mfma_big_kernel<false, NTB, 4, EpiI8>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
                configured = true;
            }
            const uint32_t mb = (uint32_t)((m + 255) / 256), nb = (uint32_t)((n_pad / 16 + NTB - 1) / NTB);
            const unsigned grid = 8u * p.share * (unsigned)((tiles + 7) / 8);   // whole groups on every XCD; surplus groups return at once
            gemm_mfma_big_kernel<false, NTB, 4, EpiI8><<<grid, 512, smem, s>>>((const uint8_t *)aq, (const uint8_t *)w_tiles, (uint32_t)m,
                                                                           (uint32_t)n, (uint32_t)(n_pad / 16), (uint32_t)(k_pad / 128), mb, nb, e);
            return;
        }
        p = plan_w8a8(m, n_pad, k_pad, num_cus, false);      // no counters or no room: the plan without shared tiles
    }
    if (p.splits > 1 && (!workspace || workspace_bytes < (uint64_t)p.splits * m * n * 4))
        p.splits = 1;                                 // no room for partial sums: one block per tile
    int32_t *partial = p.splits > 1 ? (int32_t *)workspace : nullptr;
    if (p.ntb == 16) {
        launch_big<false, 16, EpiI8>((const uint8_t *)aq, (const uint8_t *)w_tiles, m, n, n_pad / 16, k_pad / 128, e, s);
    } else if (p.ntb == 8) {
        launch_big<false, 8, EpiI8>((const uint8_t *)aq, (const uint8_t *)w_tiles, m, n, n_pad / 16, k_pad / 128, e, s);
    } else if (p.ntb) {
        launch_big<false, 14, EpiI8>((const uint8_t *)aq, (const uint8_t *)w_tiles, m, n, n_pad / 16, k_pad / 128, e, s);
    } else {
        dim3 grid((unsigned)((n_pad / 16 + NT - 1) / NT), (unsigned)((m + BM - 1) / BM), p.splits);
        gemm_mfma_kernel<false, EpiI8><<<grid, 256, 0, s>>>((const uint8_t *)aq, (const uint8_t *)w_tiles, (uint32_t)m,
                                                            (uint32_t)n, (uint32_t)(n_pad / 16), (uint32_t)(k_pad / 64), e,
                                                            partial);
    }
    if (p.splits > 1) {
        const uint64_t quads = m * ((n + 3) / 4);
        const unsigned blocks = (unsigned)std::min<uint64_t>((quads + 255) / 256, (uint64_t)num_cus * 8);
        splitk_epilogue_i8_kernel<<<blocks, 256, 0, s>>>((const int32_t *)workspace, p.splits, (uint32_t)m, (uint32_t)n, e);
    }
}

// gate | up projection of a prompt pass with SwiGLU in the epilogue: w_tiles is the [k, 2 f] weight (gate columns first),
// out receives silu(gate) * up as f32 [m, f], every value what the plain GEMM followed by the SwiGLU pass computes
// (the same two dequantizations and the same product).  Large-tile kernel only, 256 x 256 block tiles whose column
// tiles are eight gate tiles and the eight up tiles of the same product columns.
bool gemm_w8a8_swiglu_applies(uint64_t m, uint64_t f, uint64_t n_pad, uint64_t k_pad) {
    // from 65 rows (fewer take the decode kernels): the 128 x 128 kernel has one or two rows of tiles for the whole device
    // there, and this launch streams the weight once whatever the row count (one prompt of 65 / 100 / 128 / 130 / 200 / 250
    // tokens through 32 layers: 4.25 / 4.54 / 4.76 / 5.50 / 6.06 / 6.36 -> 4.01 / 4.19 / 4.28 / 4.59 / 5.21 / 5.46 ms)
    return !(g_gemm_swiglu & 1) && !g_gemm_small_tiles && m >= 65 && f != 0 && f % 128 == 0 && n_pad == 2 * f && k_pad != 0 &&
           k_pad % 128 == 0;
}
namespace {
template <int NTB>
void launch_swiglu(const int8_t *aq, const int8_t *w_tiles, const EpiI8Swiglu &e, uint64_t m, uint64_t f, uint64_t k_pad, hipStream_t s) {
    const size_t smem = (3 * 16 + 2 * (size_t)NTB) * 2048;
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mfma_big_kernel<false, NTB, 4, EpiI8Swiglu>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        configured = true;
    }
    const uint32_t mb = (uint32_t)((m + 255) / 256), nb = (uint32_t)(f / (8 * NTB));      // NTB / 2 product tiles per block
    gemm_mfma_big_kernel<false, NTB, 4, EpiI8Swiglu><<<mb * nb, 512, smem, s>>>((const uint8_t *)aq, (const uint8_t *)w_tiles, (uint32_t)m,
                                                                              (uint32_t)(2 * f), (uint32_t)(2 * f / 16),
                                                                              (uint32_t)(k_pad / 128), mb, nb, e);
}
}  // namespace
void gemm_w8a8_swiglu_mfma(const int8_t *aq, const int8_t *w_tiles, const float *sx, const float *sw, uint64_t m, uint64_t f,
                           uint64_t k_pad, float *out, int num_cus, hipStream_t s) {
    if (m == 0 || f == 0) return;
    const EpiI8Swiglu e{sx, sw, out, (uint32_t)f};
    // 256 x 256 tiles (eight gate and eight up column tiles), or 256 x 128 where the wide tiles would cover at most half the
    // device (up to 256 rows at d_ffn 14336: 112 wide tiles, 224 narrow ones; one prompt of 200 tokens through 32 layers
    // 5.56 -> 5.21 ms).  With more rows three rounds of narrow tiles measured no better than two of wide ones.
    const uint64_t mb = (m + 255) / 256;
    if (g_gemm_ntb == 8 || (g_gemm_ntb == 0 && mb * (f / 128) * 2 <= (uint64_t)num_cus))
        launch_swiglu<8>(aq, w_tiles, e, m, f, k_pad, s);
    else
        launch_swiglu<16>(aq, w_tiles, e, m, f, k_pad, s);
}

// q | k | v projection of a prompt pass with RoPE, the bf16 rounding and the K / V append in the epilogue (heads of 128 dims:
// a head is the eight column tiles of one wavefront of a 256 x 256 block tile).  Taken where the plain GEMM would run on the
// large-tile kernel too.
bool gemm_w8a8_qkv_rope_applies(uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad, uint32_t heads, uint32_t kv_heads,
                                uint32_t head_dim, int num_cus) {
    if ((g_gemm_swiglu & 2) || g_gemm_small_tiles || head_dim != 128 || m < 256 || k_pad == 0 || k_pad % 128) return false;
    if (n != (uint64_t)(heads + 2 * kv_heads) * 128 || n_pad != n || (heads + 2 * kv_heads) % 2) return false;
    return pick_big_ntb(m, n_pad / 16, num_cus) != 0;
}
void gemm_w8a8_qkv_rope_mfma(const int8_t *aq, const int8_t *w_tiles, const float *sx, const float *sw, uint64_t m, uint64_t k_pad,
                             const QkvRopeTargets &t, hipStream_t s) {
    if (m == 0) return;
    const EpiI8QkvRope e{sx, sw, t.cos_sin, t.slots, t.q_out, t.k_pool, t.v_pool, t.heads, t.kv_heads, t.pool_rows};
    constexpr int NTB = 16;
    const size_t smem = (3 * 16 + 2 * (size_t)NTB) * 2048;
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_mfma_big_kernel<false, NTB, 4, EpiI8QkvRope>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        configured = true;
    }
    const uint64_t n = (uint64_t)(t.heads + 2 * t.kv_heads) * 128;
    const uint32_t mb = (uint32_t)((m + 255) / 256), nb = (uint32_t)(n / 256);
    gemm_mfma_big_kernel<false, NTB, 4, EpiI8QkvRope><<<mb * nb, 512, smem, s>>>((const uint8_t *)aq, (const uint8_t *)w_tiles,
                                                                               (uint32_t)m, (uint32_t)n, (uint32_t)(n / 16),
                                                                               (uint32_t)(k_pad / 128), mb, nb, e);
}

static void launch_e4m3(const uint8_t *aq, const uint8_t *w_tiles, const EpiF8 &e, uint64_t m, uint64_t n, uint64_t n_pad,
                        uint64_t k_pad, int num_cus, hipStream_t s);

void gemm_e4m3_mfma(const uint8_t *aq, const uint8_t *w_tiles, const float *a_scale, const float *w_scale, uint64_t m,
                    uint64_t n, uint64_t n_pad, uint64_t k_pad, void *out, int out_bf16, int num_cus, hipStream_t s) {
    if (m == 0 || n == 0) return;
    launch_e4m3(aq, w_tiles, EpiF8{a_scale, w_scale, out, out_bf16, nullptr, nullptr, nullptr}, m, n, n_pad, k_pad, num_cus, s);
}

void gemm_e4m3_rows_mfma(const uint8_t *aq, const uint8_t *w_tiles, const float *sx, const float *sw, const float *bias,
                         uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad, void *out, int out_bf16, int num_cus,
                         hipStream_t s) {
    if (m == 0 || n == 0) return;
    launch_e4m3(aq, w_tiles, EpiF8{nullptr, nullptr, out, out_bf16, sx, sw, bias}, m, n, n_pad, k_pad, num_cus, s);
}

static void launch_e4m3(const uint8_t *aq, const uint8_t *w_tiles, const EpiF8 &e, uint64_t m, uint64_t n, uint64_t n_pad,
                        uint64_t k_pad, int num_cus, hipStream_t s) {
    if (int ntb = (g_gemm_small_tiles || k_pad == 0) ? 0 : pick_big_ntb(m, n_pad / 16, num_cus)) {
        if (ntb == 16)
            launch_big<true, 16, EpiF8>(aq, w_tiles, m, n, n_pad / 16, k_pad / 128, e, s);
        else
            launch_big<true, 14, EpiF8>(aq, w_tiles, m, n, n_pad / 16, k_pad / 128, e, s);
        return;
    }
    dim3 grid((unsigned)((n_pad / 16 + NT - 1) / NT), (unsigned)((m + BM - 1) / BM));
    gemm_mfma_kernel<true, EpiF8><<<grid, 256, 0, s>>>(aq, w_tiles, (uint32_t)m, (uint32_t)n, (uint32_t)(n_pad / 16),
                                                       (uint32_t)(k_pad / 128), e, nullptr);
}

}  // namespace k
}  // namespace fa
