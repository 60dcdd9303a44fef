// Prefill-shape quantized GEMMs on the CDNA4 matrix cores:
//   int8 : v_mfma_i32_16x16x64_i8, int32 accumulators, dequant epilogue
//   e4m3 : v_mfma_scale_f32_16x16x128_f8f6f4 (unit block scales), f32 accumulators
// The weight arrives in tile order (kernels.hpp), i.e. already in the byte
// order a wavefront needs for the B operand; activations are row-major and
// are re-ordered into the same tile order on their way into LDS.  Both operand
// tiles are double-buffered in LDS; every LDS read is a conflict-free 16-byte
// read at lane * 16.
#include <type_traits>

#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {
using namespace fa::dev;

namespace {

struct EpiI8 {
    const float *sx, *sw, *bias, *residual;
    int32_t *acc_out;
    void *out;
    int out_bf16;
};
struct EpiF8 {
    const float *a_scale, *w_scale;
    void *out;
    int out_bf16;
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
                     uint32_t n_tiles, uint32_t k_tiles, Epi ep) {
    using C = Cfg<FP8>;
    constexpr int TK = C::TK, CH = C::CH, TILE = C::TILE;
    constexpr int VPL = CH / 16;                    // 16-byte vectors per lane chunk
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][MT * TILE];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[2][NT * TILE];

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int wm = wave / 2, wn = wave % 2;
    const uint32_t m0 = blockIdx.y * BM, nt0 = blockIdx.x * NT;
    const uint64_t k_bytes = (uint64_t)k_tiles * TK;

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

    if (k_tiles > 0) {
        load_stage(0);
        store_stage(0);
    }
    __syncthreads();
    for (uint32_t kt = 0; kt < k_tiles; ++kt) {
        int buf = kt & 1;
        if (kt + 1 < k_tiles) load_stage(kt + 1);
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
        if (kt + 1 < k_tiles) store_stage(buf ^ 1);   // the other buffer was last read one iteration ago
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
                if constexpr (FP8) {
                    v = __fmul_rn(acc[i][j][e], __fmul_rn(*ep.a_scale, *ep.w_scale));
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

}  // namespace

void gemm_w8a8_mfma(const int8_t *aq, const int8_t *w_tiles, uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad,
                    const EpilogueI8 &ep, hipStream_t s) {
    if (m == 0 || n == 0) return;
    EpiI8 e{ep.sx, ep.sw, ep.bias, ep.residual, ep.acc_out, ep.out, ep.out_bf16};
    dim3 grid((unsigned)((n_pad / 16 + NT - 1) / NT), (unsigned)((m + BM - 1) / BM));
    gemm_mfma_kernel<false, EpiI8><<<grid, 256, 0, s>>>((const uint8_t *)aq, (const uint8_t *)w_tiles, (uint32_t)m,
                                                        (uint32_t)n, (uint32_t)(n_pad / 16), (uint32_t)(k_pad / 64), e);
}

void gemm_e4m3_mfma(const uint8_t *aq, const uint8_t *w_tiles, const float *a_scale, const float *w_scale, uint64_t m,
                    uint64_t n, uint64_t n_pad, uint64_t k_pad, void *out, int out_bf16, hipStream_t s) {
    if (m == 0 || n == 0) return;
    EpiF8 e{a_scale, w_scale, out, out_bf16};
    dim3 grid((unsigned)((n_pad / 16 + NT - 1) / NT), (unsigned)((m + BM - 1) / BM));
    gemm_mfma_kernel<true, EpiF8><<<grid, 256, 0, s>>>(aq, w_tiles, (uint32_t)m, (uint32_t)n, (uint32_t)(n_pad / 16),
                                                       (uint32_t)(k_pad / 128), e);
}

}  // namespace k
}  // namespace fa
