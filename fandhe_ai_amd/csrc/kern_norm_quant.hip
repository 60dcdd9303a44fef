// RMSNorm (reference contract), dynamic per-token int8 quantization, their
// fusion, and per-tensor e4m3 quantization.
#include <type_traits>

#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {
using namespace fa::dev;

int g_rows_wide = 0;        // tuning: 1 keeps the 256-thread row kernels for every row count

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;

// crates/backend-cpu/src/rmsnorm.rs:203-228: f64 sum of squares through fma,
// rstd = (f32)(1 / sqrt(fma(acc, (f64)inv_n, (f64)eps))), out = (x * rstd) * w.
// The row sum is split over the block's threads; only its order differs.
__device__ __forceinline__ float row_rstd(const float *__restrict__ row, uint64_t hidden, float inv_n, float eps,
                                          double *smem) {
    double acc = 0.0;
    for (uint64_t i = threadIdx.x; i < hidden; i += kBlock) {
        double v = (double)row[i];
        acc = fma(v, v, acc);
    }
    acc = block_sum<double, kWaves>(acc, smem);
    return (float)(1.0 / sqrt(fma(acc, (double)inv_n, (double)eps)));
}

__global__ void __launch_bounds__(kBlock) rmsnorm_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                         float *__restrict__ out, uint64_t hidden, float inv_n,
                                                         float eps) {
    __shared__ double smem[kWaves];
    const float *row = x + (uint64_t)blockIdx.x * hidden;
    float *orow = out + (uint64_t)blockIdx.x * hidden;
    float rstd = row_rstd(row, hidden, inv_n, eps, smem);
    if (w) {
        for (uint64_t i = threadIdx.x; i < hidden; i += kBlock) orow[i] = __fmul_rn(__fmul_rn(row[i], rstd), w[i]);
    } else {
        for (uint64_t i = threadIdx.x; i < hidden; i += kBlock) orow[i] = __fmul_rn(row[i], rstd);
    }
}

template <bool IN_BF16>
__device__ __forceinline__ float load_in(const void *x, uint64_t i) {
    if (IN_BF16) return bf16_to_f32(((const uint16_t *)x)[i]);
    return ((const float *)x)[i];
}

// 16 consecutive elements starting at element i (a multiple of 16 of a 16-aligned row) as f32
template <bool IN_BF16>
__device__ __forceinline__ void load16(const void *x, uint64_t i, float (&v)[16]) {
    if (IN_BF16) {
        const v4u *p = (const v4u *)((const uint16_t *)x + i);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            v4u t = p[h];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[h * 8 + 2 * e] = bf16_lo(t[e]);
                v[h * 8 + 2 * e + 1] = bf16_hi(t[e]);
            }
        }
    } else {
        const v4f *p = (const v4f *)((const float *)x + i);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            v4f t = p[q];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[q * 4 + e] = t[e];
        }
    }
}

// One block per (padded) row.  Pass 1: absmax.  Pass 2: codes, 16 per thread
// step so that the tiled output is written with 16-byte stores.
template <bool IN_BF16>
__global__ void __launch_bounds__(kBlock)
    quantize_rows_kernel(const void *__restrict__ x, int8_t *__restrict__ xq_row, int8_t *__restrict__ xq_tiled,
                         float *__restrict__ sx, uint64_t m, uint64_t k, uint64_t k_pad) {
    __shared__ float smem[kWaves];
    uint64_t r = blockIdx.x;
    uint64_t k_tiles = k_pad / 64;
    if (r >= m) {                                     // padding row of the tiled layout
        if (xq_tiled)
            for (uint64_t c = threadIdx.x; c < k_pad / 16; c += kBlock)
                *(v4i *)(xq_tiled + tiled_chunk_offset(r, c, k_tiles)) = v4i{0, 0, 0, 0};
        return;
    }
    uint64_t base = r * k;
    float amax = 0.0f;
    if (k % 16 == 0) {
        // whole 16-element chunks: 16-byte loads, and the row-major codes leave in 16-byte stores
        for (uint64_t c = threadIdx.x; c < k / 16; c += kBlock) {
            float v[16];
            load16<IN_BF16>(x, base + c * 16, v);
#pragma unroll
            for (int e = 0; e < 16; ++e) amax = fmaxf(amax, fabsf(v[e]));
        }
        amax = block_max<kWaves>(amax, smem);
        const float scale = __fdiv_rn(amax, 127.0f);
        if (threadIdx.x == 0) sx[r] = scale;
        for (uint64_t c = threadIdx.x; c < k_pad / 16; c += kBlock) {
            uint32_t words[4] = {0, 0, 0, 0};
            if (c < k / 16) {
                float v[16];
                load16<IN_BF16>(x, base + c * 16, v);
#pragma unroll
                for (int e = 0; e < 16; ++e) words[e / 4] |= ((uint32_t)quant_i8(v[e], scale) & 0xffu) << (8 * (e % 4));
            }
            if (xq_tiled)
                *(v4u *)(xq_tiled + tiled_chunk_offset(r, c, k_tiles)) = v4u{words[0], words[1], words[2], words[3]};
            if (xq_row && c < k / 16) *(v4u *)(xq_row + base + c * 16) = v4u{words[0], words[1], words[2], words[3]};
        }
        return;
    }
    for (uint64_t i = threadIdx.x; i < k; i += kBlock) amax = fmaxf(amax, fabsf(load_in<IN_BF16>(x, base + i)));
    amax = block_max<kWaves>(amax, smem);
    float scale = __fdiv_rn(amax, 127.0f);
    if (threadIdx.x == 0) sx[r] = scale;
    for (uint64_t c = threadIdx.x; c < k_pad / 16; c += kBlock) {
        uint32_t words[4];
#pragma unroll
        for (int wd = 0; wd < 4; ++wd) {
            uint32_t word = 0;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                uint64_t kk = c * 16 + wd * 4 + b;
                int q = kk < k ? quant_i8(load_in<IN_BF16>(x, base + kk), scale) : 0;
                word |= ((uint32_t)q & 0xffu) << (8 * b);
            }
            words[wd] = word;
        }
        if (xq_tiled)
            *(v4u *)(xq_tiled + tiled_chunk_offset(r, c, k_tiles)) = v4u{words[0], words[1], words[2], words[3]};
        if (xq_row) {
#pragma unroll
            for (int wd = 0; wd < 4; ++wd)
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    uint64_t kk = c * 16 + wd * 4 + b;
                    if (kk < k) xq_row[base + kk] = (int8_t)((words[wd] >> (8 * b)) & 0xffu);
                }
        }
    }
}

// RMSNorm of an f32 row followed by its per-token quantization.  Thread t owns the 16-element chunks
// t, t + 256, ... of the row and keeps them in registers (NCH chunks), so the row is read once:
// f64 sum of squares -> rstd -> y = (x * rstd) * w -> absmax -> codes, written as 16-byte tile chunks.
// ROW: the codes go to a row-major [m, hidden] matrix (the operand layout of the prefill GEMMs) instead of tiles.
template <int NCH, bool ROW = false>
__global__ void __launch_bounds__(kBlock)
    rmsnorm_quantize_kernel(const float *__restrict__ x, const float *__restrict__ w, float eps, float inv_n,
                            float *__restrict__ out_f32, int8_t *__restrict__ xq_tiled, float *__restrict__ sx,
                            uint64_t m, uint64_t hidden, uint32_t row_blocks, WeightPrefetch pull) {
    __shared__ double smem_d[kWaves];
    __shared__ float smem_f[kWaves];
    if (blockIdx.x >= row_blocks) {                      // appended blocks: weights of the linear that follows
        prefetch_weights(pull, blockIdx.x - row_blocks);
        return;
    }
    const uint64_t r = blockIdx.x;
    const uint64_t k_tiles = hidden / 64, n_chunks = hidden / 16;
    if (r >= m) {
        if (!ROW)
            for (uint64_t c = threadIdx.x; c < n_chunks; c += kBlock)
                *(v4i *)(xq_tiled + tiled_chunk_offset(r, c, k_tiles)) = v4i{0, 0, 0, 0};
        return;
    }
    const float *row = x + r * hidden;
    v4f xv[NCH][4], wv[NCH][4];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        uint64_t c = threadIdx.x + (uint64_t)i * kBlock;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            xv[i][v] = c < n_chunks ? *(const v4f *)(row + c * 16 + v * 4) : v4f{0.f, 0.f, 0.f, 0.f};
            wv[i][v] = c < n_chunks ? *(const v4f *)(w + c * 16 + v * 4) : v4f{0.f, 0.f, 0.f, 0.f};
        }
    }
    double acc = 0.0;
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                double d = (double)xv[i][v][e];
                acc = fma(d, d, acc);
            }
    acc = block_sum<double, kWaves>(acc, smem_d);
    const float rstd = (float)(1.0 / sqrt(fma(acc, (double)inv_n, (double)eps)));
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float y = __fmul_rn(__fmul_rn(xv[i][v][e], rstd), wv[i][v][e]);
                xv[i][v][e] = y;
                amax = fmaxf(amax, fabsf(y));
            }
    amax = block_max<kWaves>(amax, smem_f);
    const float scale = __fdiv_rn(amax, 127.0f);
    if (threadIdx.x == 0) sx[r] = scale;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        uint64_t c = threadIdx.x + (uint64_t)i * kBlock;
        if (c >= n_chunks) continue;
        uint32_t words[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            uint32_t word = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) word |= ((uint32_t)quant_i8(xv[i][v][e], scale) & 0xffu) << (8 * e);
            words[v] = word;
            if (out_f32) *(v4f *)(out_f32 + r * hidden + c * 16 + v * 4) = xv[i][v];
        }
        int8_t *dst = ROW ? xq_tiled + r * hidden + c * 16 : xq_tiled + tiled_chunk_offset(r, c, k_tiles);
        *(v4u *)dst = v4u{words[0], words[1], words[2], words[3]};
    }
}

// The same for few rows (a decode step: 32 rows on 32 compute units), where the kernel's time is its chain of
// dependent steps and not its bytes: a block of THREADS threads per row, thread t owning the four-element groups
// t, t + THREADS, ... (VPT of them), so that at 4096 columns a thread converts, squares, scales and divides four
// elements instead of sixteen and the row's bytes are requested by sixteen wavefronts at once.  Same arithmetic
// per element; the f64 sum of squares is split over more threads (only its order differs, as above).
template <int THREADS, int VPT, bool ROW>
__global__ void __launch_bounds__(THREADS)
    rmsnorm_quantize_wide_kernel(const float *__restrict__ x, const float *__restrict__ w, float eps, float inv_n,
                                 float *__restrict__ out_f32, int8_t *__restrict__ xq, float *__restrict__ sx, uint64_t m,
                                 uint64_t hidden, uint32_t row_blocks, WeightPrefetch pull) {
    constexpr int NW = THREADS / kWave;
    __shared__ double smem_d[NW];
    __shared__ float smem_f[NW];
    if (blockIdx.x >= row_blocks) {                      // appended blocks: weights of the linear that follows
        prefetch_weights(pull, blockIdx.x - row_blocks);
        return;
    }
    const uint64_t r = blockIdx.x;
    const uint64_t k_tiles = hidden / 64, n_vec = hidden / 4;
    if (r >= m) {
        if (!ROW)
            for (uint64_t c = threadIdx.x; c < hidden / 16; c += THREADS)
                *(v4i *)(xq + tiled_chunk_offset(r, c, k_tiles)) = v4i{0, 0, 0, 0};
        return;
    }
    const float *row = x + r * hidden;
    v4f xv[VPT], wv[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const uint64_t j = threadIdx.x + (uint64_t)i * THREADS;
        xv[i] = j < n_vec ? *(const v4f *)(row + j * 4) : v4f{0.f, 0.f, 0.f, 0.f};
        wv[i] = j < n_vec ? *(const v4f *)(w + j * 4) : v4f{0.f, 0.f, 0.f, 0.f};
    }
    double acc = 0.0;
#pragma unroll
    for (int i = 0; i < VPT; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const double d = (double)xv[i][e];
            acc = fma(d, d, acc);
        }
    acc = block_sum<double, NW, true, true>(acc, smem_d);
    const float rstd = (float)(1.0 / sqrt(fma(acc, (double)inv_n, (double)eps)));
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < VPT; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float y = __fmul_rn(__fmul_rn(xv[i][e], rstd), wv[i][e]);
            xv[i][e] = y;
            amax = fmaxf(amax, fabsf(y));
        }
    amax = block_max<NW, true, true>(amax, smem_f);
    const float scale = __fdiv_rn(amax, 127.0f);
    if (threadIdx.x == 0) sx[r] = scale;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const uint64_t j = threadIdx.x + (uint64_t)i * THREADS;
        if (j >= n_vec) continue;
        uint32_t word = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) word |= ((uint32_t)quant_i8(xv[i][e], scale) & 0xffu) << (8 * e);
        if (out_f32) *(v4f *)(out_f32 + r * hidden + j * 4) = xv[i];
        int8_t *dst = ROW ? xq + r * hidden + j * 4 : xq + tiled_chunk_offset(r, j / 4, k_tiles) + (j % 4) * 4;
        *(uint32_t *)dst = word;
    }
}

// RMSNorm alone and the per-token quantizer alone in the same few-rows form (the row stays in registers, so it is
// read once).  hidden / k a multiple of 4 (rmsnorm) or of 16 with k == k_pad a multiple of 64 for tiles (quantizer).
template <int THREADS, int VPT>
__global__ void __launch_bounds__(THREADS)
    rmsnorm_wide_kernel(const float *__restrict__ x, const float *__restrict__ w, float *__restrict__ out, uint64_t hidden,
                        float inv_n, float eps) {
    constexpr int NW = THREADS / kWave;
    __shared__ double smem_d[NW];
    const uint64_t r = blockIdx.x, n_vec = hidden / 4;
    const float *row = x + r * hidden;
    v4f xv[VPT], wv[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const uint64_t j = threadIdx.x + (uint64_t)i * THREADS;
        xv[i] = j < n_vec ? *(const v4f *)(row + j * 4) : v4f{0.f, 0.f, 0.f, 0.f};
        wv[i] = (w && j < n_vec) ? *(const v4f *)(w + j * 4) : v4f{0.f, 0.f, 0.f, 0.f};
    }
    double acc = 0.0;
#pragma unroll
    for (int i = 0; i < VPT; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const double d = (double)xv[i][e];
            acc = fma(d, d, acc);
        }
    acc = block_sum<double, NW, true, true>(acc, smem_d);
    const float rstd = (float)(1.0 / sqrt(fma(acc, (double)inv_n, (double)eps)));
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const uint64_t j = threadIdx.x + (uint64_t)i * THREADS;
        if (j >= n_vec) continue;
        v4f y;
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = w ? __fmul_rn(__fmul_rn(xv[i][e], rstd), wv[i][e]) : __fmul_rn(xv[i][e], rstd);
        *(v4f *)(out + r * hidden + j * 4) = y;
    }
}

template <int THREADS, int VPT, bool IN_BF16>
__global__ void __launch_bounds__(THREADS)
    quantize_rows_wide_kernel(const void *__restrict__ x, int8_t *__restrict__ xq_row, int8_t *__restrict__ xq_tiled,
                              float *__restrict__ sx, uint64_t m, uint64_t k) {
    constexpr int NW = THREADS / kWave;
    __shared__ float smem[NW];
    const uint64_t r = blockIdx.x, k_tiles = k / 64, n_vec = k / 4;
    if (r >= m) {                                     // padding row of the tiled layout
        if (xq_tiled)
            for (uint64_t c = threadIdx.x; c < k / 16; c += THREADS)
                *(v4i *)(xq_tiled + tiled_chunk_offset(r, c, k_tiles)) = v4i{0, 0, 0, 0};
        return;
    }
    float xv[VPT][4];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const uint64_t j = threadIdx.x + (uint64_t)i * THREADS;
#pragma unroll
        for (int e = 0; e < 4; ++e) xv[i][e] = 0.0f;
        if (j < n_vec) {
            if constexpr (IN_BF16) {
                const v2u t = *(const v2u *)((const uint16_t *)x + r * k + j * 4);
                xv[i][0] = bf16_lo(t[0]);
                xv[i][1] = bf16_hi(t[0]);
                xv[i][2] = bf16_lo(t[1]);
                xv[i][3] = bf16_hi(t[1]);
            } else {
                const v4f t = *(const v4f *)((const float *)x + r * k + j * 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) xv[i][e] = t[e];
            }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) amax = fmaxf(amax, fabsf(xv[i][e]));
    }
    amax = block_max<NW, true, true>(amax, smem);
    const float scale = __fdiv_rn(amax, 127.0f);
    if (threadIdx.x == 0) sx[r] = scale;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const uint64_t j = threadIdx.x + (uint64_t)i * THREADS;
        if (j >= n_vec) continue;
        uint32_t word = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) word |= ((uint32_t)quant_i8(xv[i][e], scale) & 0xffu) << (8 * e);
        if (xq_tiled) *(uint32_t *)(xq_tiled + tiled_chunk_offset(r, j / 4, k_tiles) + (j % 4) * 4) = word;
        if (xq_row) *(uint32_t *)(xq_row + r * k + j * 4) = word;
    }
}

// SwiGLU of gu [m, 2 f] (gate columns first) followed by the per-token quantizer of the product, row-major:
// pass 1 takes the row's absmax of silu(gate) * up, pass 2 recomputes the products (the row is in L2) and
// writes their codes, so the f32 products never go to memory.  f a multiple of 16.
// ONE = true: 1024 threads and at most one 16-element chunk per thread (f <= 16384): the products stay in
// registers between the two passes, so every element is loaded and its exponential taken once.
// PROD = true: gu is the products themselves, [m, f] (the gate | up GEMM took SwiGLU into its epilogue): the same
// quantizer over values that are the same bit for bit.
template <bool ONE, bool PROD = false>
__global__ void __launch_bounds__(ONE ? 1024 : kBlock)
    swiglu_quantize_rows_kernel(const float *__restrict__ gu, int8_t *__restrict__ xq_row, float *__restrict__ sx,
                                uint64_t f, int tiled) {
    constexpr int THREADS = ONE ? 1024 : kBlock;
    __shared__ float smem[THREADS / 64];
    const uint64_t r = blockIdx.x;
    const float *gate = gu + r * (PROD ? 1 : 2) * f, *up = gate + f;
    // the product of chunk c: silu(gate) * up, or the stored product
    auto products = [&](uint64_t c, float (&p)[16]) {
        if constexpr (PROD) {
            load16<false>(gate, c * 16, p);
        } else {
            float g[16], u[16];
            load16<false>(gate, c * 16, g);
            load16<false>(up, c * 16, u);
#pragma unroll
            for (int e = 0; e < 16; ++e) p[e] = silu_f32(g[e]) * u[e];
        }
    };
    float amax = 0.0f;
    float prod[16];
    if constexpr (ONE) {
        const uint64_t c = threadIdx.x;
#pragma unroll
        for (int e = 0; e < 16; ++e) prod[e] = 0.0f;
        if (c < f / 16) {
            products(c, prod);
#pragma unroll
            for (int e = 0; e < 16; ++e) amax = fmaxf(amax, fabsf(prod[e]));
        }
    } else {
        for (uint64_t c = threadIdx.x; c < f / 16; c += THREADS) {
            float pr[16];
            products(c, pr);
#pragma unroll
            for (int e = 0; e < 16; ++e) amax = fmaxf(amax, fabsf(pr[e]));
        }
    }
    amax = block_max<THREADS / 64>(amax, smem);
    const float scale = __fdiv_rn(amax, 127.0f);
    if (threadIdx.x == 0) sx[r] = scale;
    if constexpr (ONE) {
        const uint64_t c = threadIdx.x;
        if (c < f / 16) {
            uint32_t words[4] = {0, 0, 0, 0};
#pragma unroll
            for (int e = 0; e < 16; ++e) words[e / 4] |= ((uint32_t)quant_i8(prod[e], scale) & 0xffu) << (8 * (e % 4));
            *(v4u *)(xq_row + (tiled ? tiled_chunk_offset(r, c, f / 64) : r * f + c * 16)) = v4u{words[0], words[1], words[2], words[3]};
        }
    } else {
        for (uint64_t c = threadIdx.x; c < f / 16; c += THREADS) {
            float pr[16];
            products(c, pr);
            uint32_t words[4] = {0, 0, 0, 0};
#pragma unroll
            for (int e = 0; e < 16; ++e) words[e / 4] |= ((uint32_t)quant_i8(pr[e], scale) & 0xffu) << (8 * (e % 4));
            *(v4u *)(xq_row + (tiled ? tiled_chunk_offset(r, c, f / 64) : r * f + c * 16)) = v4u{words[0], words[1], words[2], words[3]};
        }
    }
}

// Quantizer for rows whose absmax is already known as `parts` partial maxima: every block first
// reduces its row's partials (cheap, L2-resident), then quantizes a slab of 256 groups of four elements (a thread
// takes one 16-byte load of f32, or 8 bytes of bf16, and leaves four codes: with few rows the kernel's time is one
// thread's chain of loads, divisions and stores, so the elements are spread over as many threads as there are).
template <bool IN_BF16>
__global__ void __launch_bounds__(kBlock)
    quantize_from_pmax_kernel(const void *__restrict__ x, const float *__restrict__ pmax, uint32_t parts,
                              int8_t *__restrict__ xq_tiled, float *__restrict__ sx, uint64_t m, uint64_t k) {
    __shared__ float smem[kWaves];
    const uint64_t r = blockIdx.y, k_tiles = k / 64, n_vec = k / 4;
    const uint64_t j = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (r >= m) {
        if (j < n_vec) *(uint32_t *)(xq_tiled + tiled_chunk_offset(r, j / 4, k_tiles) + (j % 4) * 4) = 0u;
        return;
    }
    // the group's values are requested before the partial maxima are reduced: one memory round trip, not two
    float xv[4];
    const uint64_t jj = j < n_vec ? j : n_vec - 1;
    if constexpr (IN_BF16) {
        const v2u t = *(const v2u *)((const uint16_t *)x + r * k + jj * 4);
        xv[0] = bf16_lo(t[0]);
        xv[1] = bf16_hi(t[0]);
        xv[2] = bf16_lo(t[1]);
        xv[3] = bf16_hi(t[1]);
    } else {
        const v4f t = *(const v4f *)((const float *)x + r * k + jj * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) xv[e] = t[e];
    }
    float amax = 0.0f;
    for (uint32_t i = threadIdx.x; i < parts; i += kBlock) amax = fmaxf(amax, pmax[r * parts + i]);
    amax = block_max<kWaves, true, true>(amax, smem);
    const float scale = __fdiv_rn(amax, 127.0f);
    if (blockIdx.x == 0 && threadIdx.x == 0) sx[r] = scale;
    if (j >= n_vec) return;
    uint32_t word = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) word |= ((uint32_t)quant_i8(xv[b], scale) & 0xffu) << (8 * b);
    *(uint32_t *)(xq_tiled + tiled_chunk_offset(r, j / 4, k_tiles) + (j % 4) * 4) = word;
}

// absmax over a tensor: block maxima merged with an integer max on the bit
// pattern (valid for non-negative floats).  `absmax` must be zero on entry.
__global__ void __launch_bounds__(kBlock) absmax_kernel(const float *__restrict__ x, uint64_t n,
                                                        float *__restrict__ absmax) {
    __shared__ float smem[kWaves];
    float a = 0.0f;
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (; i < n; i += stride) a = fmaxf(a, fabsf(x[i]));
    a = block_max<kWaves>(a, smem);
    if (threadIdx.x == 0) atomicMax((unsigned int *)absmax, __float_as_uint(a));
}

__global__ void scale_from_absmax_kernel(const float *__restrict__ absmax, float divisor, float *__restrict__ scale) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *scale = __fdiv_rn(*absmax, divisor);
}

__global__ void __launch_bounds__(kBlock) quantize_e4m3_kernel(const float *__restrict__ x, uint8_t *__restrict__ q,
                                                               const float *__restrict__ scale_p, uint64_t n) {
    float scale = *scale_p;
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (; i < n; i += stride) q[i] = scale == 0.0f ? 0 : (uint8_t)f32_to_e4m3(__fdiv_rn(x[i], scale));
}

// Per-token e4m3: one block per row, scale = absmax / 448, code = e4m3(x / scale), row-major codes with the
// row padded to k_pad by zeros.
template <bool IN_BF16>
__global__ void __launch_bounds__(kBlock)
    quantize_rows_e4m3_kernel(const void *__restrict__ x, uint8_t *__restrict__ xq, float *__restrict__ sx, uint64_t k,
                              uint64_t k_pad) {
    __shared__ float smem[kWaves];
    const uint64_t r = blockIdx.x, base = r * k;
    float amax = 0.0f;
    for (uint64_t i = threadIdx.x; i < k; i += kBlock) amax = fmaxf(amax, fabsf(load_in<IN_BF16>(x, base + i)));
    amax = block_max<kWaves>(amax, smem);
    const float scale = __fdiv_rn(amax, 448.0f);
    if (threadIdx.x == 0) sx[r] = scale;
    for (uint64_t i = threadIdx.x; i < k_pad; i += kBlock)
        xq[r * k_pad + i] = (i < k && scale != 0.0f) ? (uint8_t)f32_to_e4m3(__fdiv_rn(load_in<IN_BF16>(x, base + i), scale)) : 0;
}

__global__ void zero_f32_kernel(float *p) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *p = 0.0f;
}

}  // namespace

void rmsnorm_f32(const float *x, const float *w, float *out, uint64_t rows, uint64_t hidden, float eps,
                 hipStream_t s) {
    if (rows == 0 || hidden == 0) return;
    float inv_n = 1.0f / (float)hidden;
    // few rows: the row in registers, up to 1024 threads on it (the kernel's time is its chain of round trips)
    if (g_rows_wide != 1 && rows <= 256 && hidden % 4 == 0 && hidden <= 16384) {
        if (hidden <= 1024)
            rmsnorm_wide_kernel<256, 1><<<(unsigned)rows, 256, 0, s>>>(x, w, out, hidden, inv_n, eps);
        else if (hidden <= 4096)
            rmsnorm_wide_kernel<1024, 1><<<(unsigned)rows, 1024, 0, s>>>(x, w, out, hidden, inv_n, eps);
        else if (hidden <= 8192)
            rmsnorm_wide_kernel<1024, 2><<<(unsigned)rows, 1024, 0, s>>>(x, w, out, hidden, inv_n, eps);
        else
            rmsnorm_wide_kernel<1024, 4><<<(unsigned)rows, 1024, 0, s>>>(x, w, out, hidden, inv_n, eps);
        return;
    }
    rmsnorm_kernel<<<(unsigned)rows, kBlock, 0, s>>>(x, w, out, hidden, inv_n, eps);
}

void quantize_rows_i8(const void *x, bool in_bf16, int8_t *xq_rowmajor, int8_t *xq_tiled, float *sx, uint64_t m,
                      uint64_t m_pad, uint64_t k, uint64_t k_pad, hipStream_t s) {
    uint64_t rows = xq_tiled ? m_pad : m;
    if (rows == 0 || k_pad == 0) return;
    if (g_rows_wide != 1 && rows <= 256 && k == k_pad && k % 64 == 0 && k <= 16384) {
        auto go = [&](auto threads, auto vpt) {
            constexpr int T = decltype(threads)::value, V = decltype(vpt)::value;
            if (in_bf16)
                quantize_rows_wide_kernel<T, V, true><<<(unsigned)rows, T, 0, s>>>(x, xq_rowmajor, xq_tiled, sx, m, k);
            else
                quantize_rows_wide_kernel<T, V, false><<<(unsigned)rows, T, 0, s>>>(x, xq_rowmajor, xq_tiled, sx, m, k);
        };
        if (k <= 1024)
            go(std::integral_constant<int, 256>{}, std::integral_constant<int, 1>{});
        else if (k <= 4096)
            go(std::integral_constant<int, 1024>{}, std::integral_constant<int, 1>{});
        else if (k <= 8192)
            go(std::integral_constant<int, 1024>{}, std::integral_constant<int, 2>{});
        else
            go(std::integral_constant<int, 1024>{}, std::integral_constant<int, 4>{});
        return;
    }
    if (in_bf16)
        quantize_rows_kernel<true><<<(unsigned)rows, kBlock, 0, s>>>(x, xq_rowmajor, xq_tiled, sx, m, k, k_pad);
    else
        quantize_rows_kernel<false><<<(unsigned)rows, kBlock, 0, s>>>(x, xq_rowmajor, xq_tiled, sx, m, k, k_pad);
}

namespace {
// Few rows (at most one block per compute unit): the wide form.  Returns false when the shape is not its case.
template <bool ROW>
bool launch_rmsnorm_quantize_wide(const float *x, const float *w, float eps, float inv_n, float *out_f32, int8_t *xq, float *sx,
                                  uint64_t m, uint64_t hidden, uint32_t rows, unsigned grid, const WeightPrefetch &pf,
                                  hipStream_t s) {
    if (g_rows_wide == 1 || rows > 256 || hidden > 16384 || hidden % 16 != 0) return false;
    if (hidden <= 1024)
        rmsnorm_quantize_wide_kernel<256, 1, ROW><<<grid, 256, 0, s>>>(x, w, eps, inv_n, out_f32, xq, sx, m, hidden, rows, pf);
    else if (hidden <= 4096)
        rmsnorm_quantize_wide_kernel<1024, 1, ROW><<<grid, 1024, 0, s>>>(x, w, eps, inv_n, out_f32, xq, sx, m, hidden, rows, pf);
    else if (hidden <= 8192)
        rmsnorm_quantize_wide_kernel<1024, 2, ROW><<<grid, 1024, 0, s>>>(x, w, eps, inv_n, out_f32, xq, sx, m, hidden, rows, pf);
    else
        rmsnorm_quantize_wide_kernel<1024, 4, ROW><<<grid, 1024, 0, s>>>(x, w, eps, inv_n, out_f32, xq, sx, m, hidden, rows, pf);
    return true;
}
}  // namespace

void rmsnorm_quantize_i8(const float *x, const float *w, float eps, float *out_f32, int8_t *xq_tiled, float *sx,
                         uint64_t m, uint64_t m_pad, uint64_t hidden, hipStream_t s, const WeightPrefetch &pull) {
    if (m_pad == 0 || hidden == 0) return;
    float inv_n = 1.0f / (float)hidden;
    uint64_t per_thread = (hidden / 16 + kBlock - 1) / kBlock;       // 16-element chunks per thread
    const uint32_t rows = (uint32_t)m_pad;
    // the appended blocks only meet the next launch's blocks on their XCD when a multiple of eight blocks precedes them
    const WeightPrefetch pf = (pull.w && rows % 8 == 0) ? pull : WeightPrefetch{};
    unsigned grid = rows + pf.blocks;
    if (launch_rmsnorm_quantize_wide<false>(x, w, eps, inv_n, out_f32, xq_tiled, sx, m, hidden, rows, grid, pf, s)) return;
    if (per_thread <= 1)
        rmsnorm_quantize_kernel<1><<<grid, kBlock, 0, s>>>(x, w, eps, inv_n, out_f32, xq_tiled, sx, m, hidden, rows, pf);
    else if (per_thread <= 2)
        rmsnorm_quantize_kernel<2><<<grid, kBlock, 0, s>>>(x, w, eps, inv_n, out_f32, xq_tiled, sx, m, hidden, rows, pf);
    else
        rmsnorm_quantize_kernel<4><<<grid, kBlock, 0, s>>>(x, w, eps, inv_n, out_f32, xq_tiled, sx, m, hidden, rows, pf);
}

void rmsnorm_quantize_rows_i8(const float *x, const float *w, float eps, int8_t *xq_rowmajor, float *sx, uint64_t m,
                              uint64_t hidden, hipStream_t s) {
    if (m == 0 || hidden == 0) return;
    float inv_n = 1.0f / (float)hidden;
    uint64_t per_thread = (hidden / 16 + kBlock - 1) / kBlock;
    unsigned grid = (unsigned)m;
    if (launch_rmsnorm_quantize_wide<true>(x, w, eps, inv_n, nullptr, xq_rowmajor, sx, m, hidden, grid, grid, WeightPrefetch{}, s)) return;
    if (per_thread <= 1)
        rmsnorm_quantize_kernel<1, true><<<grid, kBlock, 0, s>>>(x, w, eps, inv_n, nullptr, xq_rowmajor, sx, m, hidden, grid, WeightPrefetch{});
    else if (per_thread <= 2)
        rmsnorm_quantize_kernel<2, true><<<grid, kBlock, 0, s>>>(x, w, eps, inv_n, nullptr, xq_rowmajor, sx, m, hidden, grid, WeightPrefetch{});
    else
        rmsnorm_quantize_kernel<4, true><<<grid, kBlock, 0, s>>>(x, w, eps, inv_n, nullptr, xq_rowmajor, sx, m, hidden, grid, WeightPrefetch{});
}

void swiglu_quantize_rows_i8(const float *gu, int8_t *xq, float *sx, uint64_t m, uint64_t f, hipStream_t s, bool tiled,
                             bool products) {
    if (m == 0 || f == 0) return;
    if (products) {
        if (f <= 16384)
            swiglu_quantize_rows_kernel<true, true><<<(unsigned)m, 1024, 0, s>>>(gu, xq, sx, f, tiled ? 1 : 0);
        else
            swiglu_quantize_rows_kernel<false, true><<<(unsigned)m, kBlock, 0, s>>>(gu, xq, sx, f, tiled ? 1 : 0);
        return;
    }
    if (f <= 16384)
        swiglu_quantize_rows_kernel<true><<<(unsigned)m, 1024, 0, s>>>(gu, xq, sx, f, tiled ? 1 : 0);
    else
        swiglu_quantize_rows_kernel<false><<<(unsigned)m, kBlock, 0, s>>>(gu, xq, sx, f, tiled ? 1 : 0);
}

void quantize_rows_from_pmax(const void *x, bool in_bf16, const float *pmax, uint32_t parts, int8_t *xq_tiled,
                             float *sx, uint64_t m, uint64_t m_pad, uint64_t k, hipStream_t s) {
    if (m_pad == 0 || k == 0) return;
    dim3 grid((unsigned)((k / 4 + kBlock - 1) / kBlock), (unsigned)m_pad);
    if (in_bf16)
        quantize_from_pmax_kernel<true><<<grid, kBlock, 0, s>>>(x, pmax, parts, xq_tiled, sx, m, k);
    else
        quantize_from_pmax_kernel<false><<<grid, kBlock, 0, s>>>(x, pmax, parts, xq_tiled, sx, m, k);
}

void quantize_rows_e4m3(const void *x, bool in_bf16, uint8_t *xq_rowmajor, float *sx, uint64_t m, uint64_t k,
                        uint64_t k_pad, hipStream_t s) {
    if (m == 0 || k_pad == 0) return;
    if (in_bf16)
        quantize_rows_e4m3_kernel<true><<<(unsigned)m, kBlock, 0, s>>>(x, xq_rowmajor, sx, k, k_pad);
    else
        quantize_rows_e4m3_kernel<false><<<(unsigned)m, kBlock, 0, s>>>(x, xq_rowmajor, sx, k, k_pad);
}

void tensor_absmax_f32(const float *x, uint64_t n, float *absmax, hipStream_t s) {
    zero_f32_kernel<<<1, 64, 0, s>>>(absmax);
    if (n == 0) return;
    uint64_t g = (n + kBlock - 1) / kBlock;
    if (g > 2048) g = 2048;
    absmax_kernel<<<(unsigned)g, kBlock, 0, s>>>(x, n, absmax);
}

void scale_from_absmax(const float *absmax, float divisor, float *scale, hipStream_t s) {
    scale_from_absmax_kernel<<<1, 64, 0, s>>>(absmax, divisor, scale);
}

void quantize_tensor_e4m3(const float *x, uint8_t *q, float *scale, float *absmax_scratch, uint64_t n,
                          hipStream_t s) {
    tensor_absmax_f32(x, n, absmax_scratch, s);
    scale_from_absmax(absmax_scratch, 448.0f, scale, s);
    if (n == 0) return;
    uint64_t g = (n + kBlock - 1) / kBlock;
    if (g > 4096) g = 4096;
    quantize_e4m3_kernel<<<(unsigned)g, kBlock, 0, s>>>(x, q, scale, n);
}

}  // namespace k
}  // namespace fa
