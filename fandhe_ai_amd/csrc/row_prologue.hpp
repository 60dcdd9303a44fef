// Row work of a decode step done inside the linear that consumes it, for batches of at most four rows.
// With one to four rows every kernel of a layer is a few microseconds of launch and round-trip latency, and the
// norm + quantizer, or the quantizer, in front of a linear is a kernel of its own that streams nothing.  Here every
// block of the linear redoes that row work for itself (4096 elements per row: eight per thread) behind its first
// weight loads, which are already in flight, and keeps the codes in LDS, where the matrix instruction's activation
// operand is read from.  The arithmetic, including the association of the f64 sum of squares, is that of the
// stand-alone kernels (kern_norm_quant.hip: rmsnorm_quantize_wide_kernel<1024, 1>, quantize_from_pmax_kernel), so a
// sequence decodes to the same bits alone and in a batch of 32.
#pragma once

#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace dev {

constexpr int kPrologueThreads = 512;     // the linears launch eight wavefronts per block
constexpr int kPrologueMaxRows = 4;

using fa::k::RowPrologue;     // declared with the launchers (kernels.hpp)

// RMSNorm + per-token quantizer of rows 0 .. m - 1 (m <= 4, 1024 < k <= 4096, k a multiple of 64) by a block of 512
// threads.  Thread t stands for threads t and t + 512 of the 1024-thread stand-alone kernel: it owns the
// four-element groups t and t + 512, reduces each inside its own "virtual" wavefront (t / 64 and 8 + t / 64) with the
// same DPP steps, and the sixteen wavefront sums are added in index order, exactly as block_sum does there.
// codes: LDS, row-major [m][k]; sx: LDS [m]; smem_d / smem_f: 16 slots each.  Ends with a barrier.
// The rows and the norm weights as the thread's registers.  Issued before the block's first weight loads: loads return
// in the order they were issued, so the row work can start while the weight tiles are still on their way (asked for
// after them, it would wait for all of them first).
struct NormRows {
    v4f xv[kPrologueMaxRows][2], wv[2];
};
__device__ __forceinline__ void prologue_norm_load(const RowPrologue &p, uint32_t m, uint32_t k, NormRows &t) {
    const uint32_t tid = threadIdx.x, n_vec = k / 4;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const uint32_t j = tid + h * kPrologueThreads;
        t.wv[h] = j < n_vec ? *(const v4f *)(p.norm_w + j * 4) : v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < kPrologueMaxRows; ++r)
            t.xv[r][h] = ((uint32_t)r < m && j < n_vec) ? *(const v4f *)(p.x + (uint64_t)r * k + j * 4) : v4f{0.f, 0.f, 0.f, 0.f};
    }
}
__device__ __forceinline__ void prologue_rmsnorm_quantize(const RowPrologue &p, NormRows &t, uint32_t m, uint32_t k, int8_t *codes,
                                                          float *sx, double *smem_d, float *smem_f) {
    const uint32_t tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave, n_vec = k / 4;
    v4f (&xv)[kPrologueMaxRows][2] = t.xv;
    v4f (&wv)[2] = t.wv;
#pragma unroll
    for (int r = 0; r < kPrologueMaxRows; ++r) {
        if ((uint32_t)r >= m) break;                    // uniform
        double part[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            double acc = 0.0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const double d = (double)xv[r][h][e];
                acc = fma(d, d, acc);
            }
            part[h] = wave_sum_dpp(acc);
        }
        if (lane == 0) {
            smem_d[wave] = part[0];
            smem_d[8 + wave] = part[1];
        }
        __syncthreads();
        double total = smem_d[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) total += smem_d[i];
        const float rstd = (float)(1.0 / sqrt(fma(total, (double)p.inv_n, (double)p.eps)));
        float am[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float amax = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float y = __fmul_rn(__fmul_rn(xv[r][h][e], rstd), wv[h][e]);
                xv[r][h][e] = y;
                amax = fmaxf(amax, fabsf(y));
            }
            am[h] = wave_max_dpp(amax);
        }
        if (lane == 0) {
            smem_f[wave] = am[0];
            smem_f[8 + wave] = am[1];
        }
        __syncthreads();                                // also: everybody has read smem_d before the next row writes it
        float amax = smem_f[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) amax = fmaxf(amax, smem_f[i]);
        const float scale = __fdiv_rn(amax, 127.0f);
        if (tid == 0) sx[r] = scale;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t j = tid + h * kPrologueThreads;
            if (j >= n_vec) continue;
            uint32_t word = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) word |= ((uint32_t)quant_i8(xv[r][h][e], scale) & 0xffu) << (8 * e);
            *(uint32_t *)(codes + (uint64_t)r * k + j * 4) = word;
        }
        __syncthreads();                                // smem_f free again; codes of the row visible
    }
}

// Per-token quantizer of rows whose absolute maximum is known as `parts` partial maxima (quantize_from_pmax_kernel):
// at most two rows of at most 16384 elements (eight four-element groups per thread and row), any k that is a multiple
// of 64, at most 1024 partial maxima per row.  The maximum is exact in any order.  Loads first, as above.
constexpr int kPmaxRows = 2, kPmaxVecs = 8;
struct PmaxRows {
    v4f xv[kPmaxRows][kPmaxVecs];
    float pm[kPmaxRows][2];
};
__device__ __forceinline__ void prologue_pmax_load(const RowPrologue &p, uint32_t m, uint32_t k, PmaxRows &t) {
    const uint32_t tid = threadIdx.x, n_vec = k / 4;
#pragma unroll
    for (int r = 0; r < kPmaxRows; ++r) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const uint32_t i = tid + u * kPrologueThreads;
            t.pm[r][u] = ((uint32_t)r < m && i < p.parts) ? p.pmax[(uint64_t)r * p.parts + i] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < kPmaxVecs; ++u) {
            const uint32_t j = tid + u * kPrologueThreads;
            t.xv[r][u] = ((uint32_t)r < m && j < n_vec) ? *(const v4f *)(p.x + (uint64_t)r * k + j * 4) : v4f{0.f, 0.f, 0.f, 0.f};
        }
    }
}
__device__ __forceinline__ void prologue_quantize_from_pmax(const RowPrologue &p, PmaxRows &t, uint32_t m, uint32_t k, int8_t *codes,
                                                            float *sx, float *smem_f) {
    const uint32_t tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave, n_vec = k / 4;
#pragma unroll
    for (int r = 0; r < kPmaxRows; ++r) {
        if ((uint32_t)r >= m) break;                    // uniform
        float amax = wave_max_dpp(fmaxf(t.pm[r][0], t.pm[r][1]));
        if (lane == 0) smem_f[wave] = amax;
        __syncthreads();
        amax = smem_f[0];
#pragma unroll
        for (int i = 1; i < kPrologueThreads / kWave; ++i) amax = fmaxf(amax, smem_f[i]);
        const float scale = __fdiv_rn(amax, 127.0f);
        if (tid == 0) sx[r] = scale;
#pragma unroll
        for (int u = 0; u < kPmaxVecs; ++u) {
            const uint32_t j = tid + u * kPrologueThreads;
            if (j >= n_vec) continue;
            uint32_t word = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) word |= ((uint32_t)quant_i8(t.xv[r][u][e], scale) & 0xffu) << (8 * e);
            *(uint32_t *)(codes + (uint64_t)r * k + j * 4) = word;
        }
        __syncthreads();
    }
}

// The launch leaves what the stand-alone kernel would have left in memory (activation tiles with rows m .. 15 zero, and
// the scales), so the stage can still be read back: every block writes a share of the 16-byte pieces (all blocks hold
// the same codes).  k a multiple of 64; codes / sx as the prologues left them.
__device__ __forceinline__ void prologue_publish(const RowPrologue &p, uint32_t m, uint32_t k, const int8_t *codes, const float *sx) {
    if (!p.xq_tiled_out) return;
    const uint32_t k_tiles = k / 64, pieces = 16 * (k / 16);
    for (uint32_t c = blockIdx.x * kPrologueThreads + threadIdx.x; c < pieces; c += gridDim.x * kPrologueThreads) {
        const uint32_t r = c / (k / 16), chunk = c % (k / 16);
        v4u v = v4u{0, 0, 0, 0};
        if (r < m) v = *(const v4u *)(codes + (uint64_t)r * k + chunk * 16);
        *(v4u *)(p.xq_tiled_out + tiled_chunk_offset(r, chunk, k_tiles)) = v;
    }
    if (blockIdx.x == 0 && threadIdx.x < m && p.sx_out) p.sx_out[threadIdx.x] = sx[threadIdx.x];
}

}  // namespace dev
}  // namespace fa
