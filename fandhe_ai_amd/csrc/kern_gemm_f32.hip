// f32 GEMM / linear with the reference's summation contract: one accumulator
// per output, k ascending, fused multiply-add
// (crates/backend-cpu/src/parity.rs:340-361).  LDS-tiled SIMT kernel; this is
// the compatibility path of linear_forward_device, not a matrix-core kernel,
// because the contract fixes the order of the f32 additions.
#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {

namespace {

constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;

__global__ void __launch_bounds__(256)
    gemm_f32_kernel(const float *__restrict__ a, const float *__restrict__ b, const float *__restrict__ bias,
                    float *__restrict__ out, uint64_t m, uint64_t n, uint64_t k, int relu) {
    __shared__ float As[BK][BM + 4];
    __shared__ float Bs[BK][BN + 4];
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const uint64_t row0 = (uint64_t)blockIdx.y * BM, col0 = (uint64_t)blockIdx.x * BN;
    float acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = 0.0f;

    for (uint64_t k0 = 0; k0 < k; k0 += BK) {
        // A tile: BM x BK, 1024 elements, 4 per thread
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int e = threadIdx.x + t * 256;
            int r = e / BK, c = e % BK;
            uint64_t gr = row0 + r, gc = k0 + c;
            As[c][r] = (gr < m && gc < k) ? a[gr * k + gc] : 0.0f;
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int e = threadIdx.x + t * 256;
            int r = e / BN, c = e % BN;
            uint64_t gr = k0 + r, gc = col0 + c;
            Bs[r][c] = (gr < k && gc < n) ? b[gr * n + gc] : 0.0f;
        }
        __syncthreads();
        // k beyond the matrix contributes fma(0, 0, acc) == acc, which keeps the order intact
        int kmax = (k - k0) < (uint64_t)BK ? (int)(k - k0) : BK;
        for (int kk = 0; kk < kmax; ++kk) {
            float av[TM], bv[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) av[i] = As[kk][ty * TM + i];
#pragma unroll
            for (int j = 0; j < TN; ++j) bv[j] = Bs[kk][tx * TN + j];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        uint64_t gr = row0 + ty * TM + i;
        if (gr >= m) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            uint64_t gc = col0 + tx * TN + j;
            if (gc >= n) continue;
            float v = acc[i][j];
            if (bias) v = __fadd_rn(v, bias[gc]);
            if (relu) v = (v != v) ? v : fmaxf(v, 0.0f);
            out[gr * n + gc] = v;
        }
    }
}

}  // namespace

void gemm_f32(const float *a, const float *b, const float *bias, float *out, uint64_t m, uint64_t n, uint64_t k,
              int relu, hipStream_t s) {
    if (m == 0 || n == 0) return;
    dim3 grid((unsigned)((n + BN - 1) / BN), (unsigned)((m + BM - 1) / BM));
    gemm_f32_kernel<<<grid, 256, 0, s>>>(a, b, bias, out, m, n, k, relu);
}

}  // namespace k
}  // namespace fa
