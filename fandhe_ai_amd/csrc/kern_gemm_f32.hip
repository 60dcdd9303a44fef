// f32 GEMM / linear with the reference's summation contract: one accumulator per output, k ascending,
// one fused multiply-add per step (crates/backend-cpu/src/parity.rs:340-361), on the matrix cores.
//
// v_mfma_f32_32x32x1_2b_f32 adds exactly one product to every accumulator it touches, and it does so with
// a single rounding: a chain of these instructions over k is, bit for bit, the chain of fmaf(a, b, acc)
// the contract prescribes (checked on the device for normal data, wide exponent ranges, cancellation,
// subnormal inputs and results, overflow, infinities and NaNs).  So the order-fixed GEMM does not need the
// vector ALUs: a wavefront owns a 64 x 64 tile as two instructions per k (the 64 rows as the instruction's two
// 32-row blocks against columns 0..31 and 32..63, each column operand repeated in both halves of the
// wavefront) and needs one A value and two B values per lane per k, which LDS supplies at a tenth of its rate.
// Block = 4 wavefronts = 128 x 128 outputs; k advances in slabs of 32 that travel global -> registers -> LDS,
// the next slab's loads in flight while the current one is multiplied (two LDS buffers, one barrier per
// slab).  Edges: rows / columns past the matrix are loaded as zeros and never stored; k needs no padding,
// the last slab simply runs fewer steps, so no accumulator ever sees a product the contract does not have.
#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {

namespace {

constexpr int BM = 128, BN = 128, BK = 32;
constexpr int A_PITCH = BK + 4;          // floats per A row in LDS (80 B: 16-byte reads of 64 rows spread over the banks)
constexpr int B_PITCH = BN + 4;

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));

// VEC: k and n are multiples of 4 and all three pointers are 16-byte aligned, so a slab moves in float4.
template <bool VEC>
__global__ void __launch_bounds__(256)
    gemm_f32_mfma_kernel(const float *__restrict__ a, const float *__restrict__ b, const float *__restrict__ bias,
                         float *__restrict__ out, uint64_t m, uint64_t n, uint64_t k, int relu, uint32_t tiles_n) {
    __shared__ __attribute__((aligned(16))) float As[2][BM * A_PITCH];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * B_PITCH];
    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const uint64_t row0 = (uint64_t)(blockIdx.x / tiles_n) * BM, col0 = (uint64_t)(blockIdx.x % tiles_n) * BN;
    const int wr = (wave / 2) * 64, wc = (wave % 2) * 64;       // this wavefront's 64 x 64 tile inside the block tile

    // slab staging: A 128 rows x BK k and B BK k x 128 cols, BK / 8 float4 of each per thread
    constexpr int NLD = BK / 8, A4 = BK / 4;
    float4 ra[NLD], rb[NLD];
    auto load_slab = [&](uint64_t k0) {
#pragma unroll
        for (int t = 0; t < NLD; ++t) {
            const int e = tid + 256 * t;
            {
                const int r = e / A4, c4 = (e % A4) * 4;
                const uint64_t gr = row0 + r, gc = k0 + c4;
                float4 v = float4{0.f, 0.f, 0.f, 0.f};
                if (gr < m) {
                    const float *src = a + gr * k + gc;
                    if (VEC) {
                        if (gc < k) v = *(const float4 *)src;
                    } else {
                        if (gc + 0 < k) v.x = src[0];
                        if (gc + 1 < k) v.y = src[1];
                        if (gc + 2 < k) v.z = src[2];
                        if (gc + 3 < k) v.w = src[3];
                    }
                }
                ra[t] = v;
            }
            {
                const int r = e / 32, c4 = (e % 32) * 4;
                const uint64_t gr = k0 + r, gc = col0 + c4;
                float4 v = float4{0.f, 0.f, 0.f, 0.f};
                if (gr < k) {
                    const float *src = b + gr * n + gc;
                    if (VEC) {
                        if (gc < n) v = *(const float4 *)src;
                    } else {
                        if (gc + 0 < n) v.x = src[0];
                        if (gc + 1 < n) v.y = src[1];
                        if (gc + 2 < n) v.z = src[2];
                        if (gc + 3 < n) v.w = src[3];
                    }
                }
                rb[t] = v;
            }
        }
    };
    auto store_slab = [&](int buf) {
#pragma unroll
        for (int t = 0; t < NLD; ++t) {
            const int e = tid + 256 * t;
            *(float4 *)&As[buf][(e / A4) * A_PITCH + (e % A4) * 4] = ra[t];
            *(float4 *)&Bs[buf][(e / 32) * B_PITCH + (e % 32) * 4] = rb[t];
        }
    };

    v32f acc0, acc1;                                             // columns wc .. wc + 31 and wc + 32 .. wc + 63
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        acc0[i] = 0.0f;
        acc1[i] = 0.0f;
    }
    // operand addresses of this lane: A row wr + lane (block lane / 32 holds rows 32 (lane / 32) ..), B column lane % 32
    const int a_row = wr + lane, b_col = wc + lane % 32;

    if (k != 0) {
        load_slab(0);
        store_slab(0);
    }
    __syncthreads();
    int buf = 0;
    for (uint64_t k0 = 0; k0 < k; k0 += BK) {
        const bool more = k0 + BK < k;
        if (more) load_slab(k0 + BK);                            // in flight while this slab is multiplied
        const int steps = (k - k0) < (uint64_t)BK ? (int)(k - k0) : BK;
        const float *as = &As[buf][a_row * A_PITCH];
        const float *bs = &Bs[buf][b_col];
        if (steps == BK) {
#pragma unroll
            for (int q = 0; q < BK / 4; ++q) {
                const float4 av = *(const float4 *)(as + 4 * q);
                const float a4[4] = {av.x, av.y, av.z, av.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int kk = 4 * q + j;
                    const float b0 = bs[kk * B_PITCH], b1 = bs[kk * B_PITCH + 32];
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x1f32(a4[j], b0, acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x1f32(a4[j], b1, acc1, 0, 0, 0);
                }
            }
        } else {
            for (int kk = 0; kk < steps; ++kk) {
                const float av = as[kk], b0 = bs[kk * B_PITCH], b1 = bs[kk * B_PITCH + 32];
                acc0 = __builtin_amdgcn_mfma_f32_32x32x1f32(av, b0, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x1f32(av, b1, acc1, 0, 0, 0);
            }
        }
        if (more) store_slab(buf ^ 1);                           // the other buffer: its readers passed the last barrier
        __syncthreads();
        buf ^= 1;
    }

    // D layout: register 16 blk + 4 j + e of lane l = row 32 blk + 8 j + 4 (l / 32) + e, column l % 32
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const uint64_t gc = col0 + wc + 32 * half + lane % 32;
        if (gc >= n) continue;
        const float bv = bias ? bias[gc] : 0.0f;
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const int blk = i / 16, j = (i % 16) / 4, e = i % 4;
            const uint64_t gr = row0 + wr + 32 * blk + 8 * j + 4 * (lane / 32) + e;
            if (gr >= m) continue;
            float v = half ? acc1[i] : acc0[i];
            if (bias) v = __fadd_rn(v, bv);
            if (relu) v = (v != v) ? v : fmaxf(v, 0.0f);
            out[gr * n + gc] = v;
        }
    }
}

// Few rows: the chain of k dependent steps per output is what takes the time (a 32 x 32 instruction issues
// for 64 clocks whatever it is fed), and there are too few outputs to fill the chip with 128 x 128 tiles.
// Here a thread owns SR rows of one column: per k one coalesced B load (256 bytes per wavefront) and SR
// v_fma_f32 whose A operands are uniform over the block and come through the scalar cache.  The same chain,
// one fused multiply-add per k in ascending order, on the vector ALUs.  (A form with the next SK B values
// requested ahead in a second register set and the A rows staged in LDS measured slower, 207 against 130 us
// at 32 x 4096 x 4096, and was not kept; SK = 8 / 16 / 32: 174 / 130 / 162 us.)
constexpr int SR = 4, SK = 16;
__global__ void __launch_bounds__(256)
    gemm_f32_rows_kernel(const float *__restrict__ a, const float *__restrict__ b, const float *__restrict__ bias,
                         float *__restrict__ out, uint64_t m, uint64_t n, uint64_t k, int relu) {
    const uint64_t col = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    const uint64_t row0 = (uint64_t)blockIdx.y * SR;
    const uint64_t colc = col < n ? col : n - 1;                  // clamped loads, no store past the edge
    const float *arow[SR];
#pragma unroll
    for (int r = 0; r < SR; ++r) arow[r] = a + (row0 + r < m ? row0 + r : m - 1) * k;
    float acc[SR];
#pragma unroll
    for (int r = 0; r < SR; ++r) acc[r] = 0.0f;
    const float *bp = b + colc;
    uint64_t k0 = 0;
    for (; k0 + SK <= k; k0 += SK) {
        float bv[SK];
#pragma unroll
        for (int j = 0; j < SK; ++j) bv[j] = bp[(k0 + j) * n];
#pragma unroll
        for (int j = 0; j < SK; ++j)
#pragma unroll
            for (int r = 0; r < SR; ++r) acc[r] = __builtin_fmaf(arow[r][k0 + j], bv[j], acc[r]);
    }
    for (; k0 < k; ++k0) {
        const float bv = bp[k0 * n];
#pragma unroll
        for (int r = 0; r < SR; ++r) acc[r] = __builtin_fmaf(arow[r][k0], bv, acc[r]);
    }
    if (col >= n) return;
    const float bias_v = bias ? bias[col] : 0.0f;
#pragma unroll
    for (int r = 0; r < SR; ++r) {
        if (row0 + r >= m) continue;
        float v = acc[r];
        if (bias) v = __fadd_rn(v, bias_v);
        if (relu) v = (v != v) ? v : fmaxf(v, 0.0f);
        out[(row0 + r) * n + col] = v;
    }
}

int compute_units() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) cus = p.multiProcessorCount;
        if (cus <= 0) cus = 256;
    }
    return cus;
}

}  // namespace

int g_gemm_f32_form = 0;      // 0 by shape, 1 the few-rows kernel, 2 the matrix-core kernel

int gemm_f32_form(uint64_t m, uint64_t n, uint64_t k) {
    if (k == 0 || (m + SR - 1) / SR > 65535) return 2;
    if (g_gemm_f32_form == 1 || g_gemm_f32_form == 2) return g_gemm_f32_form;
    const uint64_t tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    // Both forms run a chain of k steps per output; what differs is the clocks a step occupies its SIMD for (two
    // 64-clock matrix instructions per 64 x 64 tile against SR vector instructions of 4 clocks per 64 x SR
    // outputs) and how many rounds the launch needs to seat its wavefronts (one per SIMD at a time).
    const uint64_t simds = 4ull * (uint64_t)compute_units();
    const uint64_t mfma_waves = tiles_m * tiles_n * 4, rows_waves = ((m + SR - 1) / SR) * ((n + 63) / 64);
    const uint64_t mfma_cost = ((mfma_waves + simds - 1) / simds) * 128, rows_cost = ((rows_waves + simds - 1) / simds) * 4 * SR;
    return rows_cost < mfma_cost ? 1 : 2;
}

void gemm_f32(const float *a, const float *b, const float *bias, float *out, uint64_t m, uint64_t n, uint64_t k,
              int relu, hipStream_t s) {
    if (m == 0 || n == 0) return;
    if (gemm_f32_form(m, n, k) == 1) {
        dim3 grid((unsigned)((n + 255) / 256), (unsigned)((m + SR - 1) / SR));
        gemm_f32_rows_kernel<<<grid, 256, 0, s>>>(a, b, bias, out, m, n, k, relu);
        return;
    }
    const uint64_t tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    const unsigned grid = (unsigned)(tiles_m * tiles_n);
    const bool vec = k % 4 == 0 && n % 4 == 0 && ((uintptr_t)a % 16 == 0) && ((uintptr_t)b % 16 == 0);
    if (vec)
        gemm_f32_mfma_kernel<true><<<grid, 256, 0, s>>>(a, b, bias, out, m, n, k, relu, (uint32_t)tiles_n);
    else
        gemm_f32_mfma_kernel<false><<<grid, 256, 0, s>>>(a, b, bias, out, m, n, k, relu, (uint32_t)tiles_n);
}

}  // namespace k
}  // namespace fa
