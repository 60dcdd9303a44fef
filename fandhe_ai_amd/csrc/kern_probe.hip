// Measurement aid: the rate at which the matrix cores retire one instruction kind when nothing else
// limits them (operands stay in registers, no memory traffic inside the loop).  The operand bits come
// from a caller-supplied buffer, because the sustained rate of this part depends on them: with
// all-zero operands the cores run at the published peak, with random bits the clock is held lower.
#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {
using namespace fa::dev;

namespace {

// KIND 0: v_mfma_i32_16x16x64_i8, 1: v_mfma_i32_32x32x32_i8, 2: v_mfma_scale_f32_16x16x128_f8f6f4
template <int KIND>
__global__ void __launch_bounds__(256) matrix_rate_kernel(const v4i *__restrict__ src, uint32_t iters, int *sink) {
    // eight operand pairs per lane, taken round robin so that consecutive instructions see different bits
    v4i a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = src[(i * 256 + threadIdx.x) % 4096];
        b[i] = src[((i + 8) * 256 + threadIdx.x) % 4096];
    }
    v4i acc16[16];
    v16i acc32[4];
    v4f accf[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        acc16[i] = v4i{0, 0, 0, 0};
        accf[i] = v4f{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc32[i][e] = 0;
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const v4i &x = a[i % 8], &y = b[(i * 3) % 8];
            if constexpr (KIND == 0) acc16[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x, y, acc16[i], 0, 0, 0);
            if constexpr (KIND == 1) acc32[i % 4] = __builtin_amdgcn_mfma_i32_32x32x32_i8(x, y, acc32[i % 4], 0, 0, 0);
            if constexpr (KIND == 2) {
                const v4i &x1 = a[(i + 1) % 8], &y1 = b[(i * 3 + 1) % 8];
                accf[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    v8i{x[0], x[1], x[2], x[3], x1[0], x1[1], x1[2], x1[3]},
                    v8i{y[0], y[1], y[2], y[3], y1[0], y1[1], y1[2], y1[3]}, accf[i], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
            }
        }
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc16[i][0] + (int)accf[i][0];
#pragma unroll
    for (int i = 0; i < 4; ++i) s += acc32[i][0];
    if (s == 0x12345678) sink[0] = s;                 // keeps the loop alive; practically never taken
}

// Streaming read: every block reads its own contiguous share of [src, src + bytes) with 16-byte loads, eight per
// thread in flight.  What a memory-bound kernel of this size can reach on this part at best (launch ramp and
// tail included): the yardstick for the decode-shape linears and the decode attention.  ONCE: the non-temporal
// loads those kernels use for weights and K / V pages; ordinary loads for comparison.
template <bool ONCE>
__global__ void __launch_bounds__(512) stream_read_kernel(const v4u *__restrict__ src, uint64_t vecs_per_block, int *sink) {
    constexpr int U = 8;
    const v4u *base = src + (uint64_t)blockIdx.x * vecs_per_block;
    v4u acc = v4u{0, 0, 0, 0};
    for (uint64_t i = threadIdx.x; i < vecs_per_block; i += (uint64_t)blockDim.x * U) {
        v4u t[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t idx = i + (uint64_t)u * blockDim.x;
            t[u] = stream_load<ONCE>(base + (idx < vecs_per_block ? idx : vecs_per_block - 1));
        }
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= t[u];
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) sink[0] = 1;   // keeps the loads alive
}

}  // namespace

int g_probe_plain_loads = 0;

void stream_read_probe(const void *src, uint64_t bytes, int blocks, int threads, int *sink, hipStream_t s) {
    const uint64_t vecs = bytes / 16 / (uint64_t)blocks;
    if (vecs == 0) return;
    if (g_probe_plain_loads)
        stream_read_kernel<false><<<blocks, threads, 0, s>>>((const v4u *)src, vecs, sink);
    else
        stream_read_kernel<true><<<blocks, threads, 0, s>>>((const v4u *)src, vecs, sink);
}

double matrix_rate_probe(int kind, const void *operands, uint32_t iters, int num_cus, int *sink, hipStream_t s) {
    const int blocks = 2 * num_cus;                   // two wavefronts per SIMD
    const double per_instr[3] = {16.0 * 16 * 64 * 2, 32.0 * 32 * 32 * 2, 16.0 * 16 * 128 * 2};
    if (kind == 0) matrix_rate_kernel<0><<<blocks, 256, 0, s>>>((const v4i *)operands, iters, sink);
    else if (kind == 1) matrix_rate_kernel<1><<<blocks, 256, 0, s>>>((const v4i *)operands, iters, sink);
    else matrix_rate_kernel<2><<<blocks, 256, 0, s>>>((const v4i *)operands, iters, sink);
    return (double)blocks * 4 * iters * 16 * per_instr[kind];
}

}  // namespace k
}  // namespace fa
