// Measurement aid: the rate at which the matrix cores retire one instruction kind when nothing else
// limits them (operands stay in registers, no memory traffic inside the loop).  The operand bits come
// from a caller-supplied buffer, because the sustained rate of this part depends on them: with
// all-zero operands the cores run at the published peak, with random bits the clock is held lower.
#include <type_traits>

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
    // The instructions are written out with their accumulators tied to the accumulation registers: through the
    // builtins the register allocator moved accumulators between the two register files around every instruction
    // of the 16 x 16 x 64 form, and the loop then measured those moves (half the instruction's rate).
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const v4i &x = a[i % 8], &y = b[(i * 3) % 8];
            if constexpr (KIND == 0) asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc16[i]) : "v"(x), "v"(y));
            if constexpr (KIND == 1) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+a"(acc32[i % 4]) : "v"(x), "v"(y));
            if constexpr (KIND == 2) {
                const v4i &x1 = a[(i + 1) % 8], &y1 = b[(i * 3 + 1) % 8];
                const v8i xx = v8i{x[0], x[1], x[2], x[3], x1[0], x1[1], x1[2], x1[3]};
                const v8i yy = v8i{y[0], y[1], y[2], y[3], y1[0], y1[1], y1[2], y1[3]};
                const int unit = 0x7f7f7f7f;          // block scales 2^0
                asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0]"
                             : "+a"(accf[i])
                             : "v"(xx), "v"(yy), "v"(unit));
            }
        }
    }
    // the compiler does not know that the statements above are matrix instructions: wait out the pipeline before
    // anything reads an accumulator
#pragma unroll
    for (int i = 0; i < 16; ++i) asm volatile("s_nop 15\n\ts_nop 15" : "+a"(acc16[i]), "+a"(accf[i]));
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("s_nop 15\n\ts_nop 15" : "+a"(acc32[i]));
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

// The path from L2 to a compute unit, two measurements in one kernel.  Every block streams its own share of `cold`
// (memory nobody has touched: HBM) with G 16-byte loads per thread in flight and, with every cold load, R ordinary
// loads of a small region `hot` that all blocks share and that therefore sits in every XCD's L2 after the first
// touch.  cold_vecs_per_block == 0: the hot region alone, `hot_passes` times per block (G loads in flight): what a
// compute unit can pull from L2 at the launch's number of wavefronts.  R == 0: the cold stream alone.  Otherwise:
// what L2 hits mixed R : 1 into an HBM stream cost that stream.
template <int G, int R>
__global__ void __launch_bounds__(512) l2_path_kernel(const v4u *__restrict__ cold, uint64_t cold_vecs_per_block,
                                                      const v4u *__restrict__ hot, uint32_t hot_vecs, uint32_t hot_passes,
                                                      int *sink) {
    const uint32_t tid = threadIdx.x, nt = blockDim.x;
    v4u acc = v4u{0, 0, 0, 0};
    uint32_t hpos = (tid + blockIdx.x * 64u) % hot_vecs;           // blocks start at different lines of the region
    if (cold_vecs_per_block == 0) {
        const uint32_t trips = (uint32_t)(((uint64_t)hot_vecs * hot_passes + (uint64_t)nt * G - 1) / ((uint64_t)nt * G));
        for (uint32_t t = 0; t < trips; ++t) {
            v4u h[G];
#pragma unroll
            for (int u = 0; u < G; ++u) {
                h[u] = hot[hpos];
                hpos += nt;
                hpos = hpos >= hot_vecs ? hpos - hot_vecs : hpos;
            }
#pragma unroll
            for (int u = 0; u < G; ++u) acc ^= h[u];
        }
    } else {
        const v4u *cb = cold + (uint64_t)blockIdx.x * cold_vecs_per_block;
        for (uint64_t i = tid; i < cold_vecs_per_block; i += (uint64_t)nt * G) {
            v4u c[G], h[G * (R ? R : 1)];
#pragma unroll
            for (int u = 0; u < G; ++u) {
                const uint64_t idx = i + (uint64_t)u * nt;
                c[u] = stream_load<true>(cb + (idx < cold_vecs_per_block ? idx : cold_vecs_per_block - 1));
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    h[u * R + r] = hot[hpos];
                    hpos += nt;
                    hpos = hpos >= hot_vecs ? hpos - hot_vecs : hpos;
                }
                __builtin_amdgcn_sched_barrier(0);               // keep the two kinds of loads interleaved as written
            }
#pragma unroll
            for (int u = 0; u < G; ++u) acc ^= c[u];
            if (R) {
#pragma unroll
                for (int u = 0; u < G * R; ++u) acc ^= h[u];
            }
        }
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) sink[0] = 1;   // keeps the loads alive
}

}  // namespace

int g_probe_plain_loads = 0;

bool l2_path_probe(const void *cold, uint64_t cold_bytes, const void *hot, uint32_t hot_bytes, uint32_t hot_passes, int in_flight,
                   int hot_per_cold, int blocks, int threads, int *sink, hipStream_t s) {
    const uint64_t cvb = cold_bytes / 16 / (uint64_t)blocks;
    const uint32_t hv = hot_bytes / 16;
    auto go = [&](auto g, auto r) {
        l2_path_kernel<decltype(g)::value, decltype(r)::value><<<blocks, threads, 0, s>>>((const v4u *)cold, cvb, (const v4u *)hot, hv,
                                                                                         hot_passes, sink);
    };
    using I8 = std::integral_constant<int, 8>;
    using I16 = std::integral_constant<int, 16>;
    using R0 = std::integral_constant<int, 0>;
    using R2 = std::integral_constant<int, 2>;
    if (in_flight == 8 && hot_per_cold == 0) go(I8{}, R0{});
    else if (in_flight == 16 && hot_per_cold == 0) go(I16{}, R0{});
    else if (in_flight == 8 && hot_per_cold == 2) go(I8{}, R2{});
    else if (in_flight == 16 && hot_per_cold == 2) go(I16{}, R2{});
    else return false;
    return true;
}

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
