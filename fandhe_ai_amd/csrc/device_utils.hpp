// Device-side helpers shared by the gfx950 kernels (wave64 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace fa {
namespace dev {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// 16-byte load of data that this kernel reads once (weights, K / V pages).  ONCE marks the request non-temporal
// (the nt bit of global_load_dwordx4): the line is not kept in preference to others in L2, and a long read-once
// stream moves faster through the memory system (a plain read of 632 MB: 110-114 us with ordinary loads, 99-103 us
// with these; 117 MB: 20.1 against 18.5 us).  A line that is already in L2 still hits.
template <bool ONCE, typename T>
__device__ __forceinline__ T stream_load(const T *p) {
    if constexpr (ONCE)
        return __builtin_nontemporal_load(p);
    else
        return *p;
}

// round-to-nearest-even, NaN stays a quiet NaN
__device__ __forceinline__ uint16_t f32_to_bf16(float v) {
    uint32_t u = __float_as_uint(v);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
// Two roundings at once on the converter of this part (v_cvt_pk_bf16_f32): `lo` in the low half.  The same
// round-to-nearest-even, NaN quieted the same way (checked on the device against f32_to_bf16 for every upper half
// with tie / above-tie / below-tie lower halves); one instruction instead of about ten per pair.
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{lo, hi}, v2bf));
}
__device__ __forceinline__ float bf16_to_f32(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// The same reductions on the DPP data path.  A __shfl_xor compiles to ds_bpermute_b32, one LDS round trip per step
// and two per step for a double: the six steps of a wavefront reduction are a dependent chain of about a hundred
// clocks each, which is most of the running time of a kernel that handles one row per block.  Here four DPP steps
// (lane ^ 1, lane ^ 2, mirror within 8, mirror within 16: a few clocks each) leave every lane with the result of its
// row of 16 lanes, and the four rows meet through v_readlane.  Sums are therefore associated differently from
// wave_sum (pairs, quads, eights, rows, then row 0 + row 1 + row 2 + row 3); every lane gets the same value.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) { return __uint_as_float(dpp_u32<CTRL>(__float_as_uint(v))); }
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_move(uint32_t v) { return dpp_u32<CTRL>(v); }
template <int CTRL>
__device__ __forceinline__ double dpp_move(double v) {
    const uint64_t u = (uint64_t)__double_as_longlong(v);
    const uint32_t lo = dpp_u32<CTRL>((uint32_t)u), hi = dpp_u32<CTRL>((uint32_t)(u >> 32));
    return __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
}
__device__ __forceinline__ float lane_value(float v, int lane) { return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), lane)); }
__device__ __forceinline__ uint32_t lane_value(uint32_t v, int lane) { return (uint32_t)__builtin_amdgcn_readlane((int)v, lane); }
__device__ __forceinline__ double lane_value(double v, int lane) {
    const uint64_t u = (uint64_t)__double_as_longlong(v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)u, lane);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(u >> 32), lane);
    return __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;

// every lane: the sum / maximum over its row of 16 lanes
template <typename T>
__device__ __forceinline__ T row16_sum(T v) {
    v += dpp_move<kDppXor1>(v);
    v += dpp_move<kDppXor2>(v);
    v += dpp_move<kDppHalfMirror>(v);
    v += dpp_move<kDppMirror>(v);
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_move<kDppXor1>(v));
    v = fmaxf(v, dpp_move<kDppXor2>(v));
    v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_move<kDppMirror>(v));
    return v;
}
template <typename T>
__device__ __forceinline__ T wave_sum_dpp(T v) {
    v = row16_sum(v);
    return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}
__device__ __forceinline__ float wave_max_dpp(float v) {
    v = row16_max(v);
    return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}

// Block-wide reductions for blocks of NWAVES wavefronts; `smem` needs NWAVES slots.  DPP selects the wavefront
// step above (a different association of the sum).  FRESH: nobody has read `smem` since the block's last barrier,
// so the barrier that protects earlier readers is left out.
template <typename T, int NWAVES, bool DPP = false, bool FRESH = false>
__device__ __forceinline__ T block_sum(T v, T *smem) {
    v = DPP ? wave_sum_dpp(v) : wave_sum(v);
    int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (!FRESH) __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    T r = smem[0];
#pragma unroll
    for (int i = 1; i < NWAVES; ++i) r += smem[i];
    return r;
}
template <int NWAVES, bool DPP = false, bool FRESH = false>
__device__ __forceinline__ float block_max(float v, float *smem) {
    v = DPP ? wave_max_dpp(v) : wave_max(v);
    int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (!FRESH) __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float r = smem[0];
#pragma unroll
    for (int i = 1; i < NWAVES; ++i) r = fmaxf(r, smem[i]);
    return r;
}

// symmetric int8 code of x for a given scale: rne(x / scale) clamped to +-127
__device__ __forceinline__ int quant_i8(float x, float scale) {
    if (scale == 0.0f) return 0;
    float r = rintf(__fdiv_rn(x, scale));
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int)r;
}

// x * sigmoid(x) with the two-branch sigmoid of crates/tensor-core/src/scalar_op.rs:666-673 (and :355)
__device__ __forceinline__ float silu_f32(float x) {
    float s;
    if (x >= 0.0f) {
        s = __fdiv_rn(1.0f, 1.0f + expf(-x));
    } else {
        float e = expf(x);
        s = __fdiv_rn(e, 1.0f + e);
    }
    return x * s;
}

// byte offset of the 16-byte chunk `chunk` (= k / 16) of activation row r in the 16-row x 64-k tile order
// of the quantized activations
__device__ __forceinline__ uint64_t tiled_chunk_offset(uint64_t r, uint64_t chunk, uint64_t k_tiles) {
    // kt = chunk / 4, k-group g = chunk % 4
    uint64_t mt = r / 16, rr = r % 16, kt = chunk / 4, g = chunk % 4;
    return (mt * k_tiles + kt) * 1024 + (g * 16 + rr) * 16;
}

// OCP e4m3fn encode, round-to-nearest-even, saturating at +-448
__device__ __forceinline__ uint32_t f32_to_e4m3(float v) {
    uint32_t u = __float_as_uint(v);
    uint32_t sign = (u >> 24) & 0x80u;
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return 0x7fu;                    // NaN
    if (a >= 0x43e80000u) return sign | 0x7eu;            // >= 464: saturate to 448
    if (a < 0x3c800000u) {                                // < 2^-6: subnormal, spacing 2^-9
        float q = rintf(__uint_as_float(a) * 512.0f);     // 0..8 (8 carries into the first normal)
        return sign | (uint32_t)q;
    }
    // normal: keep 3 mantissa bits, RNE on the dropped 20
    uint32_t r = a + 0x7ffffu + ((a >> 20) & 1u);
    uint32_t e = (r >> 23) - 120u;                        // rebias 127 -> 7
    uint32_t m = (r >> 20) & 7u;
    return sign | (e << 3) | m;
}


// Weight bytes of the linear that runs next, pulled into the L2 of the XCD whose compute units will read them.
// The small row kernels between two linears (norm + quantizer, merge + quantizer, quantizer) are chains of
// memory round trips on 32 blocks; HBM idles for their whole duration.  Appended blocks of the same launch
// stream the first bytes of the next linear's weight tiles meanwhile.  Workgroups go to the XCDs round-robin by
// their linear id, so when the number of blocks in front of them is a multiple of eight, appended block j lands
// on the XCD of block j of the next launch and reads exactly what that block will read first; L2 keeps clean
// lines across the kernel boundary, and the linear then finds them there (a 25 MB weight read: 6.2 us cold,
// 2.6 us after such a pull, 5.0 us when the pull ran on other XCDs).  Nothing is written.
// PF: fa::k::WeightPrefetch (declared with the launchers)
template <typename PF>
__device__ __forceinline__ void prefetch_weights(const PF &pf, uint32_t j) {
    if (j >= pf.blocks) return;
    uint32_t t0, reps, step;
    uint64_t start = 0;                               // byte offset of the pull inside each tile
    if (pf.ksplit) {                                  // split-k launch: group (q / S) * 8 + xcd, member q % S
        const uint32_t S = pf.ksplit, xcd = j % 8, q = j / 8, member = q % S;
        t0 = ((q / S) * 8 + xcd) * S;
        reps = S;
        step = 1;
        start = ((uint64_t)pf.k_tiles * member / S) * 1024;
    } else {
        t0 = pf.half_tiles ? (j / pf.half_tiles) * 2 * pf.half_tiles + j % pf.half_tiles : j * pf.tile_stride;
        reps = pf.pair_step ? 2u : 1u;
        step = pf.pair_step;
    }
    const uint32_t vecs = pf.bytes / 16, nt = blockDim.x;
    v4u acc = v4u{0, 0, 0, 0};
    for (uint32_t r = 0; r < reps; ++r) {
        uint32_t tile = t0 + r * step;
        tile = tile < pf.n_tiles ? tile : pf.n_tiles - 1;
        const v4u *p = (const v4u *)(pf.w + (uint64_t)tile * pf.k_tiles * 1024 + start);
        for (uint32_t i = threadIdx.x; i < vecs; i += nt * 4) {
            v4u t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) t[u] = p[i + u * nt < vecs ? i + u * nt : i];
#pragma unroll
            for (int u = 0; u < 4; ++u) acc ^= t[u];
        }
    }
    asm volatile("" ::"v"(acc[0] ^ acc[1] ^ acc[2] ^ acc[3]));      // the loads are the point; keep them
}

}  // namespace dev
}  // namespace fa
