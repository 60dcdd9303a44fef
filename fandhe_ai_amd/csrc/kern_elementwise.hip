// Small bandwidth-bound operators around the linears: SwiGLU, residual add,
// greedy argmax, embedding gather, dtype conversion, RoPE.
#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {
using namespace fa::dev;

namespace {

// crates/tensor-core/src/scalar_op.rs:666-673 (sigmoid_stable) and :355 (Silu)
__device__ __forceinline__ float silu(float x) { return silu_f32(x); }

__global__ void silu_mul_kernel(const float *__restrict__ gate, const float *__restrict__ up,
                                float *__restrict__ out, uint64_t n) {
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) out[i] = silu(gate[i]) * up[i];
}

__global__ void add_kernel(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ out,
                           uint64_t n) {
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) out[i] = a[i] + b[i];
}

// First index of the maximum, NaN ignored, all-NaN row -> 0
// (crates/autodiff/src/generate/mod.rs:333-343, crates/backend-rocm/src/ops.rs:991-995).
__device__ __forceinline__ void argmax_take(float &mv, uint32_t &mi, float ov, uint32_t oi) {
    const bool take = oi != 0xffffffffu && (mi == 0xffffffffu || ov > mv || (ov == mv && oi < mi));
    mv = take ? ov : mv;
    mi = take ? oi : mi;
}

constexpr int kArgmaxThreads = 1024;
__global__ void __launch_bounds__(kArgmaxThreads)
    argmax_rows_kernel(const float *__restrict__ x, int32_t *__restrict__ out, uint64_t cols) {
    const float *row = x + (uint64_t)blockIdx.x * cols;
    float best = -INFINITY;
    uint32_t best_i = 0xffffffffu;      // "nothing seen yet"
    auto see = [&](float v, uint32_t i) {
        if (v == v && (best_i == 0xffffffffu || v > best)) {      // ascending i per thread: the first maximum stays
            best = v;
            best_i = i;
        }
    };
    if (cols % 4 == 0) {                                          // rows start on 16-byte boundaries
        for (uint64_t q = threadIdx.x; q < cols / 4; q += kArgmaxThreads) {
            const float4 v = *(const float4 *)(row + 4 * q);
            see(v.x, (uint32_t)(4 * q));
            see(v.y, (uint32_t)(4 * q + 1));
            see(v.z, (uint32_t)(4 * q + 2));
            see(v.w, (uint32_t)(4 * q + 3));
        }
    } else {
        for (uint64_t i = threadIdx.x; i < cols; i += kArgmaxThreads) see(row[i], (uint32_t)i);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off);
        const uint32_t oi = (uint32_t)__shfl_xor((int)best_i, off);
        argmax_take(best, best_i, ov, oi);
    }
    __shared__ float s_val[kArgmaxThreads / 64];
    __shared__ uint32_t s_idx[kArgmaxThreads / 64];
    if (threadIdx.x % 64 == 0) {
        s_val[threadIdx.x / 64] = best;
        s_idx[threadIdx.x / 64] = best_i;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kArgmaxThreads / 64; ++w) argmax_take(best, best_i, s_val[w], s_idx[w]);
        out[blockIdx.x] = best_i == 0xffffffffu ? 0 : (int32_t)best_i;
    }
}

__global__ void gather_rows_kernel(const float *__restrict__ table, uint64_t table_rows, uint64_t cols,
                                   const int32_t *__restrict__ idx, float *__restrict__ out) {
    uint64_t r = blockIdx.x;
    int32_t id = idx[r];
    bool ok = id >= 0 && (uint64_t)id < table_rows;
    const float *src = table + (uint64_t)(ok ? id : 0) * cols;
    float *dst = out + r * cols;
    for (uint64_t c = threadIdx.x; c < cols; c += blockDim.x) dst[c] = ok ? src[c] : __uint_as_float(0x7fc00000u);
}

// The same with 16-byte moves, one per thread, for rows whose length is a multiple of four: the few rows of a
// decode step spread over as many threads as they have elements / 4, so the copy is one memory round trip.
__global__ void __launch_bounds__(256)
    gather_rows_vec_kernel(const v4f *__restrict__ table, uint64_t table_rows, uint64_t vec_cols, const int32_t *__restrict__ idx,
                           v4f *__restrict__ out) {
    const uint64_t r = blockIdx.y, c = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= vec_cols) return;
    const int32_t id = idx[r];
    const bool ok = id >= 0 && (uint64_t)id < table_rows;
    const float nan = __uint_as_float(0x7fc00000u);
    out[r * vec_cols + c] = ok ? table[(uint64_t)id * vec_cols + c] : v4f{nan, nan, nan, nan};
}

__global__ void f32_to_bf16_kernel(const float *__restrict__ in, uint16_t *__restrict__ out, uint64_t n) {
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    // pairs go through the hardware converter, which the GEMM epilogues use too (an odd tail takes the integer form)
    for (; 2 * i + 1 < n; i += stride) ((uint32_t *)out)[i] = f32x2_to_bf16x2(in[2 * i], in[2 * i + 1]);
    if (n % 2 == 1 && blockIdx.x == 0 && threadIdx.x == 0) out[n - 1] = f32_to_bf16(in[n - 1]);
}
__global__ void bf16_to_f32_kernel(const uint16_t *__restrict__ in, float *__restrict__ out, uint64_t n) {
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) out[i] = bf16_to_f32(in[i]);
}
__global__ void fill_u32_kernel(uint32_t *p, uint32_t v, uint64_t n) {
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
// two normals per hash (Box-Muller): element pair (2p, 2p+1) shares one draw
__global__ void fill_normal_kernel(void *__restrict__ out, int out_bf16, uint64_t n, uint64_t seed, float mean,
                                   float std) {
    uint64_t pair = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (; pair * 2 < n; pair += stride) {
        uint64_t h = splitmix64(seed * 0xD1342543DE82EF95ull + pair);
        float u1 = ((float)(uint32_t)(h >> 40) + 1.0f) * (1.0f / 16777216.0f);     // (0, 1]
        float u2 = (float)(uint32_t)((h >> 8) & 0xffffffu) * (1.0f / 16777216.0f);  // [0, 1)
        float r = sqrtf(-2.0f * logf(u1));
        float sn, cs;
        sincosf(6.283185307179586f * u2, &sn, &cs);
        float z[2] = {mean + std * (r * cs), mean + std * (r * sn)};
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            uint64_t i = pair * 2 + e;
            if (i >= n) break;
            if (out_bf16)
                ((uint16_t *)out)[i] = f32_to_bf16(z[e]);
            else
                ((float *)out)[i] = z[e];
        }
    }
}

// Rotate-half RoPE: pair (i, i + Dh/2), angle = pos * theta^(-2i/Dh) in f64,
// cos / sin rounded to f32, four f32 products and one add / sub, no contraction.
__global__ void rope_kernel(const float *__restrict__ x, const int32_t *__restrict__ pos, float *__restrict__ out,
                            uint32_t heads, uint32_t head_dim, double theta) {
    uint32_t half = head_dim / 2;
    uint64_t r = blockIdx.x;
    double p = (double)pos[r];
    for (uint32_t i = threadIdx.x; i < half; i += blockDim.x) {
        double inv_freq = pow(theta, -2.0 * (double)i / (double)head_dim);
        double ang = p * inv_freq;
        float c = (float)cos(ang), s = (float)sin(ang);
        for (uint32_t h = 0; h < heads; ++h) {
            uint64_t base = (r * heads + h) * head_dim;
            float xi = x[base + i], xj = x[base + i + half];
            out[base + i] = __fsub_rn(__fmul_rn(xi, c), __fmul_rn(xj, s));
            out[base + i + half] = __fadd_rn(__fmul_rn(xj, c), __fmul_rn(xi, s));
        }
    }
}

inline unsigned grid_for(uint64_t n, unsigned block, unsigned cap = 65535u * 4u) {
    uint64_t g = (n + block - 1) / block;
    if (g < 1) g = 1;
    return (unsigned)(g > cap ? cap : g);
}

}  // namespace

void silu_mul_f32(const float *gate, const float *up, float *out, uint64_t n, hipStream_t s) {
    if (n == 0) return;
    silu_mul_kernel<<<grid_for(n, 256), 256, 0, s>>>(gate, up, out, n);
}
void add_f32(const float *a, const float *b, float *out, uint64_t n, hipStream_t s) {
    if (n == 0) return;
    add_kernel<<<grid_for(n, 256), 256, 0, s>>>(a, b, out, n);
}
void argmax_rows_f32(const float *x, int32_t *out, uint64_t rows, uint64_t cols, hipStream_t s) {
    if (rows == 0) return;
    argmax_rows_kernel<<<(unsigned)rows, kArgmaxThreads, 0, s>>>(x, out, cols);
}
void gather_rows_f32(const float *table, uint64_t table_rows, uint64_t cols, const int32_t *idx, float *out,
                     uint64_t rows, hipStream_t s) {
    if (rows == 0 || cols == 0) return;
    if (cols % 4 == 0 && rows <= 65535 && (uintptr_t)table % 16 == 0 && (uintptr_t)out % 16 == 0) {
        const dim3 grid((unsigned)((cols / 4 + 255) / 256), (unsigned)rows);
        gather_rows_vec_kernel<<<grid, 256, 0, s>>>((const v4f *)table, table_rows, cols / 4, idx, (v4f *)out);
        return;
    }
    gather_rows_kernel<<<(unsigned)rows, 256, 0, s>>>(table, table_rows, cols, idx, out);
}
void convert_f32_to_bf16(const float *in, uint16_t *out, uint64_t n, hipStream_t s) {
    if (n == 0) return;
    f32_to_bf16_kernel<<<grid_for(n, 256), 256, 0, s>>>(in, out, n);
}
void convert_bf16_to_f32(const uint16_t *in, float *out, uint64_t n, hipStream_t s) {
    if (n == 0) return;
    bf16_to_f32_kernel<<<grid_for(n, 256), 256, 0, s>>>(in, out, n);
}
void fill_u32(uint32_t *p, uint32_t v, uint64_t n, hipStream_t s) {
    if (n == 0) return;
    fill_u32_kernel<<<grid_for(n, 256), 256, 0, s>>>(p, v, n);
}
void fill_normal(void *out, int out_bf16, uint64_t n, uint64_t seed, float mean, float std, hipStream_t s) {
    if (n == 0) return;
    fill_normal_kernel<<<grid_for((n + 1) / 2, 256, 65535u), 256, 0, s>>>(out, out_bf16, n, seed, mean, std);
}
void rope_f32(const float *x, const int32_t *pos, float *out, uint64_t rows, uint64_t heads, uint64_t head_dim,
              double theta, hipStream_t s) {
    if (rows == 0 || heads == 0 || head_dim < 2) return;
    rope_kernel<<<(unsigned)rows, 64, 0, s>>>(x, pos, out, (uint32_t)heads, (uint32_t)head_dim, theta);
}

}  // namespace k
}  // namespace fa
