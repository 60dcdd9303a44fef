// Glue kernels of the decode step: per-step position / slot bookkeeping,
// RoPE + bf16 rounding + KV append fused after the qkv projection, and SwiGLU
// fused with the per-token quantizer of the down projection.
#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {
using namespace fa::dev;

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;

__global__ void __launch_bounds__(64)
    decode_prepare_kernel(const uint32_t *__restrict__ tables, uint32_t *__restrict__ seq_lens,
                          int32_t *__restrict__ pos, uint32_t *__restrict__ slots, float *__restrict__ cos_sin,
                          uint32_t block_size, uint32_t max_blocks_per_seq, uint32_t num_blocks, uint32_t head_dim,
                          double theta) {
    const uint32_t b = blockIdx.x;
    const uint32_t p = seq_lens[b];                 // position of the token being decoded
    const uint32_t half = head_dim / 2;
    for (uint32_t i = threadIdx.x; i < half; i += 64) {
        double inv_freq = pow(theta, -2.0 * (double)i / (double)head_dim);
        double ang = (double)p * inv_freq;
        cos_sin[(uint64_t)b * head_dim + i] = (float)cos(ang);
        cos_sin[(uint64_t)b * head_dim + half + i] = (float)sin(ang);
    }
    __syncthreads();                                // every lane has read seq_lens[b] before it changes
    if (threadIdx.x == 0) {
        uint32_t slot = 0xffffffffu;
        uint32_t blk_idx = p / block_size;
        if (blk_idx < max_blocks_per_seq) {
            uint32_t id = tables[(uint64_t)b * max_blocks_per_seq + blk_idx];
            if (id < num_blocks) slot = id * block_size + p % block_size;
        }
        pos[b] = (int32_t)p;
        slots[b] = slot;
        seq_lens[b] = p + 1;
    }
}

// grid: batch; block: 256.  qkv row = [q heads | k heads | v heads].
__global__ void __launch_bounds__(kBlock)
    qkv_rope_append_kernel(const float *__restrict__ qkv, const float *__restrict__ cos_sin,
                           const uint32_t *__restrict__ slots, uint16_t *__restrict__ q_out,
                           uint16_t *__restrict__ k_pool, uint16_t *__restrict__ v_pool, uint32_t heads,
                           uint32_t kv_heads, uint32_t head_dim, uint64_t pool_rows) {
    const uint32_t b = blockIdx.x;
    const uint32_t half = head_dim / 2;
    const uint32_t eq = heads * head_dim, ekv = kv_heads * head_dim;
    const float *row = qkv + (uint64_t)b * (eq + 2 * ekv);
    const float *cs = cos_sin + (uint64_t)b * head_dim;
    const uint64_t slot = slots[b];
    const bool ok = slot < pool_rows;
    // rotated pairs of q and k: one thread per (head, i)
    const uint32_t pairs = (heads + kv_heads) * half;
    for (uint32_t t = threadIdx.x; t < pairs; t += kBlock) {
        uint32_t h = t / half, i = t % half;
        const float *x = row + (uint64_t)h * head_dim;         // k heads follow q heads contiguously
        float c = cs[i], s = cs[half + i];
        float xi = x[i], xj = x[i + half];
        float oi = __fsub_rn(__fmul_rn(xi, c), __fmul_rn(xj, s));
        float oj = __fadd_rn(__fmul_rn(xj, c), __fmul_rn(xi, s));
        if (h < heads) {
            uint16_t *dst = q_out + (uint64_t)b * eq + (uint64_t)h * head_dim;
            dst[i] = f32_to_bf16(oi);
            dst[i + half] = f32_to_bf16(oj);
        } else if (ok) {
            uint16_t *dst = k_pool + slot * ekv + (uint64_t)(h - heads) * head_dim;
            dst[i] = f32_to_bf16(oi);
            dst[i + half] = f32_to_bf16(oj);
        }
    }
    if (ok) {
        const float *v = row + eq + ekv;
        uint16_t *dst = v_pool + slot * ekv;
        for (uint32_t t = threadIdx.x; t < ekv; t += kBlock) dst[t] = f32_to_bf16(v[t]);
    }
}

// crates/tensor-core/src/scalar_op.rs:666-673 / :355
__device__ __forceinline__ float silu(float x) {
    float s;
    if (x >= 0.0f) {
        s = __fdiv_rn(1.0f, 1.0f + expf(-x));
    } else {
        float e = expf(x);
        s = __fdiv_rn(e, 1.0f + e);
    }
    return x * s;
}

__device__ __forceinline__ uint64_t tiled_chunk_offset(uint64_t r, uint64_t chunk, uint64_t k_tiles) {
    uint64_t mt = r / 16, rr = r % 16, kt = chunk / 4, g = chunk % 4;
    return (mt * k_tiles + kt) * 1024 + (g * 16 + rr) * 16;
}

__global__ void __launch_bounds__(kBlock)
    swiglu_quantize_kernel(const float *__restrict__ gu, int8_t *__restrict__ xq_tiled, float *__restrict__ sx,
                           uint64_t m, uint64_t f) {
    __shared__ float smem[kWaves];
    const uint64_t r = blockIdx.x, k_tiles = f / 64;
    if (r >= m) {
        for (uint64_t c = threadIdx.x; c < f / 16; c += kBlock)
            *(v4i *)(xq_tiled + tiled_chunk_offset(r, c, k_tiles)) = v4i{0, 0, 0, 0};
        return;
    }
    const float *gate = gu + r * 2 * f, *up = gate + f;
    float amax = 0.0f;
    for (uint64_t i = threadIdx.x; i < f; i += kBlock) amax = fmaxf(amax, fabsf(silu(gate[i]) * up[i]));
    amax = block_max<kWaves>(amax, smem);
    float scale = __fdiv_rn(amax, 127.0f);
    if (threadIdx.x == 0) sx[r] = scale;
    for (uint64_t c = threadIdx.x; c < f / 16; c += kBlock) {
        uint32_t words[4];
#pragma unroll
        for (int wd = 0; wd < 4; ++wd) {
            uint32_t word = 0;
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) {
                uint64_t kk = c * 16 + wd * 4 + bb;
                float y = silu(gate[kk]) * up[kk];
                word |= ((uint32_t)quant_i8(y, scale) & 0xffu) << (8 * bb);
            }
            words[wd] = word;
        }
        *(v4u *)(xq_tiled + tiled_chunk_offset(r, c, k_tiles)) = v4u{words[0], words[1], words[2], words[3]};
    }
}

}  // namespace

void decode_prepare(const uint32_t *tables, uint32_t *seq_lens, int32_t *pos, uint32_t *slots, float *cos_sin,
                    uint32_t batch, uint32_t block_size, uint32_t max_blocks_per_seq, uint32_t num_blocks,
                    uint32_t head_dim, double theta, hipStream_t s) {
    if (batch == 0) return;
    decode_prepare_kernel<<<batch, 64, 0, s>>>(tables, seq_lens, pos, slots, cos_sin, block_size, max_blocks_per_seq,
                                               num_blocks, head_dim, theta);
}

void qkv_rope_append(const float *qkv, const float *cos_sin, const uint32_t *slots, uint16_t *q_out, uint16_t *k_pool,
                     uint16_t *v_pool, uint32_t batch, uint32_t heads, uint32_t kv_heads, uint32_t head_dim,
                     uint64_t pool_rows, hipStream_t s) {
    if (batch == 0) return;
    qkv_rope_append_kernel<<<batch, kBlock, 0, s>>>(qkv, cos_sin, slots, q_out, k_pool, v_pool, heads, kv_heads,
                                                    head_dim, pool_rows);
}

void swiglu_quantize_i8(const float *gu, int8_t *xq_tiled, float *sx, uint64_t m, uint64_t m_pad, uint64_t f,
                        hipStream_t s) {
    if (m_pad == 0 || f == 0) return;
    swiglu_quantize_kernel<<<(unsigned)m_pad, kBlock, 0, s>>>(gu, xq_tiled, sx, m, f);
}

}  // namespace k
}  // namespace fa
