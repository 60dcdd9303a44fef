// Glue kernels of the decoder: per-step position / slot bookkeeping and the
// cos / sin table of the step's positions (in the decode step RoPE, the KV
// append and SwiGLU live in the epilogues of the projections that feed them),
// and the same bookkeeping plus a stand-alone RoPE / KV-append pass for prompt
// chunks of several tokens per sequence.
#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {
using namespace fa::dev;

namespace {

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

// Prompt chunk of l_chunk tokens per sequence: row r = b * l_chunk + t sits at position seq_lens[b] + t.
// Same cos / sin arithmetic as the decode step, so a prompt token and the same token decoded later rotate
// identically.  seq_lens is advanced by a second launch, after every block of this one has read it.
__global__ void __launch_bounds__(64)
    prefill_prepare_kernel(const uint32_t *__restrict__ tables, const uint32_t *__restrict__ seq_lens,
                           uint32_t *__restrict__ slots, float *__restrict__ cos_sin, uint32_t l_chunk,
                           uint32_t block_size, uint32_t max_blocks_per_seq, uint32_t num_blocks, uint32_t head_dim,
                           double theta) {
    const uint32_t t = blockIdx.x, b = blockIdx.y;
    const uint64_t r = (uint64_t)b * l_chunk + t;
    const uint32_t p = seq_lens[b] + t;
    const uint32_t half = head_dim / 2;
    for (uint32_t i = threadIdx.x; i < half; i += 64) {
        double inv_freq = pow(theta, -2.0 * (double)i / (double)head_dim);
        double ang = (double)p * inv_freq;
        cos_sin[r * head_dim + i] = (float)cos(ang);
        cos_sin[r * head_dim + half + i] = (float)sin(ang);
    }
    if (threadIdx.x == 0) {
        uint32_t slot = 0xffffffffu;
        uint32_t blk_idx = p / block_size;
        if (blk_idx < max_blocks_per_seq) {
            uint32_t id = tables[(uint64_t)b * max_blocks_per_seq + blk_idx];
            if (id < num_blocks) slot = id * block_size + p % block_size;
        }
        slots[r] = slot;
    }
}

// row_lens (optional): row b's prompt is only row_lens[b] <= l_chunk tokens long and the rest of its chunk
// is padding; its last token is then row b * l_chunk + row_lens[b] - 1.  seq_lens advances by the whole chunk
// either way (the attention of the pass places token t at seq_len - l_chunk + t); trim_lens_kernel takes the
// padding off afterwards.
__global__ void advance_lens_kernel(uint32_t *__restrict__ seq_lens, int32_t *__restrict__ last_rows, uint32_t batch,
                                    uint32_t l_chunk, const uint32_t *__restrict__ row_lens) {
    const uint32_t b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b < batch) {
        seq_lens[b] += l_chunk;
        last_rows[b] = (int32_t)(b * l_chunk + (row_lens ? row_lens[b] : l_chunk) - 1);
    }
}

__global__ void trim_lens_kernel(uint32_t *__restrict__ seq_lens, const uint32_t *__restrict__ row_lens, uint32_t batch,
                                 uint32_t l_chunk) {
    const uint32_t b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b < batch) seq_lens[b] -= l_chunk - row_lens[b];
}

// qkv [rows, (heads + 2 kv_heads) head_dim] f32 -> q rotated, bf16 [rows, heads head_dim]; K rotated and V
// as they are, bf16, to pool row slots[r] (rows whose slot is out of range are skipped).  The arithmetic
// is the one of the fused decode epilogue (rotate-half pairing, one rounding to bf16).
__global__ void __launch_bounds__(256)
    rope_append_kernel(const float *__restrict__ qkv, const float *__restrict__ cos_sin, const uint32_t *__restrict__ slots,
                       uint16_t *__restrict__ q_out, uint16_t *__restrict__ k_pool, uint16_t *__restrict__ v_pool,
                       uint32_t heads, uint32_t kv_heads, uint32_t head_dim, uint64_t pool_rows) {
    const uint64_t r = blockIdx.x;
    const uint32_t half = head_dim / 2, all_heads = heads + 2 * kv_heads;
    const uint64_t eq = (uint64_t)heads * head_dim, ekv = (uint64_t)kv_heads * head_dim;
    const float *row = qkv + r * (eq + 2 * ekv);
    const uint64_t slot = slots[r];
    for (uint32_t idx = threadIdx.x; idx < all_heads * half; idx += 256) {
        const uint32_t h = idx / half, d = idx % half;
        float x0 = row[(uint64_t)h * head_dim + d], x1 = row[(uint64_t)h * head_dim + half + d];
        uint16_t *dst = nullptr;
        if (h < heads) {
            dst = q_out + r * eq + (uint64_t)h * head_dim + d;
        } else if (slot < pool_rows) {
            const uint32_t hk = h - heads;
            dst = (hk < kv_heads ? k_pool + slot * ekv + (uint64_t)hk * head_dim
                                 : v_pool + slot * ekv + (uint64_t)(hk - kv_heads) * head_dim) + d;
        }
        if (h < heads + kv_heads) {
            const float c = cos_sin[r * head_dim + d], sn = cos_sin[r * head_dim + half + d];
            const float r0 = __fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, sn));
            const float r1 = __fadd_rn(__fmul_rn(x1, c), __fmul_rn(x0, sn));
            x0 = r0;
            x1 = r1;
        }
        if (dst) {
            dst[0] = f32_to_bf16(x0);
            dst[half] = f32_to_bf16(x1);
        }
    }
}

}  // namespace

void prefill_prepare(const uint32_t *tables, const uint32_t *seq_lens, uint32_t *slots, float *cos_sin, uint32_t batch,
                     uint32_t l_chunk, uint32_t block_size, uint32_t max_blocks_per_seq, uint32_t num_blocks,
                     uint32_t head_dim, double theta, hipStream_t s) {
    if (batch == 0 || l_chunk == 0) return;
    prefill_prepare_kernel<<<dim3(l_chunk, batch), 64, 0, s>>>(tables, seq_lens, slots, cos_sin, l_chunk, block_size,
                                                              max_blocks_per_seq, num_blocks, head_dim, theta);
}

void advance_seq_lens(uint32_t *seq_lens, int32_t *last_rows, uint32_t batch, uint32_t l_chunk, const uint32_t *row_lens,
                      hipStream_t s) {
    if (batch == 0) return;
    advance_lens_kernel<<<(batch + 63) / 64, 64, 0, s>>>(seq_lens, last_rows, batch, l_chunk, row_lens);
}

void trim_seq_lens(uint32_t *seq_lens, const uint32_t *row_lens, uint32_t batch, uint32_t l_chunk, hipStream_t s) {
    if (batch == 0) return;
    trim_lens_kernel<<<(batch + 63) / 64, 64, 0, s>>>(seq_lens, row_lens, batch, l_chunk);
}

void rope_append(const float *qkv, const float *cos_sin, const uint32_t *slots, uint16_t *q_out, uint16_t *k_pool,
                 uint16_t *v_pool, uint64_t rows, uint32_t heads, uint32_t kv_heads, uint32_t head_dim, uint64_t pool_rows,
                 hipStream_t s) {
    if (rows == 0) return;
    rope_append_kernel<<<(unsigned)rows, 256, 0, s>>>(qkv, cos_sin, slots, q_out, k_pool, v_pool, heads, kv_heads, head_dim,
                                                     pool_rows);
}

void decode_prepare(const uint32_t *tables, uint32_t *seq_lens, int32_t *pos, uint32_t *slots, float *cos_sin,
                    uint32_t batch, uint32_t block_size, uint32_t max_blocks_per_seq, uint32_t num_blocks,
                    uint32_t head_dim, double theta, hipStream_t s) {
    if (batch == 0) return;
    decode_prepare_kernel<<<batch, 64, 0, s>>>(tables, seq_lens, pos, slots, cos_sin, block_size, max_blocks_per_seq,
                                               num_blocks, head_dim, theta);
}

}  // namespace k
}  // namespace fa
