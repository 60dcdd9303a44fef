// Glue kernel of the decode step: per-step position / slot bookkeeping and the
// cos / sin table of the step's positions.  (RoPE, the KV append and SwiGLU
// live in the epilogues of the projections that feed them.)
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

}  // namespace

void decode_prepare(const uint32_t *tables, uint32_t *seq_lens, int32_t *pos, uint32_t *slots, float *cos_sin,
                    uint32_t batch, uint32_t block_size, uint32_t max_blocks_per_seq, uint32_t num_blocks,
                    uint32_t head_dim, double theta, hipStream_t s) {
    if (batch == 0) return;
    decode_prepare_kernel<<<batch, 64, 0, s>>>(tables, seq_lens, pos, slots, cos_sin, block_size, max_blocks_per_seq,
                                               num_blocks, head_dim, theta);
}

}  // namespace k
}  // namespace fa
