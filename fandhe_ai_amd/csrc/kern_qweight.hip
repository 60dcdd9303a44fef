// Weight preparation: per-output-channel int8 / per-tensor e4m3 quantization
// of an f32 weight stored [k, n], and packing of the codes into the tile order
// the matrix-core kernels load (see kernels.hpp).  Runs once per weight.
#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {
using namespace fa::dev;

namespace {

// column absmax merged over k-slices with an integer max on the bit pattern;
// `absmax_bits` must be zero on entry
__global__ void __launch_bounds__(256) col_absmax_kernel(const float *__restrict__ w, uint64_t k, uint64_t n,
                                                         uint64_t rows_per_slice, unsigned int *__restrict__ absmax_bits) {
    uint64_t col = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (col >= n) return;
    uint64_t r0 = (uint64_t)blockIdx.y * rows_per_slice;
    uint64_t r1 = r0 + rows_per_slice < k ? r0 + rows_per_slice : k;
    float a = 0.0f;
    for (uint64_t r = r0; r < r1; ++r) a = fmaxf(a, fabsf(w[r * n + col]));
    atomicMax(&absmax_bits[col], __float_as_uint(a));
}

__global__ void __launch_bounds__(256) absmax_to_scale_kernel(float *__restrict__ scales, uint64_t n, uint64_t n_pad,
                                                              float divisor) {
    uint64_t col = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (col >= n_pad) return;
    scales[col] = col < n ? __fdiv_rn(scales[col], divisor) : 0.0f;
}

// One thread per 16-byte (TILE_K 64) or 32-byte (TILE_K 128) lane chunk.
// chunk id -> (nt, kt, g, c); element j of the chunk is W[TILE_K*kt + CH*g + j][16*nt + c].
template <int TILE_K, typename F>
__device__ __forceinline__ void pack_chunk(uint64_t chunk, uint64_t k_tiles, uint8_t *__restrict__ tiles, F code_at) {
    constexpr int CH = TILE_K / 4;                 // bytes per lane chunk
    uint64_t c = chunk % 16, g = (chunk / 16) % 4, tile = chunk / 64;
    uint64_t kt = tile % k_tiles, nt = tile / k_tiles;
    uint64_t col = nt * 16 + c, k0 = kt * TILE_K + g * CH;
    uint32_t words[CH / 4];
#pragma unroll
    for (int wd = 0; wd < CH / 4; ++wd) {
        uint32_t word = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) word |= (code_at(k0 + wd * 4 + b, col) & 0xffu) << (8 * b);
        words[wd] = word;
    }
    uint32_t *dst = (uint32_t *)(tiles + chunk * CH);
#pragma unroll
    for (int wd = 0; wd < CH / 4; ++wd) dst[wd] = words[wd];
}

__global__ void __launch_bounds__(256)
    quantize_pack_i8_kernel(const float *__restrict__ w, const float *__restrict__ scales, uint64_t k, uint64_t n,
                            uint64_t k_tiles, uint64_t n_chunks, int8_t *__restrict__ tiles) {
    uint64_t chunk = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (chunk >= n_chunks) return;
    pack_chunk<64>(chunk, k_tiles, (uint8_t *)tiles, [&](uint64_t kk, uint64_t col) -> uint32_t {
        if (kk >= k || col >= n) return 0u;
        return (uint32_t)quant_i8(w[kk * n + col], scales[col]);
    });
}

__global__ void __launch_bounds__(256)
    quantize_pack_e4m3_kernel(const float *__restrict__ w, const float *__restrict__ scale_p, uint64_t k, uint64_t n,
                              uint64_t k_tiles, uint64_t n_chunks, uint8_t *__restrict__ tiles) {
    uint64_t chunk = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (chunk >= n_chunks) return;
    float scale = *scale_p;
    pack_chunk<128>(chunk, k_tiles, tiles, [&](uint64_t kk, uint64_t col) -> uint32_t {
        if (kk >= k || col >= n || scale == 0.0f) return 0u;
        return f32_to_e4m3(__fdiv_rn(w[kk * n + col], scale));
    });
}

// per-column scales (scale_cols != 0) instead of one scale for the tensor
__global__ void __launch_bounds__(256)
    quantize_pack_e4m3_cols_kernel(const float *__restrict__ w, const float *__restrict__ scales, uint64_t k, uint64_t n,
                                   uint64_t k_tiles, uint64_t n_chunks, uint8_t *__restrict__ tiles) {
    uint64_t chunk = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (chunk >= n_chunks) return;
    pack_chunk<128>(chunk, k_tiles, tiles, [&](uint64_t kk, uint64_t col) -> uint32_t {
        if (kk >= k || col >= n) return 0u;
        const float scale = scales[col];
        return scale == 0.0f ? 0u : f32_to_e4m3(__fdiv_rn(w[kk * n + col], scale));
    });
}

template <int TILE_K>
__global__ void __launch_bounds__(256) pack_codes_kernel(const uint8_t *__restrict__ codes, uint64_t k, uint64_t n,
                                                         uint64_t k_tiles, uint64_t n_chunks, uint8_t *__restrict__ tiles) {
    uint64_t chunk = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (chunk >= n_chunks) return;
    pack_chunk<TILE_K>(chunk, k_tiles, tiles, [&](uint64_t kk, uint64_t col) -> uint32_t {
        if (kk >= k || col >= n) return 0u;
        return (uint32_t)codes[kk * n + col];
    });
}

template <int TILE_K>
__global__ void __launch_bounds__(256) unpack_codes_kernel(const uint8_t *__restrict__ tiles, uint64_t k, uint64_t n,
                                                           uint64_t k_tiles, uint8_t *__restrict__ codes) {
    constexpr int CH = TILE_K / 4;
    uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= k * n) return;
    uint64_t kk = idx / n, col = idx % n;
    uint64_t nt = col / 16, c = col % 16, kt = kk / TILE_K, g = (kk % TILE_K) / CH, j = kk % CH;
    codes[idx] = tiles[((nt * k_tiles + kt) * 64 + g * 16 + c) * CH + j];
}

}  // namespace

void weight_col_scales_i8(const float *w, uint64_t k, uint64_t n, uint64_t n_pad, float *scales, hipStream_t s) {
    weight_col_scales(w, k, n, n_pad, 127.0f, scales, s);
}

void weight_quantize_pack_e4m3_cols(const float *w, const float *scales, uint64_t k, uint64_t n, uint64_t k_pad,
                                    uint64_t n_pad, uint8_t *tiles, hipStream_t s) {
    uint64_t n_chunks = (k_pad / 128) * (n_pad / 16) * 64;
    if (n_chunks == 0) return;
    quantize_pack_e4m3_cols_kernel<<<(unsigned)((n_chunks + 255) / 256), 256, 0, s>>>(w, scales, k, n, k_pad / 128,
                                                                                       n_chunks, tiles);
}

void weight_col_scales(const float *w, uint64_t k, uint64_t n, uint64_t n_pad, float divisor, float *scales, hipStream_t s) {
    if (n_pad == 0) return;
    fill_u32((uint32_t *)scales, 0u, n_pad, s);
    if (k != 0 && n != 0) {
        uint64_t slices = k >= 64 ? 64 : 1;
        uint64_t rows_per_slice = (k + slices - 1) / slices;
        dim3 grid((unsigned)((n + 255) / 256), (unsigned)slices);
        col_absmax_kernel<<<grid, 256, 0, s>>>(w, k, n, rows_per_slice, (unsigned int *)scales);
    }
    absmax_to_scale_kernel<<<(unsigned)((n_pad + 255) / 256), 256, 0, s>>>(scales, n, n_pad, divisor);
}

void weight_quantize_pack_i8(const float *w, const float *scales, uint64_t k, uint64_t n, uint64_t k_pad,
                             uint64_t n_pad, int8_t *tiles, hipStream_t s) {
    uint64_t n_chunks = (k_pad / 64) * (n_pad / 16) * 64;
    if (n_chunks == 0) return;
    quantize_pack_i8_kernel<<<(unsigned)((n_chunks + 255) / 256), 256, 0, s>>>(w, scales, k, n, k_pad / 64, n_chunks,
                                                                                tiles);
}

void weight_quantize_pack_e4m3(const float *w, const float *scale, uint64_t k, uint64_t n, uint64_t k_pad,
                               uint64_t n_pad, uint8_t *tiles, hipStream_t s) {
    uint64_t n_chunks = (k_pad / 128) * (n_pad / 16) * 64;
    if (n_chunks == 0) return;
    quantize_pack_e4m3_kernel<<<(unsigned)((n_chunks + 255) / 256), 256, 0, s>>>(w, scale, k, n, k_pad / 128,
                                                                                  n_chunks, tiles);
}

void weight_pack_codes(const uint8_t *codes, uint64_t k, uint64_t n, uint64_t k_pad, uint64_t n_pad, int tile_k,
                       uint8_t *tiles, hipStream_t s) {
    uint64_t n_chunks = (k_pad / (uint64_t)tile_k) * (n_pad / 16) * 64;
    if (n_chunks == 0) return;
    unsigned grid = (unsigned)((n_chunks + 255) / 256);
    if (tile_k == 64)
        pack_codes_kernel<64><<<grid, 256, 0, s>>>(codes, k, n, k_pad / 64, n_chunks, tiles);
    else
        pack_codes_kernel<128><<<grid, 256, 0, s>>>(codes, k, n, k_pad / 128, n_chunks, tiles);
}

void weight_unpack_codes(const uint8_t *tiles, uint64_t k, uint64_t n, uint64_t k_pad, uint64_t n_pad, int tile_k,
                         uint8_t *codes, hipStream_t s) {
    (void)n_pad;
    if (k * n == 0) return;
    unsigned grid = (unsigned)((k * n + 255) / 256);
    if (tile_k == 64)
        unpack_codes_kernel<64><<<grid, 256, 0, s>>>(tiles, k, n, k_pad / 64, codes);
    else
        unpack_codes_kernel<128><<<grid, 256, 0, s>>>(tiles, k, n, k_pad / 128, codes);
}

}  // namespace k
}  // namespace fa
