// Launchers of the gfx950 kernels.  Each enqueues on `stream` and returns;
// shapes have been validated by the caller (capi_*.cpp) against what the
// kernel and its grid assume.  Sizes are element counts unless named _bytes.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace fa {
namespace k {

// What a row kernel pulls into L2 for the linear that follows it (dev::prefetch_weights): the first `bytes` of the
// weight tiles each block of that launch starts with.
struct WeightPrefetch {
    const int8_t *w = nullptr;   // tile-ordered codes of the next linear; null: nothing to pull
    uint32_t blocks = 0;         // blocks of the next launch (one appended block each)
    uint32_t n_tiles = 0;        // column tiles of the weight (tile indices are clamped to it, as the kernels do)
    uint32_t k_tiles = 0;        // KiB per column tile
    uint32_t half_tiles = 0;     // != 0: block j starts at tile (j / half) * 2 * half + j % half (the q | k | v pairing)
    uint32_t tile_stride = 1;    // otherwise block j starts at tile j * tile_stride
    uint32_t pair_step = 0;      // != 0: the block also reads tile first + pair_step
    uint32_t bytes = 0;          // bytes pulled from the start of each tile (multiple of 16)
    uint32_t ksplit = 0;         // != 0: the next launch is the split-k form with this many blocks per group; block j
                                 // reads tiles group * ksplit .. + ksplit - 1 from its member's share of k onwards
};


// ---- weight tile order ---------------------------------------------------
// int8 weights W[k, n] are stored as tiles of 16 columns x 64 k-values, one
// tile = 1 KiB laid out in the order one wavefront loads it for the int8
// matrix instruction: byte ((g*16 + c)*16 + j) of tile (nt, kt) holds
// W[64*kt + 16*g + j][16*nt + c]   (g = 0..3, c = 0..15, j = 0..15),
// tiles ordered [nt][kt].  e4m3 weights use tiles of 16 columns x 128
// k-values (2 KiB): byte ((g*16 + c)*32 + j) holds W[128*kt + 32*g + j][16*nt + c].
constexpr int kTileN = 16;
constexpr int kTileK8 = 64;     // int8 k-values per tile
constexpr int kTileKF8 = 128;   // e4m3 k-values per tile

// ---- elementwise / small ops (kern_elementwise.hip) ------------------------
void silu_mul_f32(const float *gate, const float *up, float *out, uint64_t n, hipStream_t s);
void add_f32(const float *a, const float *b, float *out, uint64_t n, hipStream_t s);
void argmax_rows_f32(const float *x, int32_t *out, uint64_t rows, uint64_t cols, hipStream_t s);
void gather_rows_f32(const float *table, uint64_t table_rows, uint64_t cols, const int32_t *idx,
                     float *out, uint64_t rows, hipStream_t s);
void convert_f32_to_bf16(const float *in, uint16_t *out, uint64_t n, hipStream_t s);
void convert_bf16_to_f32(const uint16_t *in, float *out, uint64_t n, hipStream_t s);
void rope_f32(const float *x, const int32_t *pos, float *out, uint64_t rows, uint64_t heads,
              uint64_t head_dim, double theta, hipStream_t s);
void fill_u32(uint32_t *p, uint32_t v, uint64_t n, hipStream_t s);
// N(mean, std) from a counter-based hash of (seed, index); out is f32 or bf16
void fill_normal(void *out, int out_bf16, uint64_t n, uint64_t seed, float mean, float std, hipStream_t s);

// ---- norms / quantizers (kern_norm_quant.hip) -------------------------------
void rmsnorm_f32(const float *x, const float *w, float *out, uint64_t rows, uint64_t hidden,
                 float eps, hipStream_t s);
// Per-token int8 quantization.  in_bf16 selects the input type.  xq_rowmajor
// (nullable) receives [m, k]; xq_tiled (nullable) receives the activation
// tile order used by the skinny GEMM: tiles [mt][kt] of 16 rows x 64 k in
// the same byte order as weight tiles, rows >= m zero-filled (m_pad rows).
void quantize_rows_i8(const void *x, bool in_bf16, int8_t *xq_rowmajor, int8_t *xq_tiled, float *sx,
                      uint64_t m, uint64_t m_pad, uint64_t k, uint64_t k_pad, hipStream_t s);
// Per-token quantization when the row absmax is already known as `parts` partial maxima per row
// (pmax[m, parts]): x f32 or bf16 [m, k] -> activation tiles + sx[m].  k a multiple of 64.
void quantize_rows_from_pmax(const void *x, bool in_bf16, const float *pmax, uint32_t parts, int8_t *xq_tiled,
                             float *sx, uint64_t m, uint64_t m_pad, uint64_t k, hipStream_t s);
// RMSNorm fused with the quantizer (f32 in): out_f32 nullable.
void rmsnorm_quantize_i8(const float *x, const float *w, float eps, float *out_f32, int8_t *xq_tiled,
                         float *sx, uint64_t m, uint64_t m_pad, uint64_t hidden, hipStream_t s,
                         const WeightPrefetch &pull = WeightPrefetch{});
// The same fused pair with row-major codes [m, hidden] (operand layout of the prefill GEMMs); hidden a
// multiple of 16 and at most 16384.
void rmsnorm_quantize_rows_i8(const float *x, const float *w, float eps, int8_t *xq_rowmajor, float *sx, uint64_t m,
                              uint64_t hidden, hipStream_t s);
// act = silu(gate) * up of gu [m, 2 f] (gate columns first) quantized per token, row-major codes [m, f] or
// (tiled, f a multiple of 64) activation tiles with rows padded to 16; the f32 products are not stored.  f a
// multiple of 16.  products: gu is [m, f] and holds the products already (gemm_w8a8_swiglu_mfma), only the quantizer runs.
void swiglu_quantize_rows_i8(const float *gu, int8_t *xq, float *sx, uint64_t m, uint64_t f, hipStream_t s,
                             bool tiled = false, bool products = false);
// Per-tensor absmax -> scale = absmax / 448 (one f32) then e4m3 codes.
void quantize_tensor_e4m3(const float *x, uint8_t *q, float *scale, float *absmax_scratch, uint64_t n,
                          hipStream_t s);

// Per-token e4m3 (scale = row absmax / 448): row-major codes [m, k_pad], rows zero-padded to k_pad, scales sx[m].
void quantize_rows_e4m3(const void *x, bool in_bf16, uint8_t *xq_rowmajor, float *sx, uint64_t m, uint64_t k,
                        uint64_t k_pad, hipStream_t s);

// ---- weights (kern_qweight.hip) ----------------------------------------------
// Column absmax / 127 of w[k, n] (f32, row-major) -> scales[n_pad] (padding 0)
void weight_col_scales_i8(const float *w, uint64_t k, uint64_t n, uint64_t n_pad, float *scales,
                          hipStream_t s);
// The same with scale = column absmax / divisor (448 for e4m3 weights with one scale per output channel).
void weight_col_scales(const float *w, uint64_t k, uint64_t n, uint64_t n_pad, float divisor, float *scales, hipStream_t s);
void weight_quantize_pack_e4m3_cols(const float *w, const float *scales, uint64_t k, uint64_t n, uint64_t k_pad,
                                    uint64_t n_pad, uint8_t *tiles, hipStream_t s);
void weight_quantize_pack_i8(const float *w, const float *scales, uint64_t k, uint64_t n,
                             uint64_t k_pad, uint64_t n_pad, int8_t *tiles, hipStream_t s);
// Pack row-major codes [k, n] (1 byte each) into tile order; tile_k = 64 or 128.
void weight_pack_codes(const uint8_t *codes, uint64_t k, uint64_t n, uint64_t k_pad, uint64_t n_pad,
                       int tile_k, uint8_t *tiles, hipStream_t s);
void weight_unpack_codes(const uint8_t *tiles, uint64_t k, uint64_t n, uint64_t k_pad, uint64_t n_pad,
                         int tile_k, uint8_t *codes, hipStream_t s);
void weight_quantize_pack_e4m3(const float *w, const float *scale, uint64_t k, uint64_t n,
                               uint64_t k_pad, uint64_t n_pad, uint8_t *tiles, hipStream_t s);
void tensor_absmax_f32(const float *x, uint64_t n, float *absmax, hipStream_t s);
void scale_from_absmax(const float *absmax, float divisor, float *scale, hipStream_t s);

// ---- f32 GEMM with the reference's summation order (kern_gemm_f32.hip) -------
void gemm_f32(const float *a, const float *b, const float *bias, float *out, uint64_t m, uint64_t n,
              uint64_t k, int relu, hipStream_t s);
// Which kernel that call launches: 1 the few-rows vector kernel, 2 the matrix-core kernel.
int gemm_f32_form(uint64_t m, uint64_t n, uint64_t k);

// ---- skinny (decode-shape) quantized linears (kern_qlinear.hip) ---------------
struct EpilogueI8 {
    const float *sx;      // [m] activation scales
    const float *sw;      // [n_pad] weight scales
    const float *bias;    // nullable [n]
    const float *residual;  // nullable [m, n] f32, added last (may alias out when out is f32)
    int32_t *acc_out;     // nullable [m, n]
    void *out;            // [m, n] f32 or bf16
    int out_bf16;
};
// What the row kernel in front of each of the launches below should pull (see WeightPrefetch); same arguments as
// the launch itself, `budget` = bytes of one pull.
struct QkvRopeTargets;
struct SplitKArea;
WeightPrefetch prefetch_for_linear_w8a8_skinny(const int8_t *w_tiles, uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus,
                                               uint64_t budget, const SplitKArea *sk = nullptr);
WeightPrefetch prefetch_for_linear_w8a8_qkv_rope_skinny(const int8_t *w_tiles, uint64_t m, uint64_t n_pad, uint64_t k_pad,
                                                        const QkvRopeTargets &t, uint64_t budget);
// Where the blocks of a split-k decode linear leave their partial tiles and take their tickets: one area per
// context (launches that use it are ordered by the context's stream).  The counters are zero between launches.
struct SplitKArea {
    void *partial = nullptr;
    uint64_t partial_bytes = 0;
    uint32_t *counters = nullptr;
    uint32_t n_counters = 0;
    int xcd_local = 0;          // probed: workgroups b and b + 8 of a launch run on the same XCD (share an L2)
    // Where the members of a group note the XCD they run on (one word per block of a launch, beside the partial
    // tiles) and where the last arriver reports a group whose members did not share one: a word of pinned host
    // memory that the device writes and the host reads at every entry (the results of that launch are wrong).
    uint32_t *xcc_seen = nullptr;
    uint32_t n_xcc_seen = 0;
    uint32_t *fault = nullptr;
};
// out[b] = hardware id of the XCD workgroup b of the probe launch ran on (b < blocks)
void xcc_id_probe(uint32_t *out, uint32_t blocks, hipStream_t s);
// Row work that a decode-shape linear of at most four rows does for itself (row_prologue.hpp) instead of reading
// ready-made codes: the RMSNorm + per-token quantizer of x (norm_w set), or the quantizer of x from `parts` partial
// absolute maxima per row (norm_w null).  Same arithmetic as the stand-alone row kernels, so the linear's result
// is bit-identical to theirs followed by the unfused linear.  xq_tiled_out / sx_out (nullable) receive what the
// stand-alone kernel would have written (one block of the linear writes them).
struct RowPrologue {
    const float *x = nullptr;       // [m, k] f32
    const float *norm_w = nullptr;  // [k]
    const float *pmax = nullptr;    // [m, parts]
    uint32_t parts = 0;
    float eps = 0.0f, inv_n = 0.0f;
    int8_t *xq_tiled_out = nullptr;
    float *sx_out = nullptr;
};
// Whether the three linears of a decode step take the row work in front of them into their own launch for m rows
// (the caller then skips the row kernel and passes a RowPrologue): q | k | v and gate | up take the norm + quantizer,
// the down projection the quantizer from partial maxima.
bool qkv_rope_fuses_norm(uint64_t m, uint64_t k_pad);
bool swiglu_fuses_norm(uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus);
bool plain_fuses_pmax_quantizer(uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus);
// xq_tiled: activation tiles (see quantize_rows_i8); m <= 64 (one to four row tiles of 16 per block).
// sk (optional): lets narrow weights split k over groups of blocks (m <= 32).
void linear_w8a8_skinny(const int8_t *xq_tiled, const int8_t *w_tiles, uint64_t m, uint64_t n,
                        uint64_t n_pad, uint64_t k_pad, const EpilogueI8 &ep, int num_cus,
                        hipStream_t s, const SplitKArea *sk = nullptr, const RowPrologue *pro = nullptr);
// gate_up projection fused with SwiGLU: the weight is [k, n] with gate columns [0, n/2) and up columns
// [n/2, n), n/2 a multiple of 16; act[m, n/2] = silu(gate) * up (f32) and pmax[m, n/32] receives the
// absmax of every 16-column block of act (consumed by quantize_rows_from_pmax).
void linear_w8a8_swiglu_skinny(const int8_t *xq_tiled, const int8_t *w_tiles, const float *sx, const float *sw,
                               uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad, float *act, float *pmax,
                               int waves, int num_cus, hipStream_t s, const RowPrologue *pro = nullptr);
// Fused q | k | v projection of a decode step: the weight is [k, (heads + 2 kv_heads) head_dim], head_dim a
// multiple of 32; q and k heads are rotated (rotate-half pairing, cos/sin of the row's position from
// cos_sin[m][head_dim]) and rounded once to bf16; q goes to q_out [m, heads * head_dim], the new K / V rows
// to pool row slots[r] (rows whose slot is out of range are skipped).
struct QkvRopeTargets {
    const float *cos_sin;
    const uint32_t *slots;
    uint16_t *q_out, *k_pool, *v_pool;
    uint32_t heads, kv_heads, head_dim;
    uint64_t pool_rows;
};
void linear_w8a8_qkv_rope_skinny(const int8_t *xq_tiled, const int8_t *w_tiles, const float *sx, const float *sw,
                                 uint64_t m, uint64_t n_pad, uint64_t k_pad, const QkvRopeTargets &t, hipStream_t s,
                                 const RowPrologue *pro = nullptr);
// The same for 65 to a few hundred rows, on the weight-stationary kernel (see linear_w8a8_rows): whether it applies to a
// shape, and the launch.  Bit for bit what linear_w8a8_rows into an [m, n] f32 buffer followed by rope_append leaves.
extern int g_rows_rope;
bool linear_w8a8_qkv_rope_rows_applies(uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus, const SplitKArea *sk,
                                       const QkvRopeTargets &t);
void linear_w8a8_qkv_rope_rows(const int8_t *xq_tiled, const int8_t *w_tiles, const float *sx, const float *sw, uint64_t m,
                               uint64_t n_pad, uint64_t k_pad, const QkvRopeTargets &t, hipStream_t s);
// The q | k | v projection of a prompt pass on the large-tile GEMM with rope_append's work in its epilogue (aq row-major
// codes): bit for bit what gemm_w8a8_mfma into an [m, n] f32 buffer followed by rope_append leaves in q_out and the pools.
bool gemm_w8a8_qkv_rope_applies(uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad, uint32_t heads, uint32_t kv_heads,
                                uint32_t head_dim, int num_cus);
void gemm_w8a8_qkv_rope_mfma(const int8_t *aq, const int8_t *w_tiles, const float *sx, const float *sw, uint64_t m, uint64_t k_pad,
                             const QkvRopeTargets &t, hipStream_t s);
// a: bf16 [m, k] row-major (k == k_pad required), m <= 32.
void linear_w8a16_skinny(const uint16_t *a, const int8_t *w_tiles, const float *sw, uint64_t m,
                         uint64_t n, uint64_t n_pad, uint64_t k_pad, void *out, int out_bf16,
                         int num_cus, hipStream_t s, const SplitKArea *sk = nullptr);

// A few hundred rows (65 up) against a weight with about one column tile per compute unit: the weight-stationary
// kernel (weights in registers, rows streamed in groups of 64).  xq_tiled: activation tiles with rows padded to 16,
// as for linear_w8a8_skinny.  linear_w8a8_rows_applies says whether a shape should take it.
// With a split-k area (and then a workspace of linear_w8a8_rows_workspace_bytes for the launch), weights with a deep
// k (8192 .. 14336) take a form that splits k over four blocks of an XCD, each keeping its quarter of the weights in
// registers: a block then pulls a quarter of the activations.
// g_rows_kernel: 0: by shape, 1: never (the tiled GEMMs for every prompt pass), 2: the form without the split
// whenever it can run, 3: the split form whenever it can run
extern int g_rows_kernel;
bool linear_w8a8_rows_applies(uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus, const SplitKArea *sk = nullptr);
uint64_t linear_w8a8_rows_workspace_bytes(uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus, const SplitKArea *sk);
void linear_w8a8_rows(const int8_t *xq_tiled, const int8_t *w_tiles, uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad,
                      const EpilogueI8 &ep, int num_cus, hipStream_t s, const SplitKArea *sk = nullptr, void *workspace = nullptr,
                      uint64_t workspace_bytes = 0);

// ---- prefill-shape MFMA GEMMs (kern_gemm_mfma.hip) -----------------------------
// aq: int8 [m, k_pad] row-major.  workspace (optional, gemm_w8a8_workspace_bytes): lets a matrix with too few
// output tiles to occupy the device split k across blocks; the int32 partial sums meet there and are
// added exactly, so the result does not depend on the split.
// sk (optional): with it and the workspace, a launch of at most half a device of 256 x 128 tiles lets two or four blocks
// of an XCD share a tile, a part of k each (they meet in the workspace; the last to arrive finishes the tile).
void gemm_w8a8_mfma(const int8_t *aq, const int8_t *w_tiles, uint64_t m, uint64_t n, uint64_t n_pad,
                    uint64_t k_pad, const EpilogueI8 &ep, int num_cus, hipStream_t s, void *workspace = nullptr,
                    uint64_t workspace_bytes = 0, const SplitKArea *sk = nullptr);
uint64_t gemm_w8a8_workspace_bytes(uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad, int num_cus);
// The gate | up projection with SwiGLU in its epilogue (large-tile kernel, m >= 65, f a multiple of 128, k_pad of 128):
// w_tiles is the [k, 2 f] weight with the gate columns first; out receives silu(gate) * up, f32 [m, f], bit for bit
// what gemm_w8a8_mfma into an [m, 2 f] buffer followed by the SwiGLU pass computes.
extern int g_gemm_pair;       // 1: one block per tile on the 256 x 128 tiles of the large-tile kernel; 2: shared tiles only
                              // where the tiles alone cover half the device
extern int g_gemm_swiglu;     // bit 0: SwiGLU stays a pass of its own; bit 1: so do RoPE and the K / V append (below)
bool gemm_w8a8_swiglu_applies(uint64_t m, uint64_t f, uint64_t n_pad, uint64_t k_pad);
void gemm_w8a8_swiglu_mfma(const int8_t *aq, const int8_t *w_tiles, const float *sx, const float *sw, uint64_t m, uint64_t f,
                           uint64_t k_pad, float *out, int num_cus, hipStream_t s);
// Which kernel the two launchers pick for a shape under the current tuning knobs: big_ntb column tiles of
// 16 per block of the large-tile kernel (0: the 128 x 128 kernel), wavefronts per block, k splits.
struct GemmPlan {
    int big_ntb, waves;
    uint32_t splits;
};
GemmPlan gemm_plan(bool fp8, uint64_t m, uint64_t n_pad, uint64_t k_pad, int num_cus);
// aq: e4m3 [m, k_pad] row-major; scales are device scalars.
void gemm_e4m3_mfma(const uint8_t *aq, const uint8_t *w_tiles, const float *a_scale,
                    const float *w_scale, uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad,
                    void *out, int out_bf16, int num_cus, hipStream_t s);
// The same with one scale per row of aq (sx[m]) and one per output column (sw[n_pad]):
// out = acc * (sx[row] * sw[col]) (+ bias[col]).
void gemm_e4m3_rows_mfma(const uint8_t *aq, const uint8_t *w_tiles, const float *sx, const float *sw, const float *bias,
                         uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad, void *out, int out_bf16, int num_cus,
                         hipStream_t s);
// Decode shape (m <= 64) of the same operator: a weight-streaming kernel, one block per 16-column tile, k split
// over the block's wavefronts.
void linear_e4m3_skinny(const uint8_t *aq, const uint8_t *w_tiles, const float *sx, const float *sw, const float *bias,
                        uint64_t m, uint64_t n, uint64_t n_pad, uint64_t k_pad, void *out, int out_bf16, hipStream_t s);

// ---- paged KV (kern_paged.hip) ---------------------------------------------------
struct PagedShape {
    uint32_t num_blocks, block_size, e_kv, batch, l_new, num_heads, num_kv_heads, head_dim,
        max_blocks_per_seq;
    float scale;
    // upper bound the host knows for the positions any row holds after this call's new tokens (0: unknown,
    // the table width is used); only steers the choice between the two prefill forms
    uint32_t ctx_hint = 0;
};
// Row scatter; elem_bytes 2 or 4; slots bounds-checked against pool_rows.
void paged_kv_append(const void *k_new, const void *v_new, void *k_pool, void *v_pool,
                     const uint32_t *slots, uint64_t rows, uint64_t e, uint64_t pool_rows,
                     int elem_bytes, hipStream_t s);
// Generic attention with the reference's per-row summation order; is_bf16
// selects the storage type; workspace holds query_rows * s_stride f32.
void paged_attention_generic(const void *q, const void *k_pool, const void *v_pool,
                             const uint32_t *tables, const uint32_t *seq_lens, const PagedShape &ps,
                             int is_bf16, float *workspace, uint64_t s_stride, void *out,
                             hipStream_t s);
// Decode fast path: bf16, head_dim 128, block_size 16, l_new 1, group <= 16.
// Workspace bytes needed for a given shape:
uint64_t paged_decode_workspace_bytes(const PagedShape &ps, uint32_t waves_per_cu);
void paged_attention_decode_bf16(const uint16_t *q, const uint16_t *k_pool, const uint16_t *v_pool,
                                 const uint32_t *tables, const uint32_t *seq_lens,
                                 const PagedShape &ps, uint32_t waves_per_cu, void *workspace,
                                 void *out, int out_bf16, float *pmax /*nullable: [batch, heads] absmax*/,
                                 hipStream_t s);
// The same with the merged result handed straight to the per-token int8 quantizer instead of being
// stored: rounded once to bf16, quantized per sequence into activation tiles xq_tiled (rows padded to
// m_pad, a multiple of 16) with scales sx.  Needs num_heads <= 32; otherwise call the form above and
// quantize separately.
void paged_attention_decode_bf16(const uint16_t *q, const uint16_t *k_pool, const uint16_t *v_pool,
                                 const uint32_t *tables, const uint32_t *seq_lens, const PagedShape &ps,
                                 uint32_t waves_per_cu, void *workspace, void *out, int out_bf16, float *pmax,
                                 int8_t *xq_tiled, float *sx, uint32_t m_pad, hipStream_t s,
                                 const WeightPrefetch &pull = WeightPrefetch{});

// Decode attention of a few short sequences, finished in one launch (a block per (sequence, kv head), no partial
// results, no merge): out_f32 [batch][num_heads][128] = the output values rounded to bf16 (the operator's output
// type), pmax [batch][num_heads] = absmax of every head's slice, for a per-token quantizer inside the projection that
// follows (RowPrologue).  Same shapes as the fast path above; meant for contexts up to kDecodeOneMaxCtx tokens.
constexpr uint32_t kDecodeOneMaxCtx = 1024;
extern int g_decode_one;      // 0: by shape and context, 1: never (tuning aid)
void paged_attention_decode_one_bf16(const uint16_t *q, const uint16_t *k_pool, const uint16_t *v_pool, const uint32_t *tables,
                                     const uint32_t *seq_lens, const PagedShape &ps, float *out_f32, float *pmax, hipStream_t s);

// Prefill fast path: bf16, head_dim 128, block_size 16, l_new > 1, group <= 16.  Causal over the cached
// positions: new token t of a row sees positions below seq_len - l_new + t + 1.
uint64_t paged_prefill_workspace_bytes(const PagedShape &ps, uint32_t waves_per_cu);
void paged_attention_prefill_bf16(const uint16_t *q, const uint16_t *k_pool, const uint16_t *v_pool,
                                  const uint32_t *tables, const uint32_t *seq_lens, const PagedShape &ps,
                                  uint32_t waves_per_cu, void *workspace, void *out, int out_bf16, hipStream_t s);

// ---- sampling (kern_sampling.hip) ------------------------------------------------
// one row of a per-row sampling table (the layout of fa_row_sampling)
struct RowPolicy {
    uint64_t rng_state;
    float temperature;
    uint32_t top_k;
    int32_t strategy;
    uint32_t reserved;
};
// One token per row of logits [rows, vocab] by temperature (top_k_mode 0) or top-k (1) sampling with the
// reference's arithmetic; row b takes the (b + 1)-th draw of the xorshift64* generator at rng_state, which is
// advanced by `rows` draws afterwards.  A row with a non-finite logit gets token -1.
void sample_rows(const float *logits, int32_t *tokens, uint64_t *rng_state, uint32_t rows, uint32_t vocab, int top_k_mode,
                 float temperature, uint32_t top_k, hipStream_t s);
// The f32 sampling weights of every row instead of a draw (mode 0 temperature, 1 top-k, 2 greedy: one-hot at the
// first maximum); status[row] = 1 and a NaN row where a logit is not finite, else 0.
void sampling_weights(const float *logits, float *weights, int32_t *status, uint32_t rows, uint32_t vocab, int mode,
                      float temperature, uint32_t top_k, hipStream_t s);
// Acceptance step of sampled speculative decoding for one sequence: p_weights [k + 1, vocab] (target), q_weights
// [k, vocab] (draft; unused when k == 0), the k draft tokens by value; result[0 .. 2] = accepted drafts, the token
// that follows them, status.  Draws from, and advances, the generator state.
constexpr uint32_t kMaxDraftTokens = 32;
struct DraftTokens {
    int32_t d[kMaxDraftTokens];
};
void speculative_accept(const float *p_weights, const float *q_weights, const DraftTokens &drafts, uint32_t k, uint32_t vocab,
                        uint64_t *rng_state, int32_t *result, hipStream_t s);
// The same with one RowPolicy per row (strategy 0 takes the first maximum and draws nothing; otherwise one
// draw from the row's own state, which is advanced in place).
void sample_rows_policy(const float *logits, int32_t *tokens, RowPolicy *policy, uint32_t rows, uint32_t vocab, hipStream_t s);

// ---- measurement aid (kern_probe.hip) -------------------------------------------
// Launches a register-only loop of one matrix instruction kind (0: i32_16x16x64_i8, 1: i32_32x32x32_i8,
// 2: scaled f32_16x16x128 on e4m3) whose operand bits come from `operands` (64 KiB); returns the number
// of multiply-add operations x 2 the launch performs.  sink: one int, never written in practice.
// Streaming read of `bytes` (a multiple of 16 * blocks) by `blocks` blocks of `threads` threads (non-temporal
// loads unless tuning key 15 asks for ordinary ones).
void stream_read_probe(const void *src, uint64_t bytes, int blocks, int threads, int *sink, hipStream_t s);
// The L2 -> compute unit path (l2_path_kernel): cold_bytes == 0 reads the hot region alone; in_flight 8 or 16,
// hot_per_cold 0 or 2; false for any other combination.
bool l2_path_probe(const void *cold, uint64_t cold_bytes, const void *hot, uint32_t hot_bytes, uint32_t hot_passes, int in_flight,
                   int hot_per_cold, int blocks, int threads, int *sink, hipStream_t s);
double matrix_rate_probe(int kind, const void *operands, uint32_t iters, int num_cus, int *sink, hipStream_t s);

// ---- decode-step glue (kern_decoder.hip) --------------------------------------
// Per step, before the layers: pos[b] = seq_lens[b]; slot[b] from the block
// table (UINT32_MAX when the table cannot hold the position); seq_lens[b] += 1;
// cos/sin table [batch, head_dim/2] for the positions.
void decode_prepare(const uint32_t *tables, uint32_t *seq_lens, int32_t *pos, uint32_t *slots, float *cos_sin,
                    uint32_t batch, uint32_t block_size, uint32_t max_blocks_per_seq, uint32_t num_blocks,
                    uint32_t head_dim, double theta, hipStream_t s);

// Prompt chunks (several new tokens per sequence): row b * l_chunk + t is at position seq_lens[b] + t;
// slots [batch * l_chunk] and the cos/sin table [batch * l_chunk, head_dim] as in decode_prepare.
void prefill_prepare(const uint32_t *tables, const uint32_t *seq_lens, uint32_t *slots, float *cos_sin, uint32_t batch,
                     uint32_t l_chunk, uint32_t block_size, uint32_t max_blocks_per_seq, uint32_t num_blocks,
                     uint32_t head_dim, double theta, hipStream_t s);
// seq_lens[b] += l_chunk; last_rows[b] = row of the chunk's last token of sequence b
void advance_seq_lens(uint32_t *seq_lens, int32_t *last_rows, uint32_t batch, uint32_t l_chunk, const uint32_t *row_lens,
                      hipStream_t s);
// After a padded prompt pass: seq_lens[b] -= l_chunk - row_lens[b].
void trim_seq_lens(uint32_t *seq_lens, const uint32_t *row_lens, uint32_t batch, uint32_t l_chunk, hipStream_t s);
// RoPE on the q and k heads of qkv [rows, (heads + 2 kv_heads) head_dim] (f32), one rounding to bf16;
// q to q_out [rows, heads head_dim], K / V to pool row slots[r].
void rope_append(const float *qkv, const float *cos_sin, const uint32_t *slots, uint16_t *q_out, uint16_t *k_pool,
                 uint16_t *v_pool, uint64_t rows, uint32_t heads, uint32_t kv_heads, uint32_t head_dim, uint64_t pool_rows,
                 hipStream_t s);

}  // namespace k
}  // namespace fa
