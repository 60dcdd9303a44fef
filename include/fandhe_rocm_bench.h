/*
 * fandhe_rocm_bench.h - measurement and test aids of libfandhe_rocm.so.
 *
 * Nothing in this header stands behind an interface of the reference; a
 * BackendOps / MemoryOps binding needs fandhe_rocm.h only.  These entry points
 * exist for the benchmark (synthetic data, event timers, a matrix-rate probe),
 * for experiments (launch-shape knobs) and for tests that have to know which
 * kernel a shape reaches or which device blocks a captured graph owns.
 */
#ifndef FANDHE_ROCM_BENCH_H
#define FANDHE_ROCM_BENCH_H

#include "fandhe_rocm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Synthetic data: fills an f32 or bf16 buffer with N(mean, std) values from a
 * counter-based generator (value i depends only on seed and i).  For
 * benchmarks that need tens of GB of resident inputs. */
fa_status fa_fill_normal(fa_context *ctx, fa_buffer *buf, uint64_t offset, uint64_t numel,
                         uint64_t seed, float mean, float std);

/* Queues a loop of one matrix instruction kind with operands held in registers
 * (kind 0: v_mfma_i32_16x16x64_i8, 1: v_mfma_i32_32x32x32_i8, 2: the scaled
 * 16x16x128 e4m3 form).  The operand bits are taken from `operands` (64 KiB of
 * any element type): the sustained rate of the matrix cores depends on them.
 * *ops receives the multiply-add operations x 2 of the launch; time it with an
 * fa_timer. */
fa_status fa_probe_matrix_rate(fa_context *ctx, int32_t kind, const fa_buffer *operands,
                               uint32_t iters, fa_buffer *sink, double *ops);

/* Queues a streaming read of `bytes` starting `offset_bytes` into `src`: `blocks` blocks of `threads`
 * (256 or 512) threads, each reading its own contiguous share with 16-byte loads, eight per thread in
 * flight, nothing written; the loads are the non-temporal ones the kernels use for read-once data unless
 * tuning key 15 asks for ordinary loads.  The time of this launch is the floor for a memory-bound kernel
 * that must fetch that many bytes; time it with an fa_timer. */
fa_status fa_probe_stream_read(fa_context *ctx, const fa_buffer *src, uint64_t offset_bytes, uint64_t bytes,
                               int32_t blocks, int32_t threads, fa_buffer *sink);

/* Queues the probe of the path from L2 to the compute units: `blocks` blocks of `threads` threads (64 .. 512, a
 * multiple of 64).  cold_bytes > 0: every block streams its own share of cold_bytes starting cold_offset_bytes into
 * `cold` with non-temporal 16-byte loads, in_flight (8 or 16) per thread, and with every one of them hot_per_cold
 * (0 or 2) ordinary loads of the first hot_bytes of `hot`, a region all blocks share (L2 hits).  cold_bytes == 0:
 * every block reads the hot region alone hot_passes times, in_flight loads per thread in flight.  Nothing is
 * written; time the launch with an fa_timer. */
fa_status fa_probe_l2_path(fa_context *ctx, const fa_buffer *cold, uint64_t cold_offset_bytes, uint64_t cold_bytes,
                           const fa_buffer *hot, uint32_t hot_bytes, uint32_t hot_passes, int32_t in_flight,
                           int32_t hot_per_cold, int32_t blocks, int32_t threads, fa_buffer *sink);

/* Launch-shape knobs for experiments; value 0 restores the built-in choice.
 * The knobs are plain process-wide integers read by every context's launches:
 * set them while no other thread is submitting work.
 * key 0: n-tiles per block of the decode-shape linears (1 or 2);
 * key 1: wavefronts per block of the decode-shape linears (4 or 8);
 * key 2: wavefronts per compute unit of the decode attention (1 .. 8);
 * key 3: nonzero launches only the streaming kernel of the decode attention and
 *        leaves the output unwritten (for timing that kernel by itself);
 * key 4: nonzero keeps the 128 x 128 block tile of the prefill GEMMs for every shape;
 * key 5: activation-stationary decode linears: 1 never, 2 whenever the shape allows, 3 by shape but 33 to 64 rows stay
 *        on the block-per-tile kernels;
 * key 6: wavefronts per block of the large-tile prefill GEMMs (4 or 16; default 8);
 * key 7: column tiles of 16 per block of the large-tile prefill GEMMs (14 or 16);
 * key 8: nonzero sends attention with more than one new token per row to the generic
 *        kernel (the reference's summation order) instead of the streamed one;
 * key 9: blocks per compute unit that a split-k launch of the 128 x 128 int8 GEMM aims
 *        for (default 2);
 * key 10: form of the attention with more than one new token per row: 1 always the
 *        streamed form, 2 always the block form, 0 by shape;
 * key 11: wavefronts per block of that block form (4 or 8; 0 by shape);
 * key 12: upper bound of the blocks that share the cache walk of one tile of new tokens
 *        in the block form (1: never split; 0 by shape);
 * key 13: kernel of the order-fixed f32 GEMM (gemm_device / linear_forward_device): 1 the few-rows vector
 *        kernel, 2 the matrix-core kernel, 0 by shape;
 * key 14: weights that the row kernels of the decode step pull into L2 for the projection that follows them: 1 none,
 *        n >= 2: n MiB of q | k | v and 2 n MiB of the o projection (0: 12 / 24); takes effect when a step is
 *        recorded, so set it before the first step of a batch size;
 * key 15: loads of fa_probe_stream_read: 1 ordinary loads, 0 the non-temporal loads that the kernels use for
 *        data they read once;
 * key 16: split-k form of the decode-shape linears (groups of blocks that share an XCD divide k and add their
 *        partial tiles through a workspace): 0 by shape, 1 never, 2 whenever the shape allows it with the partial
 *        tiles meeting in memory (agent-scope accesses), 3 whenever the shape allows it with the partial tiles
 *        meeting in the XCD's L2, 4 by shape but meeting in memory;
 * key 17: blocks per group of that form: 0 by shape, 2 or 4;
 * key 18: 1 keeps the 256-thread form of the row kernels (norm, quantizer, norm + quantizer) for every row count
 *        instead of the up-to-1024-thread form used for at most 256 rows;
 * key 19: 1 keeps the norm + quantizer and quantizer kernels of a decode step as launches of their own for every batch
 *        size; 0: the linears that follow do that row work themselves where that measured faster (norm + quantizer: one
 *        or two rows, quantizer from partial maxima: one row); 2: wherever the kernels can (four / two rows); takes
 *        effect when a step is recorded;
 * key 20: 1 keeps the streamed attention with its merge launch for every decode step; 0: a step whose contexts are
 *        at most 1024 tokens runs the attention as one launch (a block per sequence and kv head) while there is at
 *        most one such block per compute unit (with one or two sequences the o projection then does the quantizer);
 *        2: whenever the contexts are that short (takes effect when a step is recorded);
 * key 21: the int8 linears of 65 to a few hundred rows (fa_linear_w8a8, prompt passes of the decoder): 0 the
 *        weight-stationary kernel where the shape rule picks it (a weight with at most about two column tiles per
 *        compute unit, m x k at most 2 MiB; k of 8192 .. 14336: the form that splits k over four blocks of an XCD,
 *        up to 512 rows) and the decode kernels for prompt passes of at most 64 rows, 1 the tiled GEMMs always, 2 the
 *        weight-stationary kernel without the split whenever it can run, 3 the split form whenever it can run;
 * key 22: prompt passes on the large-tile GEMM, bits: 1 keeps SwiGLU out of the epilogue of the gate | up GEMM (the plain
 *        GEMM into [rows, 2 d_ffn] and the SwiGLU pass of the row quantizer), 2 keeps RoPE, the bf16 rounding and the K / V
 *        append out of the epilogue of the q | k | v GEMM (the plain GEMM and the RoPE + append pass); 0: both in the
 *        epilogues;
 * key 23: columns (new token x head) per wavefront of the block form of the prefill attention: 0 by shape (16 while
 *        blocks of 32 would not fill the device more than once, else 32), 1: 16 whenever the form allows, 2: 32;
 * key 24: the large-tile int8 GEMM on 256 x 128 tiles: 0: when those tiles cover at most half the device, two or four
 *        same-XCD blocks share a tile, a part of k each; 1: one block per tile; 2: shared tiles only where the tiles
 *        alone cover half the device (pairs);
 * key 25: rows (sequences x tokens) per chunk of a prompt pass, from 256 up; anything smaller: the built-in 8192;
 * key 26: prompt passes of at most 64 rows: 0: q | k | v and gate | up on the decode step's fused kernels (RoPE and the
 *        K / V append, SwiGLU, in the epilogues), 1: plain projections and separate passes;
 * key 27: prompt passes whose q | k | v projection runs on the weight-stationary kernel: 0: RoPE, the bf16 rounding and
 *        the K / V append in that kernel's epilogue, 1: a pass of their own behind it. */
fa_status fa_set_tuning(int32_t key, int32_t value);

/* What the context found when it was created: xcd_local = 1 when workgroups b and b + 8 of a launch were seen to
 * run on the same XCD (the split-k linears then let their partial tiles meet in that XCD's L2), xcd_count = the
 * number of distinct XCDs the probe launch saw. */
fa_status fa_topology_query(const fa_context *ctx, int32_t *xcd_local, int32_t *xcd_count);

/* Which kernel a prefill-shape GEMM of m rows against `qw` is launched with under the
 * current knobs (pure host function, nothing is queued).  big_ntb: column tiles of 16
 * per block of the large-tile kernel (gemm_mfma_big_kernel), 0 when the 128 x 128 kernel
 * (gemm_mfma_kernel) is used; waves: wavefronts per block; splits: blocks that share the
 * k range of one output tile (1: no split). */
typedef struct {
    int32_t big_ntb, waves;
    uint32_t splits;
} fa_gemm_plan;
fa_status fa_gemm_plan_query(const fa_context *ctx, uint64_t m, const fa_qweight *qw, fa_gemm_plan *out);

/* Which kernel fa_gemm_device / fa_linear_forward_device launch for an m x k by k x n product under the current
 * knobs: 1 the few-rows vector kernel (gemm_f32_rows_kernel), 2 the matrix-core kernel (gemm_f32_mfma_kernel). */
fa_status fa_gemm_f32_form_query(uint64_t m, uint64_t n, uint64_t k, int32_t *form);

/* Device blocks a captured graph owns (scratch that calls recorded into it took while the
 * capture was open; they return to the pool when the graph is destroyed).  Writes up to
 * `capacity` device addresses and the total count. */
fa_status fa_graph_owned_blocks(const fa_graph *graph, void **ptrs, uint64_t capacity, uint64_t *count);

/* Test aids for the decode step: run the step's launches, eagerly, up to and including stage `stop_after` and
 * stop, so that a test can read what each fused stage left behind and hold it against the matching operator of
 * the oracle.  Stage 0: per-step bookkeeping (positions, slots, cos / sin, lengths + 1) and the embedding
 * gather; stage 1 + 8 * layer + i, i = 0 .. 7: norm + quantizer, qkv projection with RoPE and cache append,
 * attention with merge + quantizer, o projection (+ residual), norm + quantizer, gate / up with SwiGLU,
 * quantizer, down projection (+ residual); then the final norm + quantizer, the head, the pick.  The sequence
 * lengths advance as in a step: reinstall the sequences before the next call.
 * fa_decoder_debug_buffer hands out the decoder's own resident buffers (not copies; do not free):
 * 0 residual stream h f32 [batch, d_model]; 1 activation codes int8 in tile order (tiles [row tile][k tile] of
 * 16 rows x 64 k, byte ((g * 16 + r) * 16 + j) = row r, k 16 g + j); 2 row scales f32; 3 q bf16 [batch, heads *
 * head_dim]; 4 SwiGLU activation f32 [batch, d_ffn]; 5 partial row maxima f32; 6 logits f32; 7 cos / sin f32
 * [batch, head_dim]; 8 cache slots u32 [batch]; 9 positions i32 [batch]. */
fa_status fa_decoder_debug_step_until(fa_context *ctx, fa_decoder *dec, int32_t stop_after);
fa_status fa_decoder_debug_buffer(fa_decoder *dec, int32_t which, fa_buffer **out);

/* A pair of HIP events recorded on the context's stream (the stream the
 * kernels run on); used by the benchmark to time launches. */
typedef struct fa_timer fa_timer;
fa_status fa_timer_create(fa_context *ctx, fa_timer **out);
fa_status fa_timer_start(fa_context *ctx, fa_timer *t);
fa_status fa_timer_stop(fa_context *ctx, fa_timer *t);
/* Blocks until the stop event has completed. */
fa_status fa_timer_elapsed_ms(fa_context *ctx, fa_timer *t, float *ms);
fa_status fa_timer_destroy(fa_context *ctx, fa_timer *t);

#ifdef __cplusplus
}
#endif
#endif
