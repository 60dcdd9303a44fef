// Internal runtime of the MI355X backend: context, stream, size-class pool,
// buffer handles, error reporting.  Everything above this header is the C ABI
// (include/fandhe_rocm.h); everything below is HIP.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "../../include/fandhe_rocm.h"
#include "../../include/fandhe_rocm_bench.h"
#include "kernels.hpp"

namespace fa {

// ------------------------------------------------------------------ errors
void set_error(const std::string &msg);
fa_status fail(fa_status s, const std::string &msg);

// ------------------------------------------------------------- size classes
// Size-class table of the reference pool (crates/tensor-core/src/pool_core.rs:102-209).
struct PoolConfig {
    uint64_t max_pool_bytes = 128ull << 20;
    uint64_t small_max_bytes = 1ull << 20;
    uint64_t large_granule_bytes = 2ull << 20;
    uint64_t huge_min_bytes = 64ull << 20;
    size_t huge_entries_per_class = 1;
};
bool size_class_for(uint64_t bytes, const PoolConfig &cfg, uint64_t *out);

// Free list of device blocks keyed by class size, insertion-ordered so that
// eviction is global LRU (pool_core.rs:211-590).  The pool never calls HIP
// itself: evicted blocks are handed back to the caller, which frees them
// after the lock is released.
class SizeClassPool {
  public:
    explicit SizeClassPool(PoolConfig cfg = PoolConfig()) : cfg_(cfg) {}
    const PoolConfig &config() const { return cfg_; }
    void *take(uint64_t class_bytes);
    void record_allocation(uint64_t logical, uint64_t cls);
    void record_reuse(uint64_t logical, uint64_t cls);
    void record_loan_end(uint64_t logical, uint64_t cls);
    std::vector<std::pair<uint64_t, void *>> put(uint64_t class_bytes, void *ptr);
    bool take_one_for_release(std::pair<uint64_t, void *> *out);
    void record_release(uint64_t class_bytes);
    fa_pool_stats stats();

  private:
    PoolConfig cfg_;
    std::mutex mu_;
    std::vector<std::pair<uint64_t, void *>> free_;
    uint64_t alloc_count_ = 0, reuse_count_ = 0, cached_bytes_ = 0, waste_ = 0, released_ = 0;
};

size_t dtype_size(fa_dtype t);

}  // namespace fa

// a pool block on loan: device address, logical size, size class
struct fa_owned_block {
    void *ptr;
    uint64_t bytes, cls;
};

struct fa_context {
    uint32_t magic;
    int device;
    hipStream_t stream;
    fa::SizeClassPool pool;
    bool poisoned;
    bool capturing;
    hipDeviceProp_t props;
    // device staging for per-call host tables (slot mappings, block tables)
    void *table_stage;
    uint64_t table_stage_bytes;
    // scratch for split-KV attention partials and similar kernel workspaces
    void *workspace;
    uint64_t workspace_bytes;
    // workspaces that were outgrown: captured graphs may still hold their addresses, so they stay
    // allocated until the context is destroyed (growth is geometric, the total stays below twice the last)
    std::vector<void *> retired_workspaces;
    // Scratch that calls recorded into the open capture took: the recorded kernels hold these addresses, so
    // the blocks belong to the graph (moved into it when the capture ends) instead of going back to the pool.
    std::vector<fa_owned_block> capture_owned;
    // blocks the pool evicted while a capture was open: released to the driver when the capture ends
    std::vector<void *> deferred_frees;
    // class bytes of the blocks on loan to an open capture or to live graphs (PoolStats::pending_return_bytes:
    // idle-side memory that is neither cached nor in use by a buffer and comes back when its holder ends)
    uint64_t pending_return_bytes = 0;
    // where the blocks of a split-k decode linear meet (allocated with the context, outside the pool; the counters
    // are zero whenever no such launch is running)
    fa::k::SplitKArea splitk;
    int xcd_count = 0;            // distinct XCDs seen by the probe launch at creation
    // graphs recorded on this context that are still alive; a context is not destroyed while one of them holds
    // device blocks of its pool
    uint64_t live_graphs = 0;
};

struct fa_buffer {
    uint32_t magic;
    fa_context *ctx;
    void *ptr;
    uint64_t numel;
    fa_dtype dtype;
    uint64_t logical_bytes;
    uint64_t class_bytes;
};

struct fa_qweight {
    uint32_t magic;
    fa_context *ctx;
    fa_qweight_kind kind;
    uint64_t k, n;          // logical shape [k, n]
    uint64_t k_pad, n_pad;  // padded to the tile grid
    fa_buffer *codes;       // tile-ordered codes, k_pad * n_pad bytes
    fa_buffer *scales;      // f32: n_pad (int8) or 1 (e4m3)
};

struct fa_graph {
    uint32_t magic;
    fa_context *ctx;          // the context whose stream recorded it: the only one that may replay or destroy it
    hipGraph_t graph;
    hipGraphExec_t exec;
    // device blocks whose addresses the recorded kernels hold; returned to the pool when the graph is destroyed
    std::vector<fa_owned_block> owned;
};

struct fa_timer {
    hipEvent_t start, stop;
};

namespace fa {

constexpr uint32_t kCtxMagic = 0xFA0C7C01u;
constexpr uint32_t kBufMagic = 0xFA0B0F01u;
constexpr uint32_t kQwMagic = 0xFA0A0E01u;
constexpr uint32_t kGraphMagic = 0xFA06A901u;

// Common entry checks; each returns FA_OK or records the error.
fa_status check_ctx(const fa_context *ctx);
fa_status check_buf(const fa_context *ctx, const fa_buffer *b, const char *what);
fa_status check_buf_typed(const fa_context *ctx, const fa_buffer *b, fa_dtype t, uint64_t min_numel,
                          const char *what);
fa_status hip_fail(fa_context *ctx, hipError_t e, const char *what, fa_status as);
// Checks hipGetLastError after a launch.
fa_status after_launch(fa_context *ctx, const char *kernel);

// Pool-backed raw allocation used by buffers and by internal scratch.
fa_status pool_alloc(fa_context *ctx, uint64_t bytes, void **ptr, uint64_t *class_bytes);
void pool_free(fa_context *ctx, void *ptr, uint64_t logical, uint64_t class_bytes);
// End of a loan taken for the duration of one call (kernel scratch).  Outside a capture the block goes back
// to the pool (the stream is in order, so the next user is queued behind this call's kernels).  While a
// capture is open the recorded kernels keep the address for every replay: the block is handed to the graph.
void scratch_release(fa_context *ctx, void *ptr, uint64_t logical, uint64_t class_bytes);
fa_status make_buffer(fa_context *ctx, fa_dtype dtype, uint64_t numel, bool zero, fa_buffer **out);
// Ensures ctx->workspace holds at least `bytes` (grows outside capture only).
fa_status ensure_workspace(fa_context *ctx, uint64_t bytes);
fa_status ensure_table_stage(fa_context *ctx, uint64_t bytes);
// Resolves the device address of the static scratch of fa_paged_attention_decode_static on `device`, which
// must be current; once per device.
void static_scratch_init(int device);

}  // namespace fa
