// Context, stream, memory pool, transfers, graph capture and timers.
#include "runtime.hpp"

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <exception>
#include <new>

namespace fa {

static thread_local std::string g_last_error;

void set_error(const std::string &msg) { g_last_error = msg; }
fa_status fail(fa_status s, const std::string &msg) {
    g_last_error = msg;
    return s;
}

size_t dtype_size(fa_dtype t) {
    switch (t) {
        case FA_F32: return 4;
        case FA_BF16: return 2;
        case FA_I8: return 1;
        case FA_E4M3: return 1;
        case FA_I32: return 4;
        case FA_U32: return 4;
    }
    return 0;
}

// crates/tensor-core/src/pool_core.rs:157-209
bool size_class_for(uint64_t bytes, const PoolConfig &cfg, uint64_t *out) {
    if (bytes == 0) { *out = 0; return true; }
    if (bytes >= cfg.huge_min_bytes) { *out = bytes; return true; }
    if (bytes > cfg.small_max_bytes) {
        uint64_t granule = std::max<uint64_t>(cfg.large_granule_bytes, 1);
        uint64_t padded;
        if (__builtin_add_overflow(bytes, granule - 1, &padded)) return false;
        return !__builtin_mul_overflow(padded / granule, granule, out);
    }
    if (bytes <= 255) { *out = 256; return true; }
    int octave = 63 - __builtin_clzll(bytes);
    uint64_t base = 1ull << octave, step = base / 4;
    for (uint64_t mult = 0; mult < 4; ++mult) {
        uint64_t cls = base + step * mult;
        if (cls >= bytes) { *out = cls; return true; }
    }
    return !__builtin_mul_overflow(base, (uint64_t)2, out);
}

// ------------------------------------------------------------------- pool
void *SizeClassPool::take(uint64_t class_bytes) {
    std::lock_guard<std::mutex> g(mu_);
    for (size_t i = 0; i < free_.size(); ++i) {
        if (free_[i].first == class_bytes) {
            void *p = free_[i].second;
            free_.erase(free_.begin() + (long)i);
            cached_bytes_ -= std::min(cached_bytes_, class_bytes);
            return p;
        }
    }
    return nullptr;
}
void SizeClassPool::record_allocation(uint64_t logical, uint64_t cls) {
    std::lock_guard<std::mutex> g(mu_);
    ++alloc_count_;
    waste_ += cls > logical ? cls - logical : 0;
}
void SizeClassPool::record_reuse(uint64_t logical, uint64_t cls) {
    std::lock_guard<std::mutex> g(mu_);
    ++reuse_count_;
    waste_ += cls > logical ? cls - logical : 0;
}
void SizeClassPool::record_loan_end(uint64_t logical, uint64_t cls) {
    std::lock_guard<std::mutex> g(mu_);
    uint64_t w = cls > logical ? cls - logical : 0;
    waste_ -= std::min(waste_, w);
}
std::vector<std::pair<uint64_t, void *>> SizeClassPool::put(uint64_t class_bytes, void *ptr) {
    std::lock_guard<std::mutex> g(mu_);
    std::vector<std::pair<uint64_t, void *>> evicted;
    free_.emplace_back(class_bytes, ptr);
    cached_bytes_ += class_bytes;
    if (class_bytes >= cfg_.huge_min_bytes) {       // per-class cap of the huge band
        for (;;) {
            size_t count = 0, first = free_.size();
            for (size_t i = 0; i < free_.size(); ++i)
                if (free_[i].first == class_bytes) {
                    if (first == free_.size()) first = i;
                    ++count;
                }
            if (count <= cfg_.huge_entries_per_class || first == free_.size()) break;
            evicted.push_back(free_[first]);
            cached_bytes_ -= std::min(cached_bytes_, free_[first].first);
            free_.erase(free_.begin() + (long)first);
        }
    }
    while (cached_bytes_ > cfg_.max_pool_bytes && !free_.empty()) {   // global LRU
        evicted.push_back(free_.front());
        cached_bytes_ -= std::min(cached_bytes_, free_.front().first);
        free_.erase(free_.begin());
    }
    return evicted;
}
bool SizeClassPool::take_one_for_release(std::pair<uint64_t, void *> *out) {
    std::lock_guard<std::mutex> g(mu_);
    if (free_.empty()) return false;
    *out = free_.back();
    free_.pop_back();
    cached_bytes_ -= std::min(cached_bytes_, out->first);
    return true;
}
void SizeClassPool::record_release(uint64_t class_bytes) {
    std::lock_guard<std::mutex> g(mu_);
    released_ += class_bytes;
}
fa_pool_stats SizeClassPool::stats() {
    std::lock_guard<std::mutex> g(mu_);
    fa_pool_stats s;
    s.alloc_count = alloc_count_;
    s.reuse_count = reuse_count_;
    s.cached_bytes = cached_bytes_;
    s.pending_return_bytes = 0;
    s.capacity_waste_bytes = waste_;
    s.released_bytes = released_;
    return s;
}

// ----------------------------------------------------------------- checks
fa_status check_ctx(const fa_context *ctx) {
    if (!ctx || ctx->magic != kCtxMagic) return fail(FA_ERR_INVALID_ARGUMENT, "context: null or not a context");
    if (ctx->poisoned) return fail(FA_ERR_CONTEXT_POISONED, "context: poisoned by an earlier device failure");
    // a split-k linear found the blocks of a group on different XCDs although the probe at creation said they share
    // one: its partial tiles met through two L2s and what it wrote cannot be trusted
    if (ctx->splitk.fault && *(volatile uint32_t *)ctx->splitk.fault != 0)
        return fail(FA_ERR_CONTEXT_POISONED, "context: a split-k linear ran its groups across XCDs (results invalid); "
                                             "recreate the context, or set tuning key 16 to 4 to let partial tiles meet in memory");
    return FA_OK;
}
fa_status check_buf(const fa_context *ctx, const fa_buffer *b, const char *what) {
    if (!b || b->magic != kBufMagic) return fail(FA_ERR_INVALID_ARGUMENT, std::string(what) + ": null or not a buffer");
    if (b->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, std::string(what) + ": buffer belongs to another context");
    return FA_OK;
}
fa_status check_buf_typed(const fa_context *ctx, const fa_buffer *b, fa_dtype t, uint64_t min_numel,
                          const char *what) {
    if (fa_status s = check_buf(ctx, b, what)) return s;
    if (b->dtype != t) return fail(FA_ERR_INVALID_ARGUMENT, std::string(what) + ": wrong element type");
    if (b->numel < min_numel)
        return fail(FA_ERR_SHAPE_MISMATCH, std::string(what) + ": buffer holds " + std::to_string(b->numel) +
                                               " elements, needs " + std::to_string(min_numel));
    return FA_OK;
}
fa_status hip_fail(fa_context *ctx, hipError_t e, const char *what, fa_status as) {
    if (ctx && as != FA_ERR_ALLOCATION_FAILED) ctx->poisoned = true;
    return fail(as, std::string(what) + ": " + hipGetErrorString(e));
}
fa_status after_launch(fa_context *ctx, const char *kernel) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(ctx, e, kernel, FA_ERR_KERNEL_LAUNCH_FAILED);
    return FA_OK;
}

// ------------------------------------------------------------- allocation
fa_status pool_alloc(fa_context *ctx, uint64_t bytes, void **ptr, uint64_t *class_bytes) {
    uint64_t cls;
    if (!size_class_for(bytes, ctx->pool.config(), &cls))
        return fail(FA_ERR_ALLOCATION_FAILED, "size class rounding overflowed");
    void *p = ctx->pool.take(cls);
    if (p) {
        ctx->pool.record_reuse(bytes, cls);
    } else if (ctx->capturing) {
        // Scratch of a call that is being recorded (buffers cannot be created during a capture: the entry
        // points that make them return FA_ERR_CAPTURE_IN_PROGRESS first).  The capture is thread-local, which
        // forbids allocation calls on this thread; the relaxed mode lifts that for the one call.  Nothing
        // is released to make room here (hipFree is not allowed either).
        hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
        hipError_t e = hipThreadExchangeStreamCaptureMode(&mode);
        if (e == hipSuccess) {
            e = hipMalloc(&p, cls);
            hipError_t back = hipThreadExchangeStreamCaptureMode(&mode);
            if (e == hipSuccess && back != hipSuccess) {
                (void)hipFree(p);
                e = back;
            }
        }
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return fail(FA_ERR_CAPTURE_IN_PROGRESS,
                        std::string("scratch allocation during graph capture failed: ") + hipGetErrorString(e));
        }
        ctx->pool.record_allocation(bytes, cls);
    } else {
        hipError_t e = hipMalloc(&p, cls);
        if (e != hipSuccess) {
            // give cached blocks back to the driver once, then retry
            std::pair<uint64_t, void *> ent;
            while (ctx->pool.take_one_for_release(&ent)) {
                if (hipFree(ent.second) == hipSuccess) ctx->pool.record_release(ent.first);
            }
            (void)hipGetLastError();
            e = hipMalloc(&p, cls);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                return hip_fail(ctx, e, "hipMalloc", FA_ERR_ALLOCATION_FAILED);
            }
        }
        ctx->pool.record_allocation(bytes, cls);
    }
    *ptr = p;
    *class_bytes = cls;
    return FA_OK;
}

void pool_free(fa_context *ctx, void *ptr, uint64_t logical, uint64_t class_bytes) {
    if (!ptr) return;
    ctx->pool.record_loan_end(logical, class_bytes);
    auto evicted = ctx->pool.put(class_bytes, ptr);
    for (auto &e : evicted) {
        if (ctx->capturing) {
            // no hipFree while this thread records a capture: released when the capture ends
            try {
                ctx->deferred_frees.push_back(e.second);
            } catch (const std::exception &) {
                // out of host memory for the list: the block stays allocated until the process ends
            }
            continue;
        }
        // hipFree waits for the device, so work still queued on the stream is safe
        if (hipFree(e.second) != hipSuccess) (void)hipGetLastError();
    }
}

void scratch_release(fa_context *ctx, void *ptr, uint64_t logical, uint64_t class_bytes) {
    if (!ptr) return;
    if (ctx->capturing) {
        try {
            ctx->capture_owned.push_back(fa_owned_block{ptr, logical, class_bytes});
            ctx->pending_return_bytes += class_bytes;
            return;
        } catch (const std::exception &) {
            // cannot track it: leak the block rather than let the pool hand it to someone else
            return;
        }
    }
    pool_free(ctx, ptr, logical, class_bytes);
}

fa_status make_buffer(fa_context *ctx, fa_dtype dtype, uint64_t numel, bool zero, fa_buffer **out) {
    size_t esz = dtype_size(dtype);
    if (esz == 0) return fail(FA_ERR_INVALID_ARGUMENT, "unknown element type");
    uint64_t bytes;
    if (__builtin_mul_overflow(numel, (uint64_t)esz, &bytes))
        return fail(FA_ERR_ALLOCATION_FAILED, "buffer size overflows 64 bits");
    fa_buffer *b = new (std::nothrow) fa_buffer();
    if (!b) return fail(FA_ERR_ALLOCATION_FAILED, "host allocation of the handle failed");
    b->magic = kBufMagic;
    b->ctx = ctx;
    b->ptr = nullptr;
    b->numel = numel;
    b->dtype = dtype;
    b->logical_bytes = bytes;
    b->class_bytes = 0;
    if (bytes != 0 && ctx->capturing) {
        // a buffer outlives the call that makes it, and zeroing it would record a memset node
        delete b;
        return fail(FA_ERR_CAPTURE_IN_PROGRESS, "buffer allocation during graph capture");
    }
    if (bytes != 0) {     // numel == 0 never touches the device (buffer.rs:50-59)
        fa_status s = pool_alloc(ctx, bytes, &b->ptr, &b->class_bytes);
        if (s != FA_OK) {
            delete b;
            return s;
        }
        if (zero) {
            hipError_t e = hipMemsetAsync(b->ptr, 0, bytes, ctx->stream);
            if (e != hipSuccess) {
                pool_free(ctx, b->ptr, bytes, b->class_bytes);
                delete b;
                return hip_fail(ctx, e, "hipMemsetAsync", FA_ERR_ALLOCATION_FAILED);
            }
        }
    }
    *out = b;
    return FA_OK;
}

fa_status ensure_workspace(fa_context *ctx, uint64_t bytes) {
    if (ctx->workspace_bytes >= bytes) return FA_OK;
    if (ctx->capturing)
        return fail(FA_ERR_CAPTURE_IN_PROGRESS, "workspace must be sized before graph capture");
    uint64_t want = std::max<uint64_t>(std::max<uint64_t>(bytes, 2 * ctx->workspace_bytes), 1ull << 20);
    if (ctx->workspace) {
        try {
            ctx->retired_workspaces.reserve(ctx->retired_workspaces.size() + 1);
        } catch (const std::exception &) {
            return fail(FA_ERR_ALLOCATION_FAILED, "workspace: out of host memory");
        }
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, want);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return hip_fail(ctx, e, "hipMalloc(workspace)", FA_ERR_ALLOCATION_FAILED);
    }
    if (ctx->workspace) ctx->retired_workspaces.push_back(ctx->workspace);   // a captured graph may replay with it
    ctx->workspace = p;
    ctx->workspace_bytes = want;
    return FA_OK;
}

fa_status ensure_table_stage(fa_context *ctx, uint64_t bytes) {
    if (ctx->table_stage_bytes >= bytes) return FA_OK;
    if (ctx->capturing)
        return fail(FA_ERR_CAPTURE_IN_PROGRESS, "host tables cannot be staged during graph capture");
    uint64_t want = std::max<uint64_t>(bytes, 1ull << 16);
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, want);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return hip_fail(ctx, e, "hipMalloc(table stage)", FA_ERR_ALLOCATION_FAILED);
    }
    if (ctx->table_stage) (void)hipFree(ctx->table_stage);
    ctx->table_stage = p;
    ctx->table_stage_bytes = want;
    return FA_OK;
}

}  // namespace fa

using namespace fa;

// =================================================================== C ABI
extern "C" {

const char *fa_last_error_message(void) { return g_last_error.c_str(); }

const char *fa_status_name(fa_status s) {
    switch (s) {
        case FA_OK: return "Ok";
        case FA_ERR_INVALID_ARGUMENT: return "InvalidArgument";
        case FA_ERR_SHAPE_MISMATCH: return "ShapeMismatch";
        case FA_ERR_DEVICE_MISMATCH: return "DeviceMismatch";
        case FA_ERR_ALLOCATION_FAILED: return "DeviceAllocationFailed";
        case FA_ERR_KERNEL_LAUNCH_FAILED: return "KernelLaunchFailed";
        case FA_ERR_DEVICE_UNAVAILABLE: return "DeviceUnavailable";
        case FA_ERR_TRANSFER_FAILED: return "TransferFailed";
        case FA_ERR_UNSUPPORTED: return "Unsupported";
        case FA_ERR_CONTEXT_POISONED: return "DeviceContextPoisoned";
        case FA_ERR_CAPTURE_IN_PROGRESS: return "DeviceContextCaptureInProgress";
        case FA_ERR_STORE_POISONED: return "StorePoisoned";
    }
    return "Unknown";
}

uint32_t fa_abi_version(void) { return 1; }

static bool is_gfx950(const hipDeviceProp_t &p) { return std::strncmp(p.gcnArchName, "gfx950", 6) == 0; }

fa_status fa_device_count(int32_t *count) {
    if (!count) return fail(FA_ERR_INVALID_ARGUMENT, "fa_device_count: null output");
    *count = 0;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(FA_ERR_DEVICE_UNAVAILABLE, std::string("hipGetDeviceCount: ") + hipGetErrorString(e));
    }
    int ok = 0;
    for (int i = 0; i < n; ++i) {
        hipDeviceProp_t p;
        if (hipGetDeviceProperties(&p, i) == hipSuccess && is_gfx950(p)) ++ok;
    }
    *count = ok;
    return FA_OK;
}

fa_status fa_context_create(int32_t ordinal, fa_context **out) {
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "fa_context_create: null output");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return fail(FA_ERR_DEVICE_UNAVAILABLE, "no HIP device is visible");
    }
    if (ordinal < 0 || ordinal >= n)
        return fail(FA_ERR_DEVICE_UNAVAILABLE, "device ordinal " + std::to_string(ordinal) + " does not exist");
    hipDeviceProp_t p;
    e = hipGetDeviceProperties(&p, ordinal);
    if (e != hipSuccess) return fail(FA_ERR_DEVICE_UNAVAILABLE, std::string("hipGetDeviceProperties: ") + hipGetErrorString(e));
    if (!is_gfx950(p))
        return fail(FA_ERR_DEVICE_UNAVAILABLE, std::string("device is ") + p.gcnArchName + ", this backend is built for gfx950 only");
    e = hipSetDevice(ordinal);
    if (e != hipSuccess) return fail(FA_ERR_DEVICE_UNAVAILABLE, std::string("hipSetDevice: ") + hipGetErrorString(e));
    fa_context *ctx = new (std::nothrow) fa_context();
    if (!ctx) return fail(FA_ERR_ALLOCATION_FAILED, "host allocation of the context failed");
    ctx->magic = kCtxMagic;
    ctx->device = ordinal;
    ctx->poisoned = false;
    ctx->capturing = false;
    ctx->props = p;
    ctx->table_stage = nullptr;
    ctx->table_stage_bytes = 0;
    ctx->workspace = nullptr;
    ctx->workspace_bytes = 0;
    static_scratch_init(ordinal);
    e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete ctx;
        return fail(FA_ERR_DEVICE_UNAVAILABLE, std::string("hipStreamCreate: ") + hipGetErrorString(e));
    }
    // Meeting area of the split-k decode linears: 16 MiB of partial tiles, 4096 arrival counters.  Whether the
    // workgroups b and b + 8 of a launch share an XCD (and with it an L2) is read off the hardware once: 2048
    // workgroups report the XCD they run on.  Without that property the partial tiles meet in memory instead.
    {
        constexpr uint64_t kPartial = 16ull << 20;
        constexpr uint32_t kCounters = 4096, kProbe = 2048, kXccSeen = 16384;
        void *area = nullptr;
        if (hipMalloc(&area, kPartial + (kCounters + kXccSeen) * 4) == hipSuccess) {
            uint32_t *counters = (uint32_t *)((uint8_t *)area + kPartial);
            std::vector<uint32_t> ids(kProbe, 0xffu);
            fa::k::xcc_id_probe(counters, kProbe, ctx->stream);
            bool ok = hipGetLastError() == hipSuccess &&
                      hipMemcpyAsync(ids.data(), counters, kProbe * 4, hipMemcpyDeviceToHost, ctx->stream) == hipSuccess &&
                      hipStreamSynchronize(ctx->stream) == hipSuccess;
            bool round_robin = ok;
            for (uint32_t b = 0; round_robin && b < kProbe; ++b) round_robin = ids[b] == ids[b % 8];
            for (uint32_t b = 0; round_robin && b < 8; ++b)
                for (uint32_t c = 0; c < b; ++c) round_robin = round_robin && ids[b] != ids[c];
            if (ok) {
                bool seen[16] = {};
                for (uint32_t b = 0; b < kProbe; ++b) seen[ids[b] & 15u] = true;
                for (bool x : seen) ctx->xcd_count += x ? 1 : 0;
            }
            ok = ok && hipMemsetAsync(area, 0, kPartial + (kCounters + kXccSeen) * 4, ctx->stream) == hipSuccess &&
                 hipStreamSynchronize(ctx->stream) == hipSuccess;
            if (ok) {
                ctx->splitk.partial = area;
                ctx->splitk.partial_bytes = kPartial;
                ctx->splitk.counters = counters;
                ctx->splitk.n_counters = kCounters;
                ctx->splitk.xcd_local = round_robin ? 1 : 0;
                // one word per block of a launch (the groups' XCD notes) behind the counters, and the word of pinned
                // host memory a launch reports a split group to
                ctx->splitk.xcc_seen = counters + kCounters;
                ctx->splitk.n_xcc_seen = kXccSeen;
                void *flag = nullptr;
                if (hipHostMalloc(&flag, 64, hipHostMallocMapped) == hipSuccess) {
                    *(volatile uint32_t *)flag = 0;
                    ctx->splitk.fault = (uint32_t *)flag;
                } else {
                    (void)hipGetLastError();
                    ctx->splitk.xcc_seen = nullptr;        // nowhere to report to: no notes
                }
            } else {
                (void)hipGetLastError();
                (void)hipFree(area);                 // the linears then keep to their unsplit forms
            }
        } else {
            (void)hipGetLastError();
        }
    }
    *out = ctx;
    return FA_OK;
}

fa_status fa_topology_query(const fa_context *ctx, int32_t *xcd_local, int32_t *xcd_count) {
    if (!ctx || ctx->magic != kCtxMagic || !xcd_local || !xcd_count)
        return fail(FA_ERR_INVALID_ARGUMENT, "fa_topology_query: bad argument");
    *xcd_local = ctx->splitk.xcd_local;
    *xcd_count = ctx->xcd_count;
    return FA_OK;
}

fa_status fa_context_destroy(fa_context *ctx) {
    if (!ctx || ctx->magic != kCtxMagic) return fail(FA_ERR_INVALID_ARGUMENT, "fa_context_destroy: not a context");
    if (ctx->live_graphs != 0)
        return fail(FA_ERR_INVALID_ARGUMENT, "fa_context_destroy: " + std::to_string(ctx->live_graphs) +
                                                 " graph(s) recorded on this context are still alive; destroy them first");
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    std::pair<uint64_t, void *> ent;
    while (ctx->pool.take_one_for_release(&ent)) (void)hipFree(ent.second);
    if (ctx->table_stage) (void)hipFree(ctx->table_stage);
    if (ctx->workspace) (void)hipFree(ctx->workspace);
    if (ctx->splitk.partial) (void)hipFree(ctx->splitk.partial);
    if (ctx->splitk.fault) (void)hipHostFree(ctx->splitk.fault);
    for (void *w : ctx->retired_workspaces) (void)hipFree(w);
    for (auto &b : ctx->capture_owned) (void)hipFree(b.ptr);   // a capture that was never ended
    for (void *p : ctx->deferred_frees) (void)hipFree(p);
    (void)hipStreamDestroy(ctx->stream);
    (void)hipGetLastError();
    ctx->magic = 0;
    delete ctx;
    return FA_OK;
}

fa_status fa_context_info(const fa_context *ctx, fa_device_info *out) {
    if (!ctx || ctx->magic != kCtxMagic || !out) return fail(FA_ERR_INVALID_ARGUMENT, "fa_context_info: bad argument");
    std::memset(out, 0, sizeof(*out));
    out->ordinal = ctx->device;
    out->compute_units = ctx->props.multiProcessorCount;
    out->clock_khz = ctx->props.clockRate;
    out->wavefront_size = ctx->props.warpSize;
    out->total_memory_bytes = ctx->props.totalGlobalMem;
    std::snprintf(out->arch, sizeof(out->arch), "%s", ctx->props.gcnArchName);
    std::snprintf(out->name, sizeof(out->name), "%s", ctx->props.name);
    return FA_OK;
}

void *fa_context_stream(fa_context *ctx) { return ctx && ctx->magic == kCtxMagic ? (void *)ctx->stream : nullptr; }

// ------------------------------------------------------------------ memory
static fa_status reject_in_capture(fa_context *ctx, const char *what) {
    if (ctx->capturing)
        return fail(FA_ERR_CAPTURE_IN_PROGRESS, std::string(what) + " is not allowed during graph capture");
    return FA_OK;
}

fa_status fa_alloc_zeroed(fa_context *ctx, fa_dtype dtype, uint64_t numel, fa_buffer **out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "fa_alloc_zeroed: null output");
    if (fa_status s = reject_in_capture(ctx, "fa_alloc_zeroed")) return s;
    return make_buffer(ctx, dtype, numel, true, out);
}

fa_status fa_alloc_uninit(fa_context *ctx, fa_dtype dtype, uint64_t numel, fa_buffer **out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "fa_alloc_uninit: null output");
    if (fa_status s = reject_in_capture(ctx, "fa_alloc_uninit")) return s;
    return make_buffer(ctx, dtype, numel, false, out);
}

// Host memory handed to upload is pageable in general; the copy is finished
// (source consumed) before the call returns, as MemoryOps::upload requires.
static fa_status h2d(fa_context *ctx, void *dst, const void *host, uint64_t bytes) {
    if (bytes == 0) return FA_OK;
    hipError_t e = hipMemcpyAsync(dst, host, bytes, hipMemcpyHostToDevice, ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipMemcpyAsync(H2D)", FA_ERR_TRANSFER_FAILED);
    e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamSynchronize(H2D)", FA_ERR_TRANSFER_FAILED);
    return FA_OK;
}

fa_status fa_upload(fa_context *ctx, fa_dtype dtype, const void *host, uint64_t numel, fa_buffer **out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!out || (!host && numel != 0)) return fail(FA_ERR_INVALID_ARGUMENT, "fa_upload: null argument");
    if (fa_status s = reject_in_capture(ctx, "fa_upload")) return s;
    fa_buffer *b = nullptr;
    if (fa_status s = make_buffer(ctx, dtype, numel, false, &b)) return s;
    fa_status s = h2d(ctx, b->ptr, host, b->logical_bytes);
    if (s != FA_OK) {
        pool_free(ctx, b->ptr, b->logical_bytes, b->class_bytes);
        delete b;
        return s;
    }
    *out = b;
    return FA_OK;
}

fa_status fa_upload_into(fa_context *ctx, const void *host, uint64_t numel, fa_buffer *dst, uint64_t dst_offset) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf(ctx, dst, "fa_upload_into: dst")) return s;
    if (fa_status s = reject_in_capture(ctx, "fa_upload_into")) return s;
    uint64_t end;
    if (__builtin_add_overflow(dst_offset, numel, &end) || end > dst->numel)
        return fail(FA_ERR_INVALID_ARGUMENT, "fa_upload_into: range exceeds the destination buffer");
    if (numel == 0) return FA_OK;
    if (!host) return fail(FA_ERR_INVALID_ARGUMENT, "fa_upload_into: null host pointer");
    size_t esz = dtype_size(dst->dtype);
    return h2d(ctx, (char *)dst->ptr + dst_offset * esz, host, numel * esz);
}

fa_status fa_download(fa_context *ctx, const fa_buffer *src, uint64_t src_offset, void *host, uint64_t numel) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf(ctx, src, "fa_download: src")) return s;
    if (fa_status s = reject_in_capture(ctx, "fa_download")) return s;
    uint64_t end;
    if (__builtin_add_overflow(src_offset, numel, &end) || end > src->numel)
        return fail(FA_ERR_INVALID_ARGUMENT, "fa_download: range exceeds the source buffer");
    if (numel != 0 && !host) return fail(FA_ERR_INVALID_ARGUMENT, "fa_download: null host pointer");
    size_t esz = dtype_size(src->dtype);
    if (numel != 0) {
        hipError_t e = hipMemcpyAsync(host, (const char *)src->ptr + src_offset * esz, numel * esz,
                                      hipMemcpyDeviceToHost, ctx->stream);
        if (e != hipSuccess) return hip_fail(ctx, e, "hipMemcpyAsync(D2H)", FA_ERR_TRANSFER_FAILED);
    }
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamSynchronize(D2H)", FA_ERR_TRANSFER_FAILED);
    return FA_OK;
}

fa_status fa_download_owned(fa_context *ctx, fa_buffer *src, void *host, uint64_t numel) {
    fa_status s = fa_download(ctx, src, 0, host, numel);
    // consumed either way; a handle that is not a buffer of this context was reported by the download
    if (src && ctx && ctx->magic == kCtxMagic && src->magic == kBufMagic && src->ctx == ctx) {
        const std::string msg = fa_last_error_message();
        (void)fa_buffer_free(ctx, src);
        if (s != FA_OK) set_error(msg);
    }
    return s;
}

fa_status fa_with_host_view(fa_context *ctx, const fa_buffer *src, fa_host_view_fn f, void *user) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = check_buf(ctx, src, "fa_with_host_view: src")) return s;
    if (!f) return fail(FA_ERR_INVALID_ARGUMENT, "fa_with_host_view: null callback");
    if (src->numel == 0) {
        f(user, nullptr, 0);
        return FA_OK;
    }
    std::vector<unsigned char> host;
    try {
        host.resize(src->logical_bytes);
    } catch (const std::exception &) {
        return fail(FA_ERR_ALLOCATION_FAILED, "fa_with_host_view: out of host memory");
    }
    if (fa_status s = fa_download(ctx, src, 0, host.data(), src->numel)) return s;
    f(user, host.data(), src->numel);
    return FA_OK;
}

fa_status fa_buffer_free(fa_context *ctx, fa_buffer *buf) {
    if (!buf) return FA_OK;
    if (!ctx || ctx->magic != kCtxMagic) return fail(FA_ERR_INVALID_ARGUMENT, "fa_buffer_free: not a context");
    if (buf->magic != kBufMagic) return fail(FA_ERR_INVALID_ARGUMENT, "fa_buffer_free: not a buffer (double free?)");
    if (buf->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, "fa_buffer_free: buffer belongs to another context");
    pool_free(ctx, buf->ptr, buf->logical_bytes, buf->class_bytes);
    buf->magic = 0;
    delete buf;
    return FA_OK;
}

uint64_t fa_buffer_numel(const fa_buffer *b) { return b && b->magic == kBufMagic ? b->numel : 0; }
fa_dtype fa_buffer_dtype(const fa_buffer *b) { return b && b->magic == kBufMagic ? b->dtype : FA_F32; }
void *fa_buffer_device_ptr(const fa_buffer *b) { return b && b->magic == kBufMagic ? b->ptr : nullptr; }

fa_status fa_synchronize_device(fa_context *ctx) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = reject_in_capture(ctx, "fa_synchronize_device")) return s;
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamSynchronize", FA_ERR_KERNEL_LAUNCH_FAILED);
    return FA_OK;
}

fa_status fa_context_poisoned(const fa_context *ctx, int32_t *poisoned) {
    if (!ctx || ctx->magic != kCtxMagic || !poisoned) return fail(FA_ERR_INVALID_ARGUMENT, "fa_context_poisoned: bad argument");
    *poisoned = ctx->poisoned ? 1 : 0;
    return FA_OK;
}

fa_status fa_device_memory_pool_stats(fa_context *ctx, fa_pool_stats *out) {
    if (!ctx || ctx->magic != kCtxMagic || !out) return fail(FA_ERR_INVALID_ARGUMENT, "fa_device_memory_pool_stats: bad argument");
    *out = ctx->pool.stats();
    out->pending_return_bytes = ctx->pending_return_bytes;
    return FA_OK;
}

fa_status fa_release_cached_device_memory(fa_context *ctx) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (fa_status s = reject_in_capture(ctx, "fa_release_cached_device_memory")) return s;
    std::pair<uint64_t, void *> ent;
    while (ctx->pool.take_one_for_release(&ent)) {
        hipError_t e = hipFree(ent.second);
        if (e == hipSuccess) {
            ctx->pool.record_release(ent.first);
        } else {
            (void)hipGetLastError();
            return hip_fail(ctx, e, "hipFree", FA_ERR_KERNEL_LAUNCH_FAILED);
        }
    }
    return FA_OK;
}

fa_status fa_size_class_for(uint64_t bytes, uint64_t *class_bytes) {
    if (!class_bytes) return fail(FA_ERR_INVALID_ARGUMENT, "fa_size_class_for: null output");
    if (!size_class_for(bytes, PoolConfig(), class_bytes))
        return fail(FA_ERR_ALLOCATION_FAILED, "size class rounding overflowed");
    return FA_OK;
}

// ------------------------------------------------------------------ graphs
fa_status fa_graph_capture_begin(fa_context *ctx) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (ctx->capturing) return fail(FA_ERR_CAPTURE_IN_PROGRESS, "a capture is already in progress");
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamBeginCapture", FA_ERR_KERNEL_LAUNCH_FAILED);
    ctx->capturing = true;
    return FA_OK;
}

fa_status fa_graph_capture_end(fa_context *ctx, fa_graph **out) {
    if (!ctx || ctx->magic != kCtxMagic || !out) return fail(FA_ERR_INVALID_ARGUMENT, "fa_graph_capture_end: bad argument");
    if (!ctx->capturing) return fail(FA_ERR_INVALID_ARGUMENT, "no capture in progress");
    ctx->capturing = false;
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &g);
    for (void *p : ctx->deferred_frees)
        if (hipFree(p) != hipSuccess) (void)hipGetLastError();
    ctx->deferred_frees.clear();
    // without a graph nothing will replay the recorded kernels: their scratch goes straight back to the pool
    auto drop_owned = [&]() {
        for (auto &b : ctx->capture_owned) {
            ctx->pending_return_bytes -= std::min(ctx->pending_return_bytes, b.cls);
            pool_free(ctx, b.ptr, b.bytes, b.cls);
        }
        ctx->capture_owned.clear();
    };
    if (e != hipSuccess || !g) {
        drop_owned();
        return hip_fail(ctx, e, "hipStreamEndCapture", FA_ERR_KERNEL_LAUNCH_FAILED);
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        drop_owned();
        return hip_fail(ctx, e, "hipGraphInstantiate", FA_ERR_KERNEL_LAUNCH_FAILED);
    }
    fa_graph *gr = new (std::nothrow) fa_graph();
    if (!gr) {
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(g);
        drop_owned();
        return fail(FA_ERR_ALLOCATION_FAILED, "host allocation of the graph handle failed");
    }
    gr->magic = kGraphMagic;
    gr->ctx = ctx;
    ctx->live_graphs += 1;
    gr->graph = g;
    gr->exec = exec;
    gr->owned.swap(ctx->capture_owned);
    *out = gr;
    return FA_OK;
}

fa_status fa_graph_launch(fa_context *ctx, fa_graph *graph) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!graph || graph->magic != kGraphMagic) return fail(FA_ERR_INVALID_ARGUMENT, "fa_graph_launch: not a graph");
    if (graph->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, "fa_graph_launch: the graph was recorded on another context");
    if (ctx->capturing) return fail(FA_ERR_CAPTURE_IN_PROGRESS, "fa_graph_launch during capture");
    hipError_t e = hipGraphLaunch(graph->exec, ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipGraphLaunch", FA_ERR_KERNEL_LAUNCH_FAILED);
    return FA_OK;
}

fa_status fa_graph_destroy(fa_context *ctx, fa_graph *graph) {
    if (!graph) return FA_OK;
    if (graph->magic != kGraphMagic) return fail(FA_ERR_INVALID_ARGUMENT, "fa_graph_destroy: not a graph");
    // The blocks a graph owns come from the pool of the context that recorded it and go back there, so that context
    // and no other has to be passed (and has to be alive: fa_context_destroy refuses while graphs of it live).
    if (!ctx || ctx->magic != kCtxMagic) return fail(FA_ERR_INVALID_ARGUMENT, "fa_graph_destroy: the graph's context is needed");
    if (graph->ctx != ctx) return fail(FA_ERR_DEVICE_MISMATCH, "fa_graph_destroy: the graph was recorded on another context");
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipGraphExecDestroy(graph->exec);
    (void)hipGraphDestroy(graph->graph);
    // every replay has finished (synchronized above): the scratch the recorded kernels used is free again
    for (auto &b : graph->owned) {
        ctx->pending_return_bytes -= std::min(ctx->pending_return_bytes, b.cls);
        pool_free(ctx, b.ptr, b.bytes, b.cls);
    }
    graph->owned.clear();
    if (ctx->live_graphs) ctx->live_graphs -= 1;
    graph->magic = 0;
    delete graph;
    return FA_OK;
}

fa_status fa_graph_owned_blocks(const fa_graph *graph, void **ptrs, uint64_t capacity, uint64_t *count) {
    if (!graph || graph->magic != kGraphMagic || !count) return fail(FA_ERR_INVALID_ARGUMENT, "fa_graph_owned_blocks: bad argument");
    *count = graph->owned.size();
    for (uint64_t i = 0; i < graph->owned.size() && i < capacity && ptrs; ++i) ptrs[i] = graph->owned[i].ptr;
    return FA_OK;
}

// ------------------------------------------------------------------ timers
fa_status fa_timer_create(fa_context *ctx, fa_timer **out) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!out) return fail(FA_ERR_INVALID_ARGUMENT, "fa_timer_create: null output");
    fa_timer *t = new (std::nothrow) fa_timer();
    if (!t) return fail(FA_ERR_ALLOCATION_FAILED, "host allocation of the timer failed");
    hipError_t e = hipEventCreate(&t->start);
    if (e == hipSuccess) e = hipEventCreate(&t->stop);
    if (e != hipSuccess) {
        delete t;
        return hip_fail(ctx, e, "hipEventCreate", FA_ERR_KERNEL_LAUNCH_FAILED);
    }
    *out = t;
    return FA_OK;
}
fa_status fa_timer_start(fa_context *ctx, fa_timer *t) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!t) return fail(FA_ERR_INVALID_ARGUMENT, "fa_timer_start: null timer");
    hipError_t e = hipEventRecord(t->start, ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipEventRecord", FA_ERR_KERNEL_LAUNCH_FAILED);
    return FA_OK;
}
fa_status fa_timer_stop(fa_context *ctx, fa_timer *t) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!t) return fail(FA_ERR_INVALID_ARGUMENT, "fa_timer_stop: null timer");
    hipError_t e = hipEventRecord(t->stop, ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipEventRecord", FA_ERR_KERNEL_LAUNCH_FAILED);
    return FA_OK;
}
fa_status fa_timer_elapsed_ms(fa_context *ctx, fa_timer *t, float *ms) {
    if (fa_status s = check_ctx(ctx)) return s;
    if (!t || !ms) return fail(FA_ERR_INVALID_ARGUMENT, "fa_timer_elapsed_ms: null argument");
    hipError_t e = hipEventSynchronize(t->stop);
    if (e == hipSuccess) e = hipEventElapsedTime(ms, t->start, t->stop);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipEventElapsedTime", FA_ERR_KERNEL_LAUNCH_FAILED);
    return FA_OK;
}
fa_status fa_timer_destroy(fa_context *ctx, fa_timer *t) {
    (void)ctx;
    if (!t) return FA_OK;
    (void)hipEventDestroy(t->start);
    (void)hipEventDestroy(t->stop);
    delete t;
    return FA_OK;
}

}  // extern "C"
