// C++ host side above the C ABI of fandhe_rocm.h: the reference's operator, memory, generation and
// scheduling interfaces for the quantized decode path, with the reference's names, argument meaning and
// error behaviour (the reference is Rust; this is what a C++ caller, or the Rust glue crate, sits on).
//
//   Context / Buffer / QWeight     DeviceProvider::select, MemoryOps + DeviceBuffer
//                                  (crates/tensor-core/src/device.rs:149-168, buffer.rs:91-521), quantized weights
//   RocmBackendOps                 the BackendOps entries of the path (crates/tensor-core/src/backend_ops.rs:
//                                  1998 gemm_device, 4296 linear_forward_device, 4694 paged_kv_append,
//                                  4742 paged_attention_forward, 5113 rmsnorm, 4897 synchronize_device)
//   Decoder                        the resident decoder of the library (composition of the operators)
//   SamplingStrategy, GenerateConfig, generate
//                                  crates/autodiff/src/generate/mod.rs:101-248, 500-640
//   SchedulerLimits, PageAllocator, BatchScheduler
//                                  crates/autodiff/src/generate/scheduler.rs:75-127, 395-720;
//                                  crates/autodiff/src/nn/paged_kv.rs:147-191 (allocation order)
//   generate_speculative           crates/autodiff/src/generate/speculative.rs:334-531 (greedy and sampled forms)
//   BlockTable, PagedKvCache       crates/autodiff/src/nn/paged_kv.rs:147-363, paged_kv_device.rs:67-372
//
// Header only, C++17, no dependency besides the C header; every device call goes through the C ABI, so
// nothing here computes on the host what the library computes on the device.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <deque>
#include <optional>
#include <set>
#include <stdexcept>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "fandhe_rocm.h"

namespace fandhe {

// ------------------------------------------------------------------------------------------------ errors
// BackendError (crates/tensor-core/src/device.rs:225-371): the status of the failed call and its message.
class BackendError : public std::runtime_error {
  public:
    BackendError(fa_status s, const std::string &msg) : std::runtime_error(std::string(fa_status_name(s)) + ": " + msg), status(s) {}
    fa_status status;
};
// AutodiffError::InvalidArgument: a request the host layer rejects before anything is queued.
class InvalidArgument : public std::invalid_argument {
  public:
    using std::invalid_argument::invalid_argument;
};
inline void check(fa_status s) {
    if (s != FA_OK) throw BackendError(s, fa_last_error_message());
}

// ----------------------------------------------------------------------------------------------- context
class Context {
  public:
    static int32_t device_count() {
        int32_t n = 0;
        check(fa_device_count(&n));
        return n;
    }
    explicit Context(int32_t ordinal = 0) { check(fa_context_create(ordinal, &h_)); }
    ~Context() {
        if (h_) fa_context_destroy(h_);
    }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    fa_context *handle() const { return h_; }
    fa_device_info info() const {
        fa_device_info i;
        check(fa_context_info(h_, &i));
        return i;
    }
    void synchronize_device() const { check(fa_synchronize_device(h_)); }
    fa_pool_stats device_memory_pool_stats() const {
        fa_pool_stats s;
        check(fa_device_memory_pool_stats(h_, &s));
        return s;
    }
    void release_cached_device_memory() const { check(fa_release_cached_device_memory(h_)); }

  private:
    fa_context *h_ = nullptr;
};

// ------------------------------------------------------------------------------------------------ memory
template <typename T> struct dtype_of;
template <> struct dtype_of<float> { static constexpr fa_dtype value = FA_F32; };
template <> struct dtype_of<int32_t> { static constexpr fa_dtype value = FA_I32; };
template <> struct dtype_of<uint32_t> { static constexpr fa_dtype value = FA_U32; };
template <> struct dtype_of<int8_t> { static constexpr fa_dtype value = FA_I8; };

// DeviceBuffer: owns one pooled allocation; dropping it returns the block to the pool.
class Buffer {
  public:
    Buffer() = default;
    Buffer(const Context &ctx, fa_buffer *h) : ctx_(&ctx), h_(h) {}
    ~Buffer() { reset(); }
    Buffer(Buffer &&o) noexcept : ctx_(o.ctx_), h_(o.h_) { o.h_ = nullptr; }
    Buffer &operator=(Buffer &&o) noexcept {
        if (this != &o) {
            reset();
            ctx_ = o.ctx_;
            h_ = o.h_;
            o.h_ = nullptr;
        }
        return *this;
    }
    Buffer(const Buffer &) = delete;
    Buffer &operator=(const Buffer &) = delete;

    static Buffer alloc_zeroed(const Context &ctx, fa_dtype dtype, uint64_t numel) {
        fa_buffer *h = nullptr;
        check(fa_alloc_zeroed(ctx.handle(), dtype, numel, &h));
        return Buffer(ctx, h);
    }
    static Buffer alloc_uninit(const Context &ctx, fa_dtype dtype, uint64_t numel) {
        fa_buffer *h = nullptr;
        check(fa_alloc_uninit(ctx.handle(), dtype, numel, &h));
        return Buffer(ctx, h);
    }
    template <typename T> static Buffer upload(const Context &ctx, const std::vector<T> &host) {
        fa_buffer *h = nullptr;
        check(fa_upload(ctx.handle(), dtype_of<T>::value, host.data(), host.size(), &h));
        return Buffer(ctx, h);
    }
    // bf16 values travel as their 16-bit patterns
    static Buffer upload_bf16(const Context &ctx, const std::vector<uint16_t> &bits) {
        fa_buffer *h = nullptr;
        check(fa_upload(ctx.handle(), FA_BF16, bits.data(), bits.size(), &h));
        return Buffer(ctx, h);
    }
    template <typename T> void upload_into(const std::vector<T> &host, uint64_t dst_offset) {
        check(fa_upload_into(ctx_->handle(), host.data(), host.size(), h_, dst_offset));
    }
    template <typename T> std::vector<T> download(uint64_t offset = 0, uint64_t count = UINT64_MAX) const {
        const uint64_t n = count == UINT64_MAX ? numel() - offset : count;
        std::vector<T> out(n);
        check(fa_download(ctx_->handle(), h_, offset, out.data(), n));
        return out;
    }
    uint64_t numel() const { return h_ ? fa_buffer_numel(h_) : 0; }
    fa_dtype dtype() const { return fa_buffer_dtype(h_); }
    fa_buffer *handle() const { return h_; }
    explicit operator bool() const { return h_ != nullptr; }
    void reset() {
        if (h_) fa_buffer_free(ctx_->handle(), h_);
        h_ = nullptr;
    }

  private:
    const Context *ctx_ = nullptr;
    fa_buffer *h_ = nullptr;
};

// DeviceBufferView (buffer.rs:277-373): a buffer and an element offset; the extent is the operator's.
struct BufferView {
    const Buffer *buffer = nullptr;
    uint64_t offset = 0;
};

// A quantized weight: codes in the matrix-core tile order plus scales, produced on the device.
class QWeight {
  public:
    QWeight() = default;
    ~QWeight() { reset(); }
    QWeight(QWeight &&o) noexcept : ctx_(o.ctx_), h_(o.h_) { o.h_ = nullptr; }
    QWeight &operator=(QWeight &&o) noexcept {
        if (this != &o) {
            reset();
            ctx_ = o.ctx_;
            h_ = o.h_;
            o.h_ = nullptr;
        }
        return *this;
    }
    QWeight(const QWeight &) = delete;
    QWeight &operator=(const QWeight &) = delete;
    // w[k, n] f32 (the layout of linear_forward_device)
    static QWeight from_f32(const Context &ctx, BufferView w, uint64_t k, uint64_t n, fa_qweight_kind kind = FA_QW_INT8_CHANNEL) {
        QWeight q;
        q.ctx_ = &ctx;
        check(fa_qweight_from_f32(ctx.handle(), w.buffer->handle(), w.offset, k, n, kind, &q.h_));
        return q;
    }
    static QWeight from_codes(const Context &ctx, const void *codes, const float *scales, uint64_t k, uint64_t n,
                              fa_qweight_kind kind = FA_QW_INT8_CHANNEL) {
        QWeight q;
        q.ctx_ = &ctx;
        check(fa_qweight_from_codes(ctx.handle(), codes, scales, k, n, kind, &q.h_));
        return q;
    }
    uint64_t k() const { return fa_qweight_k(h_); }
    uint64_t n() const { return fa_qweight_n(h_); }
    fa_qweight *handle() const { return h_; }
    void reset() {
        if (h_) fa_qweight_free(ctx_->handle(), h_);
        h_ = nullptr;
    }

  private:
    const Context *ctx_ = nullptr;
    fa_qweight *h_ = nullptr;
};

// ---------------------------------------------------------------------------------------------- operators
// PagedKvLayout::new (crates/tensor-core/src/paged_kv.rs:47-131): rejected here as in the reference.
inline fa_paged_layout paged_layout(uint64_t num_blocks, uint64_t block_size, uint64_t embed_dim) {
    fa_paged_layout l{num_blocks, block_size, embed_dim};
    // an append of zero rows validates the layout alone
    check(fa_validate_paged_kv_append(0, 0, num_blocks * block_size * embed_dim, num_blocks * block_size * embed_dim, nullptr, 0, &l));
    return l;
}
inline float default_scale(uint64_t head_dim) { return 1.0f / std::sqrt((float)head_dim); }

// The BackendOps entries of the path.  Outputs are allocated from the context's pool and returned, as the
// reference's operators do; all calls are asynchronous on the context's stream.
class RocmBackendOps {
  public:
    explicit RocmBackendOps(const Context &ctx) : ctx_(ctx) {}
    const Context &context() const { return ctx_; }

    Buffer gemm_device(const Buffer &a, const Buffer &b, uint64_t m, uint64_t n, uint64_t k) const {
        Buffer out = Buffer::alloc_uninit(ctx_, FA_F32, m * n);
        check(fa_gemm_device(ctx_.handle(), a.handle(), b.handle(), m, n, k, out.handle()));
        return out;
    }
    Buffer linear_forward_device(const Buffer &a, uint64_t m, uint64_t k, BufferView w, uint64_t n,
                                 std::optional<BufferView> bias, fa_activation act = FA_ACT_NONE) const {
        Buffer out = Buffer::alloc_uninit(ctx_, FA_F32, m * n);
        check(fa_linear_forward_device(ctx_.handle(), a.handle(), m, k, w.buffer->handle(), w.offset, n,
                                       bias ? bias->buffer->handle() : nullptr, bias ? bias->offset : 0, act, out.handle()));
        return out;
    }
    Buffer rmsnorm(const Buffer &x, const Buffer *w, float eps, uint64_t rows, uint64_t hidden) const {
        Buffer out = Buffer::alloc_uninit(ctx_, FA_F32, rows * hidden);
        check(fa_rmsnorm(ctx_.handle(), x.handle(), w ? w->handle() : nullptr, eps, rows, hidden, out.handle()));
        return out;
    }
    // x f32 or bf16 [m, k]; out f32 unless out_dtype says bf16
    Buffer linear_w8a8(const Buffer &x, uint64_t m, const QWeight &qw, fa_dtype out_dtype = FA_F32) const {
        Buffer out = Buffer::alloc_uninit(ctx_, out_dtype, m * qw.n());
        check(fa_linear_w8a8(ctx_.handle(), x.handle(), m, qw.handle(), nullptr, 0, nullptr, out.handle()));
        return out;
    }
    Buffer linear_w8a16(const Buffer &a_bf16, uint64_t m, const QWeight &qw, fa_dtype out_dtype = FA_BF16) const {
        Buffer out = Buffer::alloc_uninit(ctx_, out_dtype, m * qw.n());
        check(fa_linear_w8a16(ctx_.handle(), a_bf16.handle(), m, qw.handle(), out.handle()));
        return out;
    }
    void paged_kv_append(const Buffer &k_new, const Buffer &v_new, Buffer &k_pool, Buffer &v_pool,
                         const std::vector<uint32_t> &slot_mapping, const fa_paged_layout &layout) const {
        check(fa_paged_kv_append(ctx_.handle(), k_new.handle(), v_new.handle(), k_pool.handle(), v_pool.handle(),
                                 slot_mapping.data(), slot_mapping.size(), &layout));
    }
    Buffer paged_attention_forward(const Buffer &q, const Buffer &k_pool, const Buffer &v_pool,
                                   const std::vector<uint32_t> &block_tables, const std::vector<uint32_t> &seq_lens,
                                   const fa_paged_args &args) const {
        const uint64_t hkv = args.num_kv_heads ? args.num_kv_heads : args.num_heads;
        const uint64_t e_q = hkv ? args.num_heads * (args.layout.embed_dim / hkv) : 0;
        Buffer out = Buffer::alloc_uninit(ctx_, q.dtype(), args.batch * args.l_new * e_q);
        check(fa_paged_attention_forward(ctx_.handle(), q.handle(), k_pool.handle(), v_pool.handle(), block_tables.data(),
                                         block_tables.size(), seq_lens.data(), seq_lens.size(), &args, out.handle()));
        return out;
    }

  private:
    const Context &ctx_;
};

// ------------------------------------------------------------------------------------------- cache layer
// BlockTable (crates/autodiff/src/nn/paged_kv.rs:147-363): page table with free-block bookkeeping; pure host
// state.  Free blocks are the stack of returned ids (last in, first out), then the never-used ids ascending;
// all rows have one length; every call either succeeds or leaves the table unchanged.
class BlockTable {
  public:
    explicit BlockTable(uint64_t max_blocks, uint64_t block_size) : max_blocks_(max_blocks), block_size_(block_size) {
        check(fa_block_table_create(&h_));
    }
    ~BlockTable() {
        if (h_) fa_block_table_destroy(h_);
    }
    BlockTable(const BlockTable &o) : max_blocks_(o.max_blocks_), block_size_(o.block_size_) { check(fa_block_table_clone(o.h_, &h_)); }
    BlockTable &operator=(const BlockTable &) = delete;
    fa_block_table_state state() const {
        fa_block_table_state st;
        check(fa_block_table_state_get(h_, max_blocks_, &st));
        return st;
    }
    uint64_t seq_len() const { return state().seq_len; }
    uint64_t free_blocks() const { return state().free_blocks; }
    std::optional<uint32_t> alloc() {
        uint32_t id = 0;
        int32_t got = 0;
        check(fa_block_table_alloc(h_, max_blocks_, &id, &got));
        return got ? std::optional<uint32_t>(id) : std::nullopt;
    }
    // slots of the b * l_new new tokens, rows first
    std::vector<uint32_t> extend_for_append(uint64_t b, uint64_t l_new) {
        std::vector<uint32_t> slots(b * l_new);
        uint64_t n = 0;
        check(fa_block_table_extend_for_append(h_, max_blocks_, block_size_, b, l_new, slots.data(), slots.size(), &n));
        slots.resize(n);
        return slots;
    }
    // [rows, max_blocks_per_seq], UINT32_MAX in unused entries
    std::vector<uint32_t> flatten_tables(uint64_t max_blocks_per_seq) const {
        std::vector<uint32_t> out(state().batch * max_blocks_per_seq);
        uint64_t n = 0;
        check(fa_block_table_flatten(h_, max_blocks_per_seq, out.data(), out.size(), &n));
        out.resize(n);
        return out;
    }
    void rewind_to(uint64_t new_len) { check(fa_block_table_rewind_to(h_, new_len, block_size_)); }
    void reset() { check(fa_block_table_reset(h_)); }

  private:
    fa_block_table *h_ = nullptr;
    uint64_t max_blocks_, block_size_;
};

// PagedKvCache (crates/autodiff/src/nn/paged_kv_device.rs:67-372): the one-layer device-resident cache.
class PagedKvCache {
  public:
    PagedKvCache(const Context &ctx, uint64_t block_size, uint64_t max_blocks, uint64_t embed_dim, fa_dtype dtype = FA_F32)
        : ctx_(ctx), embed_dim_(embed_dim), dtype_(dtype) {
        check(fa_paged_cache_create(ctx.handle(), block_size, max_blocks, embed_dim, dtype, &h_));
    }
    ~PagedKvCache() {
        if (h_) fa_paged_cache_destroy(ctx_.handle(), h_);
    }
    PagedKvCache(const PagedKvCache &) = delete;
    PagedKvCache &operator=(const PagedKvCache &) = delete;
    fa_block_table_state state(bool *poisoned = nullptr) const {
        fa_block_table_state st;
        int32_t p = 0;
        check(fa_paged_cache_state_get(h_, &st, &p));
        if (poisoned) *poisoned = p != 0;
        return st;
    }
    uint64_t seq_len() const { return state().seq_len; }
    uint64_t num_free_blocks() const { return state().free_blocks; }
    bool is_poisoned() const {
        bool p = false;
        state(&p);
        return p;
    }
    // k_new / v_new [b, l_new, embed_dim] of the pools' type
    void append(const Buffer &k_new, const Buffer &v_new, uint64_t b, uint64_t l_new) {
        check(fa_paged_cache_append(ctx_.handle(), h_, k_new.handle(), v_new.handle(), b, l_new));
    }
    // q / out [b, l_new, num_heads * head_dim]
    Buffer attention(const Buffer &q, uint64_t b, uint64_t l_new, uint64_t num_heads, uint64_t num_kv_heads, float scale) const {
        const uint64_t hkv = num_kv_heads ? num_kv_heads : num_heads;
        Buffer out = Buffer::alloc_uninit(ctx_, dtype_, b * l_new * num_heads * (embed_dim_ / hkv));
        check(fa_paged_cache_attention(ctx_.handle(), h_, q.handle(), b, l_new, num_heads, num_kv_heads, scale, out.handle()));
        return out;
    }
    void rewind_to(uint64_t new_len) { check(fa_paged_cache_rewind_to(h_, new_len)); }
    void clear() { check(fa_paged_cache_clear(h_)); }

  private:
    const Context &ctx_;
    fa_paged_cache *h_ = nullptr;
    uint64_t embed_dim_;
    fa_dtype dtype_;
};

// ------------------------------------------------------------------------------------------------ decoder
// The resident decoder: weights are borrowed (the caller keeps buffers and quantized weights alive).
class Decoder {
  public:
    Decoder(const Context &ctx, const fa_decoder_config &cfg) : ctx_(ctx), cfg_(cfg) {
        check(fa_decoder_create(ctx.handle(), &cfg_, &h_));
    }
    ~Decoder() {
        if (h_) fa_decoder_destroy(ctx_.handle(), h_);
    }
    Decoder(const Decoder &) = delete;
    Decoder &operator=(const Decoder &) = delete;
    const fa_decoder_config &config() const { return cfg_; }
    fa_decoder *handle() const { return h_; }

    void set_layer(uint32_t layer, const Buffer &attn_norm, const Buffer &ffn_norm, const QWeight &wqkv, const QWeight &wo,
                   const QWeight &wgu, const QWeight &wdown) {
        check(fa_decoder_set_layer(h_, layer, attn_norm.handle(), ffn_norm.handle(), wqkv.handle(), wo.handle(), wgu.handle(),
                                   wdown.handle()));
    }
    void set_head(const Buffer &embed, const Buffer &final_norm, const QWeight &lm_head) {
        check(fa_decoder_set_head(h_, embed.handle(), final_norm.handle(), lm_head.handle()));
    }
    // tables [batch, max_blocks_per_seq] row-major, unused entries UINT32_MAX; lens [batch]
    void set_sequences(const std::vector<uint32_t> &block_tables, const std::vector<uint32_t> &seq_lens) {
        if (block_tables.size() != seq_lens.size() * (size_t)cfg_.max_blocks_per_seq)
            throw InvalidArgument("set_sequences: block_tables must hold max_blocks_per_seq entries per sequence");
        check(fa_decoder_set_sequences(ctx_.handle(), h_, (uint32_t)seq_lens.size(), block_tables.data(), seq_lens.data()));
        batch_ = (uint32_t)seq_lens.size();
    }
    void set_tokens(const std::vector<int32_t> &tokens) {
        if (tokens.size() != batch_) throw InvalidArgument("set_tokens: one token per installed sequence");
        check(fa_decoder_set_tokens(ctx_.handle(), h_, tokens.data()));
    }
    void set_sampling(fa_sampling strategy, float temperature, uint64_t top_k, uint64_t seed) {
        check(fa_decoder_set_sampling(ctx_.handle(), h_, strategy, temperature, top_k, seed));
    }
    void set_row_sampling(const std::vector<fa_row_sampling> &rows) {
        if (rows.size() != batch_) throw InvalidArgument("set_row_sampling: one record per installed sequence");
        check(fa_decoder_set_row_sampling(ctx_.handle(), h_, rows.data()));
    }
    std::vector<fa_row_sampling> read_row_sampling() const {
        std::vector<fa_row_sampling> rows(batch_);
        check(fa_decoder_read_row_sampling(ctx_.handle(), h_, rows.data()));
        return rows;
    }
    // tokens [batch, l_new] row-major
    void prefill(const std::vector<int32_t> &tokens, uint32_t l_new) {
        if (tokens.size() != (size_t)batch_ * l_new) throw InvalidArgument("prefill: tokens must be [batch, l_new]");
        check(fa_decoder_prefill(ctx_.handle(), h_, tokens.data(), l_new));
    }
    // prompts of different lengths in one pass; every row ends as after its own prefill
    void prefill_padded(const std::vector<std::vector<int32_t>> &prompts) {
        if (prompts.size() != batch_) throw InvalidArgument("prefill_padded: one prompt per installed sequence");
        uint32_t l_max = 0;
        for (const auto &p : prompts) l_max = std::max<uint32_t>(l_max, (uint32_t)p.size());
        std::vector<int32_t> padded((size_t)batch_ * l_max, 0);
        std::vector<uint32_t> lens(batch_);
        for (uint32_t b = 0; b < batch_; ++b) {
            std::copy(prompts[b].begin(), prompts[b].end(), padded.begin() + (size_t)b * l_max);
            lens[b] = (uint32_t)prompts[b].size();
        }
        check(fa_decoder_prefill_padded(ctx_.handle(), h_, padded.data(), l_max, lens.data()));
    }
    // every position's pick (and logits when asked): tokens [batch, l_new]
    std::vector<int32_t> verify(const std::vector<int32_t> &tokens, uint32_t l_new, std::vector<float> *logits = nullptr) {
        if (tokens.size() != (size_t)batch_ * l_new) throw InvalidArgument("verify: tokens must be [batch, l_new]");
        std::vector<int32_t> picked(tokens.size());
        if (logits) logits->resize(tokens.size() * (size_t)cfg_.vocab);
        check(fa_decoder_verify(ctx_.handle(), h_, tokens.data(), l_new, picked.data(), logits ? logits->data() : nullptr));
        return picked;
    }
    void rewind(const std::vector<uint32_t> &seq_lens) {
        if (seq_lens.size() != batch_) throw InvalidArgument("rewind: one length per installed sequence");
        check(fa_decoder_rewind(ctx_.handle(), h_, seq_lens.data()));
    }
    void step(bool use_graph = true) { check(fa_decoder_step(ctx_.handle(), h_, use_graph ? 1 : 0)); }
    std::vector<int32_t> tokens() const {
        std::vector<int32_t> out(batch_);
        check(fa_decoder_read_tokens(ctx_.handle(), h_, out.data()));
        return out;
    }
    std::vector<float> logits() const {
        std::vector<float> out((size_t)batch_ * cfg_.vocab);
        check(fa_decoder_read_logits(ctx_.handle(), h_, out.data()));
        return out;
    }
    std::vector<uint32_t> seq_lens() const {
        std::vector<uint32_t> out(batch_);
        check(fa_decoder_read_seq_lens(ctx_.handle(), h_, out.data()));
        return out;
    }
    // the resident logits [max_batch, vocab] (owned by the decoder)
    fa_buffer *logits_buffer() const {
        fa_buffer *b = nullptr;
        check(fa_decoder_logits_buffer(h_, &b));
        return b;
    }
    const Context &context() const { return ctx_; }

  private:
    const Context &ctx_;
    fa_decoder_config cfg_;
    fa_decoder *h_ = nullptr;
    uint32_t batch_ = 0;
};

// --------------------------------------------------------------------------------------------- generation
// SamplingStrategy::{Greedy, TopK(k), Temperature(t)} (generate/mod.rs:101-113).
struct SamplingStrategy {
    fa_sampling kind = FA_SAMPLE_GREEDY;
    uint64_t k = 0;
    float t = 1.0f;
    static SamplingStrategy Greedy() { return {}; }
    static SamplingStrategy TopK(uint64_t k) { return {FA_SAMPLE_TOP_K, k, 1.0f}; }
    static SamplingStrategy Temperature(float t) { return {FA_SAMPLE_TEMPERATURE, 0, t}; }
};

// GenerateConfig (generate/mod.rs:124-229): max_length counts the prompt; temperature and top_k follow from
// the strategy, and a configuration that contradicts it is rejected, never repaired.
struct GenerateConfig {
    uint64_t max_length;
    SamplingStrategy strategy;
    uint64_t seed = 0;
    float temperature;
    std::optional<uint64_t> top_k;

    GenerateConfig(uint64_t max_length_, SamplingStrategy s)
        : max_length(max_length_), strategy(s), temperature(s.kind == FA_SAMPLE_TEMPERATURE ? s.t : 1.0f),
          top_k(s.kind == FA_SAMPLE_TOP_K ? std::optional<uint64_t>(s.k) : std::nullopt) {}
    GenerateConfig &with_temperature(float t) {
        temperature = t;
        return *this;
    }
    GenerateConfig &with_seed(uint64_t s) {
        seed = s;
        return *this;
    }
    void validate() const {
        if (!(std::isfinite(temperature) && temperature > 0.0f))
            throw InvalidArgument("GenerateConfig: temperature must be finite and positive");
        switch (strategy.kind) {
            case FA_SAMPLE_GREEDY:
                if (temperature != 1.0f || top_k) throw InvalidArgument("GenerateConfig: Greedy requires temperature == 1.0 and top_k == None");
                break;
            case FA_SAMPLE_TOP_K:
                if (!top_k || *top_k != strategy.k) throw InvalidArgument("GenerateConfig: TopK(k) requires top_k == k");
                if (strategy.k < 1) throw InvalidArgument("GenerateConfig: TopK needs k >= 1");
                break;
            case FA_SAMPLE_TEMPERATURE:
                if (top_k) throw InvalidArgument("GenerateConfig: Temperature requires top_k == None");
                if (temperature != strategy.t) throw InvalidArgument("GenerateConfig: Temperature(t) requires temperature == t");
                break;
            default: throw InvalidArgument("GenerateConfig: unknown strategy");
        }
    }
    // generate/mod.rs:236-248: k beyond the vocabulary is an error, not clamped
    void validate_top_k_le_vocab(uint64_t vocab) const {
        if (strategy.kind == FA_SAMPLE_TOP_K && strategy.k > vocab) throw InvalidArgument("GenerateConfig: TopK k exceeds vocab_size");
    }
};

namespace detail {
// positions 0 .. max_length - 2 are written (the last generated token is never fed back)
inline uint64_t pages_for(uint64_t max_length, uint64_t block_size) {
    const uint64_t n = (max_length - 1 + block_size - 1) / block_size;
    return n ? n : 1;
}
inline void check_output_bytes(uint64_t elems) {
    if (elems > (uint64_t)INT64_MAX / 4) throw InvalidArgument("output exceeds the allocation limit");
}
}  // namespace detail

// generate (generate/mod.rs:500-640) on a resident decoder: prompt pass, then one decode step per token
// until every row holds max_length tokens.  input_ids [B][T], all rows of one length; the B rows draw in row
// order from the one generator config.seed starts.  Uses pages 0 .. of the decoder's pools and replaces
// whatever sequences were installed.  DecoderT: Decoder, or anything with its members (tests use a host toy).
template <typename DecoderT>
std::vector<std::vector<int32_t>> generate(DecoderT &decoder, const std::vector<std::vector<int32_t>> &input_ids,
                                           const GenerateConfig &config) {
    config.validate();
    const uint64_t b = input_ids.size();
    if (b == 0) throw InvalidArgument("generate: the batch is empty");
    const uint64_t prompt_len = input_ids[0].size();
    for (const auto &row : input_ids)
        if (row.size() != prompt_len) throw InvalidArgument("generate: all prompts of a batch have one length");
    if (prompt_len == 0) throw InvalidArgument("generate: the prompt is empty");
    if (config.max_length < prompt_len) throw InvalidArgument("generate: max_length must be at least the prompt length");
    detail::check_output_bytes(b * config.max_length);
    std::vector<std::vector<int32_t>> out = input_ids;
    if (config.max_length == prompt_len) return out;              // nothing to generate, no forward pass
    const auto &cfg = decoder.config();
    const uint64_t pages = detail::pages_for(config.max_length, cfg.block_size);
    if (b > cfg.max_batch || pages > cfg.max_blocks_per_seq || b * pages > cfg.num_blocks)
        throw InvalidArgument("generate: the rows do not fit the decoder's batch or page pool");
    config.validate_top_k_le_vocab(cfg.vocab);
    std::vector<uint32_t> tables((size_t)b * cfg.max_blocks_per_seq, UINT32_MAX), lens(b, 0);
    for (uint64_t r = 0; r < b; ++r)
        for (uint64_t p = 0; p < pages; ++p) tables[r * cfg.max_blocks_per_seq + p] = (uint32_t)(r * pages + p);
    decoder.set_sequences(tables, lens);
    decoder.set_sampling(config.strategy.kind, config.temperature, config.top_k.value_or(0), config.seed);
    std::vector<int32_t> flat;
    flat.reserve(b * prompt_len);
    for (const auto &row : input_ids) flat.insert(flat.end(), row.begin(), row.end());
    decoder.prefill(flat, (uint32_t)prompt_len);
    for (uint64_t pos = prompt_len; pos < config.max_length; ++pos) {
        if (pos > prompt_len) decoder.step();
        const std::vector<int32_t> tok = decoder.tokens();
        for (uint64_t r = 0; r < b; ++r) {
            if (tok[r] < 0) throw InvalidArgument("generate: logits hold non-finite values");
            out[r].push_back(tok[r]);
        }
    }
    return out;
}

namespace detail {
// The probabilities of sampled speculative decoding, kept on the device: the f32 weight rows of the target
// (k + 1) and of the draft (k), one generator for every draw of the call (speculative.rs:438-447) and the
// acceptance kernel behind fa_speculative_accept.  Only (accepted, token, status) come back to the host.
class DeviceAcceptance {
  public:
    DeviceAcceptance(const Context &ctx, const GenerateConfig &config, uint64_t vocab, uint64_t k)
        : ctx_(ctx), vocab_(vocab), kind_(config.strategy.kind), temperature_(config.temperature), top_k_(config.top_k.value_or(0)),
          gen_(Buffer::alloc_zeroed(ctx, FA_U32, 2)), pw_(Buffer::alloc_uninit(ctx, FA_F32, (k + 1) * vocab)),
          qw_(Buffer::alloc_uninit(ctx, FA_F32, k * vocab)), status_(Buffer::alloc_zeroed(ctx, FA_I32, k + 1)),
          result_(Buffer::alloc_zeroed(ctx, FA_I32, 4)) {
        check(fa_rng_seed(ctx.handle(), gen_.handle(), config.seed));
    }
    // one token from row `row` of `logits` (sample_from over sampling_weights_f32); the weights stay behind as
    // draft row keep_as_q for the acceptance step when keep_as_q >= 0
    int32_t draw(const fa_buffer *logits, uint64_t row, int64_t keep_as_q = -1) {
        Buffer &dst = keep_as_q < 0 ? pw_ : qw_;
        const uint64_t dst_row = keep_as_q < 0 ? 0 : (uint64_t)keep_as_q;
        check(fa_sampling_weights(ctx_.handle(), logits, row * vocab_, 1, vocab_, kind_, temperature_, top_k_, dst.handle(),
                                  dst_row * vocab_, status_.handle()));
        check(fa_speculative_accept(ctx_.handle(), dst.handle(), dst_row * vocab_, nullptr, 0, nullptr, 0, vocab_, gen_.handle(),
                                    result_.handle()));
        return finish(1).second;
    }
    // verify_sampling: rows 0 .. drafts.size() of `logits` are the verification pass
    std::pair<uint64_t, int32_t> verify(const fa_buffer *logits, const std::vector<int32_t> &drafts) {
        const uint64_t rows = drafts.size() + 1;
        check(fa_sampling_weights(ctx_.handle(), logits, 0, rows, vocab_, kind_, temperature_, top_k_, pw_.handle(), 0, status_.handle()));
        check(fa_speculative_accept(ctx_.handle(), pw_.handle(), 0, qw_.handle(), 0, drafts.data(), drafts.size(), vocab_, gen_.handle(),
                                    result_.handle()));
        return finish(rows);
    }

  private:
    std::pair<uint64_t, int32_t> finish(uint64_t rows) {
        const std::vector<int32_t> r = result_.download<int32_t>();
        if (r[2] == 0) return {(uint64_t)r[0], r[1]};
        if (r[2] == 3) {
            const std::vector<int32_t> st = status_.download<int32_t>(0, rows);
            if (std::any_of(st.begin(), st.end(), [](int32_t v) { return v != 0; }))
                throw InvalidArgument("generate_speculative: logits hold non-finite values");
        }
        static const char *why[] = {"", "", "q(x) is not positive, or a probability is not finite",
                                    "probability weights are negative, not finite or sum to zero", "the residual distribution sums to zero",
                                    "a draft token lies outside the vocabulary"};
        throw InvalidArgument(std::string("generate_speculative: ") + (r[2] >= 2 && r[2] <= 5 ? why[r[2]] : "acceptance failed"));
    }
    const Context &ctx_;
    uint64_t vocab_;
    fa_sampling kind_;
    float temperature_;
    uint64_t top_k_;
    Buffer gen_, pw_, qw_, status_, result_;
};
}  // namespace detail

// generate_speculative (crates/autodiff/src/generate/speculative.rs:334-531) on two resident decoders: per round
// the draft decodes k_eff = min(k, remaining - 1) tokens, the target consumes the pending token and those drafts
// in one verification, a prefix of the drafts is kept and one more token from the target's own distribution is
// appended.  Greedy: the longest prefix that equals the target's greedy tokens, then the target's token at the
// first disagreement (or after the last draft).  Temperature / top-k: standard speculative sampling (draft i is
// kept with probability min(1, p / q), the first refused one is replaced by a draw from max(0, p - q), a fully
// accepted round ends with a bonus draw) with one generator seeded from config.seed for every draw of the call in
// the reference's order and all probabilities on the device (detail::DeviceAcceptance).  Both caches are then cut
// back to the accepted length: paged rows past a sequence's length are dead, so nothing is replayed (the
// reference restores a snapshot and replays, kv_rewind.rs:157-215).  One sequence per call.  When the pending
// token and the drafts fit the decoder's rows (k + 1 <= min(32, max_batch)) the verification is one decode step
// whose rows are the k + 1 positions of the one sequence (the same block table in every row, lengths ctx,
// ctx + 1, ...); longer look-aheads take the prompt-shape verification pass.
struct SpeculativeOutput {
    std::vector<int32_t> tokens;
    uint64_t rounds = 0, accepted = 0;
};
template <typename DecoderT>
SpeculativeOutput generate_speculative(DecoderT &target, DecoderT &draft, const std::vector<int32_t> &input_ids,
                                       const GenerateConfig &config, uint64_t k) {
    config.validate();
    if (k < 1) throw InvalidArgument("generate_speculative: k must be at least 1");
    if (input_ids.empty()) throw InvalidArgument("generate_speculative: the prompt is empty");
    const uint64_t max_length = config.max_length, prompt_len = input_ids.size();
    if (max_length < prompt_len) throw InvalidArgument("generate_speculative: max_length must be at least the prompt length");
    detail::check_output_bytes(max_length);
    const bool sampled = config.strategy.kind != FA_SAMPLE_GREEDY;
    SpeculativeOutput out;
    std::vector<int32_t> &row = out.tokens;
    row = input_ids;
    if (max_length == prompt_len) return out;
    if (target.config().vocab != draft.config().vocab) throw InvalidArgument("generate_speculative: the models disagree on the vocabulary");
    const uint64_t vocab = target.config().vocab;
    config.validate_top_k_le_vocab(vocab);
    if (sampled && k > 32) throw InvalidArgument("generate_speculative: the sampled form verifies at most 32 drafts per round");
    const bool by_step = k + 1 <= std::min<uint64_t>(32, target.config().max_batch);
    for (DecoderT *dec : {&target, &draft}) {
        const auto &cfg = dec->config();
        const uint64_t pages = detail::pages_for(max_length + 1, cfg.block_size);   // the verification also writes the last draft
        if (pages > cfg.max_blocks_per_seq || pages > cfg.num_blocks)
            throw InvalidArgument("generate_speculative: the tokens do not fit the decoder's page pool");
    }
    std::optional<detail::DeviceAcceptance> acc;
    if (sampled) acc.emplace(target.context(), config, vocab, k);
    std::vector<uint32_t> target_table;
    for (DecoderT *dec : {&target, &draft}) {
        const auto &cfg = dec->config();
        const uint64_t pages = detail::pages_for(max_length + 1, cfg.block_size);
        std::vector<uint32_t> table(cfg.max_blocks_per_seq, UINT32_MAX);
        for (uint64_t p = 0; p < pages; ++p) table[p] = (uint32_t)p;
        dec->set_sequences(table, {0});
        dec->set_sampling(FA_SAMPLE_GREEDY, 1.0f, 0, 0);          // the decoders' own picks are not used when sampling
        dec->prefill(input_ids, (uint32_t)prompt_len);
        if (dec == &target) target_table = table;
    }
    auto pick = [&](DecoderT &dec) -> int32_t {                   // the next token from row 0 of a decoder's logits
        if (sampled) return acc->draw(dec.logits_buffer(), 0);
        const int32_t tok = dec.tokens()[0];
        if (tok < 0) throw InvalidArgument("generate_speculative: logits hold non-finite values");
        return tok;
    };
    row.push_back(pick(target));
    while (row.size() < max_length) {
        const uint64_t cur = row.size();
        const int32_t last = row.back();
        const uint64_t remaining = max_length - cur;
        if (remaining == 1) {
            target.set_tokens({last});
            target.step();
            row.push_back(pick(target));
            break;
        }
        const uint64_t k_eff = std::min(k, remaining - 1);
        std::vector<int32_t> drafts;
        int32_t x = last;
        for (uint64_t i = 0; i < k_eff; ++i) {                    // the draft's cache grows by last, d1 .. d_{k_eff - 1}
            draft.set_tokens({x});
            draft.step();
            x = sampled ? acc->draw(draft.logits_buffer(), 0, (int64_t)i) : pick(draft);
            drafts.push_back(x);
        }
        std::vector<int32_t> fed{last};
        fed.insert(fed.end(), drafts.begin(), drafts.end());
        std::vector<int32_t> picked;
        uint64_t n_acc = 0;
        int32_t correction = 0;
        if (by_step) {
            const uint64_t n = k_eff + 1;
            std::vector<uint32_t> tables, lens;
            for (uint64_t r = 0; r < n; ++r) {
                tables.insert(tables.end(), target_table.begin(), target_table.end());
                lens.push_back((uint32_t)(cur - 1 + r));
            }
            target.set_sequences(tables, lens);
            target.set_tokens(fed);
            target.step();
            if (sampled) {
                std::tie(n_acc, correction) = acc->verify(target.logits_buffer(), drafts);
            } else {
                picked = target.tokens();
                for (int32_t t : picked)
                    if (t < 0) throw InvalidArgument("generate_speculative: logits hold non-finite values");
            }
        } else if (sampled) {
            std::vector<float> host_logits;
            (void)target.verify(fed, (uint32_t)fed.size(), &host_logits);
            const Buffer staged = Buffer::upload(target.context(), host_logits);
            std::tie(n_acc, correction) = acc->verify(staged.handle(), drafts);
        } else {
            picked = target.verify(fed, (uint32_t)fed.size());
        }
        if (!sampled) {
            while (n_acc < k_eff && drafts[n_acc] == picked[n_acc]) ++n_acc;
            correction = picked[n_acc];
        }
        row.insert(row.end(), drafts.begin(), drafts.begin() + n_acc);
        row.push_back(correction);
        out.rounds += 1;
        out.accepted += n_acc;
        if (row.size() >= max_length) break;
        const uint32_t keep = (uint32_t)(cur + n_acc);            // tokens before the new pending one
        if (by_step)
            target.set_sequences(target_table, {keep});
        else
            target.rewind({keep});
        if (n_acc == k_eff) {
            draft.set_tokens({x});                                // the draft never consumed its own last token
            draft.step();
        } else {
            draft.rewind({keep});
        }
    }
    row.resize(std::min<uint64_t>(row.size(), max_length));
    return out;
}

// ---------------------------------------------------------------------------------------------- scheduler
// scheduler.rs:80-127: every limit is mandatory and at least 1.
struct SchedulerLimits {
    uint64_t max_active, max_queued, max_length;
    SchedulerLimits(uint64_t active, uint64_t queued, uint64_t length) : max_active(active), max_queued(queued), max_length(length) {
        if (active < 1 || queued < 1 || length < 1) throw InvalidArgument("SchedulerLimits: every limit must be at least 1");
        detail::check_output_bytes(length);
    }
};

// Page ids of the shared pools: returned pages are handed out again last in, first out, then the ids never
// used before in ascending order (crates/autodiff/src/nn/paged_kv.rs:147-191).
class PageAllocator {
  public:
    explicit PageAllocator(uint64_t num_blocks) : num_blocks_(num_blocks) {}
    uint64_t free_pages() const { return returned_.size() + num_blocks_ - next_; }
    std::vector<uint32_t> take(uint64_t n) {
        if (n > free_pages()) throw InvalidArgument("page pool exhausted");
        std::vector<uint32_t> out;
        out.reserve(n);
        for (uint64_t i = 0; i < n; ++i) {
            if (!returned_.empty()) {
                out.push_back(returned_.back());
                returned_.pop_back();
            } else {
                out.push_back((uint32_t)next_++);
            }
        }
        return out;
    }
    void give_back(const std::vector<uint32_t> &pages) { returned_.insert(returned_.end(), pages.begin(), pages.end()); }

  private:
    uint64_t num_blocks_, next_ = 0;
    std::vector<uint32_t> returned_;
};

// What the device was asked to do so far: prompt passes, their rows including padding, decode steps, their rows.
struct SchedulerStats {
    uint64_t prompt_passes = 0, prompt_rows = 0, decode_steps = 0, decode_rows = 0;
};

// BatchScheduler (scheduler.rs:395-720) over a resident decoder.  The KV pages of all requests share the
// decoder's pools; every request owns a block-table row, a sampling record with its own generator (seeded
// from its config, one draw per generated token) and its token list.  One step admits queued requests while
// rows and pages are free (pages for the whole max_length are reserved at admission, so an admitted request
// can always finish; one that needs more pages than are free waits at the head of the queue), ingests the
// prompts of the newly admitted requests (requests that join together share padded passes) and advances all
// other active requests together by one decode step.  Requests finish when they reach max_length (no
// end-of-sequence stop, as in the reference) and leave the batch between steps.  A failure of one request
// (non-finite logits, an invalid prompt token) does not touch the others; a device failure takes the rows of
// the failed call with it.
template <typename DecoderT> class BatchScheduler {
  public:
    using Finished = std::pair<uint64_t, std::vector<int32_t>>;
    using Failed = std::pair<uint64_t, std::string>;
    static constexpr uint64_t kMaxPromptRows = 4096;                 // rows (requests x longest prompt) of one padded pass

    BatchScheduler(DecoderT &decoder, SchedulerLimits limits) : dec_(decoder), limits_(limits), pages_(decoder.config().num_blocks) {
        if (limits.max_active > decoder.config().max_batch) throw InvalidArgument("scheduler: max_active exceeds the decoder's max_batch");
    }
    uint64_t queued_len() const { return queue_.size(); }
    uint64_t active_len() const { return active_.size(); }
    uint64_t free_pages() const { return pages_.free_pages(); }
    const SchedulerStats &stats() const { return stats_; }

    // Queues a request without touching the device; checks in the reference's order (config, empty prompt,
    // max_length against the prompt and the limit, queue room); on any error the scheduler is unchanged.
    uint64_t submit(const std::vector<int32_t> &input_ids, const GenerateConfig &config) {
        config.validate();
        if (input_ids.empty()) throw InvalidArgument("scheduler: the prompt is empty");
        if (config.max_length < input_ids.size()) throw InvalidArgument("scheduler: max_length must be at least the prompt length");
        if (config.max_length > limits_.max_length) throw InvalidArgument("scheduler: max_length exceeds the limit");
        detail::check_output_bytes(config.max_length);
        if (queue_.size() >= limits_.max_queued) throw InvalidArgument("scheduler: the queue is full");
        queue_.push_back(Pending{next_id_, input_ids, config});
        return next_id_++;
    }

    // Admits, ingests new prompts, advances everyone else by one token.  Returns how many requests finished
    // successfully in this call; failures of single requests go to take_failed.
    uint64_t step() {
        uint64_t completed = admit();
        const size_t n_fin = finished_.size(), n_fail = failed_.size();
        std::vector<Active *> fresh, old;
        for (auto &a : active_) (a.fresh ? fresh : old).push_back(&a);
        std::set<uint64_t> gone;
        if (!fresh.empty()) {
            pull_resident_state({});                              // the prompt passes overwrite the installed batch
            for (auto &group : prompt_groups(fresh)) {
                std::vector<Active *> bad;
                try {
                    bad = ingest(group);
                } catch (const BackendError &e) {                 // a device failure takes the whole pass with it
                    for (Active *a : group) fail(*a, e.what(), gone);
                    continue;
                }
                for (Active *a : group) {
                    if (std::find(bad.begin(), bad.end(), a) != bad.end())
                        fail(*a, "generate: logits hold non-finite values", gone);
                    else
                        completed += maybe_finish(*a, gone);
                }
            }
        }
        if (!old.empty()) {
            std::vector<uint64_t> ids;
            for (Active *a : old) ids.push_back(a->id);
            try {
                if (!resident_ || *resident_ != ids) install(old);
                dec_.step();
                const std::vector<int32_t> picked = dec_.tokens();
                stats_.decode_steps += 1;
                stats_.decode_rows += old.size();
                for (size_t i = 0; i < old.size(); ++i) {
                    if (picked[i] < 0) {
                        fail(*old[i], "generate: logits hold non-finite values", gone);
                        continue;
                    }
                    old[i]->tokens.push_back(picked[i]);
                    completed += maybe_finish(*old[i], gone);
                }
            } catch (const BackendError &e) {                     // a device failure takes the whole batch with it
                for (Active *a : old)
                    if (!gone.count(a->id)) fail(*a, e.what(), gone);
                resident_.reset();
            }
        }
        if (!gone.empty()) {
            pull_resident_state(gone);                            // the rows move: keep the survivors' generator states
            active_.erase(std::remove_if(active_.begin(), active_.end(), [&](const Active &a) { return gone.count(a.id) != 0; }),
                          active_.end());
        }
        // within one iteration requests are reported in request order, as if they had been advanced one by one
        std::sort(finished_.begin() + n_fin, finished_.end(), [](const Finished &x, const Finished &y) { return x.first < y.first; });
        std::sort(failed_.begin() + n_fail, failed_.end(), [](const Failed &x, const Failed &y) { return x.first < y.first; });
        return completed;
    }
    std::vector<Finished> take_finished() { return std::exchange(finished_, {}); }
    std::vector<Failed> take_failed() { return std::exchange(failed_, {}); }

  private:
    struct Pending {
        uint64_t id;
        std::vector<int32_t> prompt;
        GenerateConfig config;
    };
    struct Active {
        uint64_t id;
        std::vector<int32_t> tokens;
        std::vector<uint32_t> pages;
        fa_row_sampling policy;
        GenerateConfig config;
        bool fresh;
    };

    uint64_t admit() {
        const auto &cfg = dec_.config();
        uint64_t completed = 0;
        while (active_.size() < limits_.max_active && !queue_.empty()) {
            Pending &p = queue_.front();
            if (p.config.max_length == p.prompt.size()) {         // nothing to generate: the prompt is the answer
                finished_.emplace_back(p.id, p.prompt);
                queue_.pop_front();
                ++completed;
                continue;
            }
            const uint64_t need = detail::pages_for(p.config.max_length, cfg.block_size);
            try {
                p.config.validate_top_k_le_vocab(cfg.vocab);
                if (need > cfg.max_blocks_per_seq || need > cfg.num_blocks)
                    throw InvalidArgument("scheduler: max_length needs more pages than the decoder holds");
                for (int32_t t : p.prompt)
                    if (t < 0 || (uint64_t)t >= cfg.vocab) throw InvalidArgument("scheduler: prompt token outside the vocabulary");
            } catch (const InvalidArgument &e) {
                failed_.emplace_back(p.id, e.what());
                queue_.pop_front();
                continue;
            }
            if (need > pages_.free_pages()) break;                // waits for pages, in order
            Active a{p.id, p.prompt, pages_.take(need), fa_row_sampling{}, p.config, true};
            check(fa_rng_state_from_seed(p.config.seed, &a.policy.rng_state));
            a.policy.temperature = p.config.temperature;
            a.policy.top_k = (uint32_t)p.config.top_k.value_or(0);
            a.policy.strategy = (int32_t)p.config.strategy.kind;
            a.policy.reserved = 0;
            queue_.pop_front();
            active_.push_back(std::move(a));
        }
        return completed;
    }
    void table_rows(const std::vector<Active *> &rows, std::vector<uint32_t> &tables) const {
        const uint64_t w = dec_.config().max_blocks_per_seq;
        tables.assign(rows.size() * w, UINT32_MAX);
        for (size_t r = 0; r < rows.size(); ++r) std::copy(rows[r]->pages.begin(), rows[r]->pages.end(), tables.begin() + r * w);
    }
    static std::vector<fa_row_sampling> policy_rows(const std::vector<Active *> &rows) {
        std::vector<fa_row_sampling> out;
        for (const Active *a : rows) out.push_back(a->policy);
        return out;
    }
    void install(const std::vector<Active *> &rows) {
        pull_resident_state({});
        std::vector<uint32_t> tables, lens;
        std::vector<int32_t> last;
        table_rows(rows, tables);
        for (const Active *a : rows) {
            lens.push_back((uint32_t)a->tokens.size() - 1);
            last.push_back(a->tokens.back());
        }
        dec_.set_sequences(tables, lens);
        dec_.set_tokens(last);
        dec_.set_row_sampling(policy_rows(rows));
        resident_.emplace();
        for (const Active *a : rows) resident_->push_back(a->id);
    }
    // generator states advance on the device: fetch them before the installed batch is replaced
    void pull_resident_state(const std::set<uint64_t> &skip) {
        if (!resident_) return;
        const std::vector<fa_row_sampling> rows = dec_.read_row_sampling();
        for (size_t i = 0; i < resident_->size(); ++i) {
            const uint64_t rid = (*resident_)[i];
            if (skip.count(rid)) continue;
            for (auto &a : active_)
                if (a.id == rid) a.policy = rows[i];
        }
        resident_.reset();
    }
    // requests that join in the same iteration share prompt passes: sorted by prompt length and cut into groups
    // whose padded size stays within one pass and whose longest prompt is at most twice the shortest
    std::vector<std::vector<Active *>> prompt_groups(std::vector<Active *> fresh) const {
        std::sort(fresh.begin(), fresh.end(), [](const Active *x, const Active *y) {
            return x->tokens.size() != y->tokens.size() ? x->tokens.size() < y->tokens.size() : x->id < y->id;
        });
        std::vector<std::vector<Active *>> groups;
        std::vector<Active *> cur;
        for (Active *a : fresh) {
            const uint64_t n = a->tokens.size();
            if (!cur.empty() && ((cur.size() + 1) * n > kMaxPromptRows || n > 2 * cur[0]->tokens.size() ||
                                 cur.size() >= dec_.config().max_batch)) {
                groups.push_back(std::move(cur));
                cur.clear();
            }
            cur.push_back(a);
        }
        if (!cur.empty()) groups.push_back(std::move(cur));
        return groups;
    }
    // one prompt pass for the group; returns the requests whose logits were not finite
    std::vector<Active *> ingest(const std::vector<Active *> &group) {
        std::vector<uint32_t> tables;
        table_rows(group, tables);
        dec_.set_sequences(tables, std::vector<uint32_t>(group.size(), 0));
        dec_.set_row_sampling(policy_rows(group));
        uint64_t l_max = 0;
        for (const Active *a : group) l_max = std::max<uint64_t>(l_max, a->tokens.size());
        stats_.prompt_passes += 1;
        stats_.prompt_rows += group.size() * l_max;
        if (group.size() == 1) {
            dec_.prefill(group[0]->tokens, (uint32_t)group[0]->tokens.size());
        } else {
            std::vector<std::vector<int32_t>> prompts;
            for (const Active *a : group) prompts.push_back(a->tokens);
            dec_.prefill_padded(prompts);
        }
        const std::vector<int32_t> toks = dec_.tokens();
        const std::vector<fa_row_sampling> rows = dec_.read_row_sampling();
        std::vector<Active *> bad;
        for (size_t i = 0; i < group.size(); ++i) {
            group[i]->policy = rows[i];
            group[i]->fresh = false;
            if (toks[i] < 0)
                bad.push_back(group[i]);
            else
                group[i]->tokens.push_back(toks[i]);
        }
        return bad;
    }
    uint64_t maybe_finish(Active &a, std::set<uint64_t> &gone) {
        if (a.tokens.size() < a.config.max_length) return 0;
        finished_.emplace_back(a.id, a.tokens);
        pages_.give_back(a.pages);
        gone.insert(a.id);
        return 1;
    }
    void fail(Active &a, const std::string &why, std::set<uint64_t> &gone) {
        failed_.emplace_back(a.id, why);
        pages_.give_back(a.pages);
        gone.insert(a.id);
    }

    DecoderT &dec_;
    SchedulerLimits limits_;
    PageAllocator pages_;
    std::deque<Pending> queue_;
    std::vector<Active> active_;
    std::vector<Finished> finished_;
    std::vector<Failed> failed_;
    std::optional<std::vector<uint64_t>> resident_;               // ids whose decode state is installed, in row order
    uint64_t next_id_ = 0;
    SchedulerStats stats_;
};

}  // namespace fandhe
