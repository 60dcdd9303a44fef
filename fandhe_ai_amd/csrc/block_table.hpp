// Page table and free-block bookkeeping of a paged KV cache (host logic), and
// the one-layer device-resident cache built on it.  Follows the reference's
// BlockTable (crates/autodiff/src/nn/paged_kv.rs:147-363) and PagedKvCache
// (crates/autodiff/src/nn/paged_kv_device.rs:67-372): free blocks are a stack
// of returned ids (last in, first out) followed by the never-used ids in
// ascending order; every row of the batch has the same length; operations
// either succeed or leave the table as it was.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace fa {

struct BlockTable {
    std::vector<uint32_t> returned;
    size_t next_unused = 0;
    std::vector<std::vector<uint32_t>> tables;
    std::vector<size_t> seq_lens;
    bool has_batch = false;
    size_t batch = 0;

    size_t free_blocks(size_t max_blocks) const;
    // false when no block is free (callers check the count first)
    bool alloc(size_t max_blocks, uint32_t *id);
    void reset();
    size_t seq_len() const { return seq_lens.empty() ? 0 : seq_lens[0]; }
    size_t used_blocks() const;
    // Reserves blocks for l_new more tokens in each of b rows and returns the slot of every new
    // token, rows first (slot = block_id * block_size + pos % block_size).  Mutates *this: callers
    // work on a copy and commit it after the device write succeeded.  Empty string on success,
    // otherwise the reason (and *this may be partly updated: discard the copy).
    std::string extend_for_append(size_t max_blocks, size_t block_size, size_t b, size_t l_new,
                                  std::vector<uint32_t> *slots);
    // [rows, max_blocks_per_seq] with UINT32_MAX in unused entries
    std::string flatten_tables(size_t max_blocks_per_seq, std::vector<uint32_t> *out) const;
    // Shrinks every row to new_len tokens and returns the blocks past it to the free stack.
    std::string rewind_to(size_t new_len, size_t block_size);
};

// PagedKvCacheConfig::new (paged_kv.rs:79-108): block_size a power of two in 1..256, max_blocks in
// 1..UINT32_MAX, embed_dim >= 1, both pools together at most PTRDIFF_MAX bytes at `elem_bytes` each.
std::string check_cache_config(size_t block_size, size_t max_blocks, size_t embed_dim, size_t elem_bytes);

}  // namespace fa
