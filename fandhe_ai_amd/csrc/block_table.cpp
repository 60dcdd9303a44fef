#include "block_table.hpp"

#include <limits>

namespace fa {

namespace {
bool mul_overflows(size_t a, size_t b, size_t *out) { return __builtin_mul_overflow(a, b, out); }
size_t div_ceil(size_t a, size_t b) { return a / b + (a % b != 0); }
}  // namespace

size_t BlockTable::free_blocks(size_t max_blocks) const {
    return returned.size() + (max_blocks > next_unused ? max_blocks - next_unused : 0);
}

bool BlockTable::alloc(size_t max_blocks, uint32_t *id) {
    if (!returned.empty()) {
        *id = returned.back();
        returned.pop_back();
        return true;
    }
    if (next_unused < max_blocks && next_unused <= std::numeric_limits<uint32_t>::max()) {
        *id = (uint32_t)next_unused;
        ++next_unused;
        return true;
    }
    return false;
}

void BlockTable::reset() {
    returned.clear();
    next_unused = 0;
    tables.clear();
    seq_lens.clear();
    has_batch = false;
    batch = 0;
}

size_t BlockTable::used_blocks() const {
    size_t n = 0;
    for (const auto &t : tables) n += t.size();
    return n;
}

std::string BlockTable::extend_for_append(size_t max_blocks, size_t block_size, size_t b, size_t l_new,
                                          std::vector<uint32_t> *slots) {
    slots->clear();
    if (b == 0) return "batch size 0 cannot be appended";
    if (has_batch && batch != b) return "batch does not match the cache's batch";
    if (l_new == 0) return "";
    const size_t s_prev = seq_len();
    size_t s_total;
    if (__builtin_add_overflow(s_prev, l_new, &s_total)) return "sequence length overflowed";
    const size_t held = div_ceil(s_prev, block_size);
    const size_t extra_per_row = div_ceil(s_total, block_size) - held;
    size_t extra_total;
    if (mul_overflows(extra_per_row, b, &extra_total)) return "number of blocks needed overflowed";
    if (extra_total > free_blocks(max_blocks)) return "not enough free blocks";
    size_t rows;
    if (mul_overflows(b, l_new, &rows)) return "number of appended rows overflowed";
    try {
        slots->reserve(rows);
        if (!has_batch) {
            tables.assign(b, std::vector<uint32_t>());
            seq_lens.assign(b, 0);
            has_batch = true;
            batch = b;
        }
        for (auto &row : tables) row.reserve(row.size() + extra_per_row);
    } catch (const std::exception &) {
        return "out of host memory";
    }
    for (size_t row = 0; row < b; ++row) {
        for (size_t i = 0; i < l_new; ++i) {
            const size_t pos = s_prev + i;
            if (pos % block_size == 0) {
                uint32_t id;
                if (!alloc(max_blocks, &id)) return "internal inconsistency: no free block after the check";
                tables[row].push_back(id);
            }
            if (pos / block_size >= tables[row].size()) return "block table index out of range";
            const uint32_t blk = tables[row][pos / block_size];
            size_t slot;
            if (mul_overflows((size_t)blk, block_size, &slot) || __builtin_add_overflow(slot, pos % block_size, &slot) ||
                slot > std::numeric_limits<uint32_t>::max())
                return "slot number does not fit 32 bits";
            slots->push_back((uint32_t)slot);
        }
    }
    for (auto &len : seq_lens) len = s_total;
    return "";
}

std::string BlockTable::flatten_tables(size_t max_blocks_per_seq, std::vector<uint32_t> *out) const {
    out->clear();
    size_t n;
    if (mul_overflows(tables.size(), max_blocks_per_seq, &n)) return "block table size overflowed";
    try {
        out->reserve(n);
    } catch (const std::exception &) {
        return "out of host memory";
    }
    for (const auto &row : tables) {
        if (row.size() > max_blocks_per_seq) return "a row holds more blocks than max_blocks_per_seq";
        out->insert(out->end(), row.begin(), row.end());
        out->resize(out->size() + (max_blocks_per_seq - row.size()), std::numeric_limits<uint32_t>::max());
    }
    return "";
}

std::string BlockTable::rewind_to(size_t new_len, size_t block_size) {
    const size_t cur = seq_len();
    if (new_len > cur) return "rewind target exceeds the current length";
    if (!has_batch || new_len == cur) return "";
    if (new_len == 0) {
        reset();
        return "";
    }
    const size_t keep = div_ceil(new_len, block_size);
    size_t release = 0;
    for (const auto &t : tables) release += t.size() > keep ? t.size() - keep : 0;
    try {
        returned.reserve(returned.size() + release);
    } catch (const std::exception &) {
        return "out of host memory";
    }
    for (auto &row : tables) {
        while (row.size() > keep) {
            returned.push_back(row.back());
            row.pop_back();
        }
    }
    for (auto &len : seq_lens) len = new_len;
    return "";
}

std::string check_cache_config(size_t block_size, size_t max_blocks, size_t embed_dim, size_t elem_bytes) {
    if (block_size == 0 || block_size > 256 || (block_size & (block_size - 1)) != 0)
        return "block_size must be a power of two in 1..256";
    if (max_blocks == 0 || (uint64_t)max_blocks > (uint64_t)std::numeric_limits<uint32_t>::max())
        return "max_blocks must be in 1..UINT32_MAX";
    if (embed_dim == 0) return "embed_dim must be at least 1";
    size_t n;
    if (mul_overflows(max_blocks, block_size, &n) || mul_overflows(n, embed_dim, &n)) return "pool size overflows";
    if (mul_overflows(n, elem_bytes, &n) || mul_overflows(n, (size_t)2, &n) ||
        n > (size_t)std::numeric_limits<ptrdiff_t>::max())
        return "pool bytes exceed PTRDIFF_MAX";
    return "";
}

}  // namespace fa
