"""Oracle: page-table and free-block bookkeeping of the paged KV cache.

TEST INFRASTRUCTURE ONLY.  This is a CPU restatement of the reference's host logic, written to be
read next to it; only tests, the smoke check and the benchmark's CPU leg may import it.  The shipped
implementation is the C++ one behind ``fa_block_table_*`` / ``fa_paged_cache_*``.

Follows crates/autodiff/src/nn/paged_kv.rs:
  config check            79-108 (+ the byte bound 127-145)
  free_blocks / alloc     168-183
  reset                   185-191
  seq_len                 196-198
  extend_for_append       208-300
  flatten_tables          304-324
  rewind_to               328-363
and the cache-level composition of crates/autodiff/src/nn/paged_kv_device.rs:187-253 (append on a
copy, commit after the write), 262-345 (attention arguments), 350-372 (rewind / snapshot / clear).

Pinned by the reference's own unit vectors (paged_kv.rs:851-873, paged_kv_device.rs:619-637,
745-765, 805-822) in tests/test_block_table_cpu.py.
"""
U32_MAX = 0xFFFFFFFF
USIZE_MAX = (1 << 64) - 1
ISIZE_MAX = (1 << 63) - 1
MAX_BLOCK_SIZE = 256


class TableError(ValueError):
    pass


def check_config(block_size, max_blocks, embed_dim, elem_bytes=4):
    """paged_kv.rs:79-108 and 127-145: raises TableError for a rejected configuration."""
    if block_size == 0 or block_size > MAX_BLOCK_SIZE or block_size & (block_size - 1):
        raise TableError("block_size must be a power of two in 1..=256")
    if max_blocks == 0 or max_blocks > U32_MAX:
        raise TableError("max_blocks must be in 1..=u32::MAX")
    if embed_dim == 0:
        raise TableError("embed_dim must be at least 1")
    total = max_blocks * block_size * embed_dim * elem_bytes * 2
    # every partial product is a checked usize multiplication in the reference
    if max_blocks * block_size > USIZE_MAX or max_blocks * block_size * embed_dim > USIZE_MAX or total > ISIZE_MAX:
        raise TableError("pool bytes exceed isize::MAX")


def ceil_div(a, b):
    return -(-a // b)


class BlockTable:
    def __init__(self):
        self.returned, self.next_unused, self.tables, self.seq_lens, self.batch = [], 0, [], [], None

    def clone(self):
        c = BlockTable()
        c.returned, c.next_unused = list(self.returned), self.next_unused
        c.tables, c.seq_lens, c.batch = [list(r) for r in self.tables], list(self.seq_lens), self.batch
        return c

    def free_blocks(self, max_blocks):
        return len(self.returned) + max(0, max_blocks - self.next_unused)

    def alloc(self, max_blocks):
        if self.returned:
            return self.returned.pop()
        if self.next_unused < max_blocks:
            if self.next_unused > U32_MAX:
                return None
            self.next_unused += 1
            return self.next_unused - 1
        return None

    def reset(self):
        self.__init__()

    def seq_len(self):
        return self.seq_lens[0] if self.seq_lens else 0

    def used_blocks(self):
        return sum(len(r) for r in self.tables)

    def extend_for_append(self, max_blocks, block_size, b, l_new):
        """Mutates self; callers apply it to a clone and commit on success."""
        if b == 0:
            raise TableError("batch 0 cannot be appended")
        if self.batch is not None and self.batch != b:
            raise TableError("batch does not match the cache")
        if l_new == 0:
            return []
        s_prev = self.seq_len()
        s_total = s_prev + l_new
        if s_total > USIZE_MAX:
            raise TableError("sequence length overflows")
        extra_per_row = ceil_div(s_total, block_size) - ceil_div(s_prev, block_size)
        extra_total = extra_per_row * b
        if extra_total > USIZE_MAX:
            raise TableError("block count overflows")
        if extra_total > self.free_blocks(max_blocks):
            raise TableError("not enough free blocks")
        if b * l_new > USIZE_MAX:
            raise TableError("row count overflows")
        if self.batch is None:
            self.tables, self.seq_lens, self.batch = [[] for _ in range(b)], [0] * b, b
        slots = []
        for row in range(b):
            for i in range(l_new):
                pos = s_prev + i
                if pos % block_size == 0:
                    bid = self.alloc(max_blocks)
                    if bid is None:
                        raise TableError("no free block after the check passed")
                    self.tables[row].append(bid)
                slot = self.tables[row][pos // block_size] * block_size + pos % block_size
                if slot > U32_MAX:
                    raise TableError("slot does not fit 32 bits")
                slots.append(slot)
        self.seq_lens = [s_total] * len(self.seq_lens)
        return slots

    def flatten_tables(self, max_blocks_per_seq):
        out = []
        for row in self.tables:
            if len(row) > max_blocks_per_seq:
                raise TableError("row holds more blocks than max_blocks_per_seq")
            out.extend(row)
            out.extend([U32_MAX] * (max_blocks_per_seq - len(row)))
        return out

    def rewind_to(self, new_len, block_size):
        cur = self.seq_len()
        if new_len > cur:
            raise TableError("rewind target beyond the cached length")
        if self.batch is None or new_len == cur:
            return
        if new_len == 0:
            self.reset()
            return
        keep = ceil_div(new_len, block_size)
        for row in self.tables:
            while len(row) > keep:
                self.returned.append(row.pop())
        self.seq_lens = [new_len] * len(self.seq_lens)
