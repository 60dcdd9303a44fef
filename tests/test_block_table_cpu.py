"""Host logic of the paged KV cache: the block table behind ``fa_block_table_*`` against the
reference's own unit vectors and against the oracle restatement on random operation sequences.
No device is needed: the table is plain host bookkeeping.
"""
import os
import random
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
import block_table as ob  # noqa: E402

import fandhe_ai_amd as fa  # noqa: E402
from fandhe_ai_amd import capi  # noqa: E402
from fandhe_ai_amd.paged_cache import BlockTable, PagedKvCacheConfig  # noqa: E402

U32MAX = 0xFFFFFFFF
USIZE_MAX = (1 << 64) - 1
ISIZE_MAX = (1 << 63) - 1


def _both_config(block_size, max_blocks, embed_dim):
    try:
        ob.check_config(block_size, max_blocks, embed_dim)
        oracle_ok = True
    except ob.TableError:
        oracle_ok = False
    try:
        PagedKvCacheConfig.new(block_size, max_blocks, embed_dim)
        ours_ok = True
    except fa.InvalidArgument:
        ours_ok = False
    assert oracle_ok == ours_ok, (block_size, max_blocks, embed_dim)
    return ours_ok


def test_config_rejects_bad_block_size_and_overflow():
    # crates/autodiff/src/nn/paged_kv.rs:833-849
    assert not _both_config(0, 4, 8)
    assert not _both_config(3, 4, 8)
    assert not _both_config(512, 4, 8)
    assert _both_config(256, 4, 8)
    assert not _both_config(4, 0, 8)
    assert not _both_config(4, 4, 0)
    assert not _both_config(256, U32MAX, USIZE_MAX // 4)
    assert not _both_config(256, 1, ISIZE_MAX // (2 * 4 * 256) + 1)
    assert _both_config(256, 1, ISIZE_MAX // (2 * 4 * 256))
    assert not _both_config(4, U32MAX + 1, 1)
    assert _both_config(1, U32MAX, 1)


def test_block_table_alloc_order_is_deterministic():
    # crates/autodiff/src/nn/paged_kv.rs:851-860
    for t in (BlockTable(), ob.BlockTable()):
        assert t.alloc(3) == 0
        assert t.alloc(3) == 1
        if isinstance(t, BlockTable):
            t.push_returned(0)
        else:
            t.returned.append(0)
        assert t.free_blocks(3) == 2
        assert t.alloc(3) == 0
        assert t.alloc(3) == 2
        assert t.alloc(3) is None


@pytest.mark.parametrize("length,blocks", [(1, 1), (3, 1), (4, 1), (5, 2), (13, 4)])
def test_ceil_boundaries_use_expected_block_counts(length, blocks):
    # crates/autodiff/src/nn/paged_kv.rs:862-873 (block_size 4, max_blocks 8)
    for t in (BlockTable(), ob.BlockTable()):
        t.extend_for_append(8, 4, 1, length)
        assert t.used_blocks() == blocks
        assert t.seq_len() == length


def test_slot_mappings_of_the_reference_cache_tests():
    # crates/autodiff/src/nn/paged_kv_device.rs:619-637: block_size 2, max_blocks 3
    for t in (BlockTable(), ob.BlockTable()):
        err = fa.InvalidArgument if isinstance(t, BlockTable) else ob.TableError
        with pytest.raises(err):
            t.clone().extend_for_append(3, 2, 2, 3)            # needs 4 blocks, 3 free
        assert list(t.extend_for_append(3, 2, 1, 3)) == [0, 1, 2]
        assert t.seq_len() == 3 and t.used_blocks() == 2
        assert list(t.extend_for_append(3, 2, 1, 2)) == [3, 4]
        assert t.free_blocks(3) == 0
        # paged_kv_device.rs:745-765: rewind, last-in-first-out reuse, clear
        with pytest.raises(err):
            t.rewind_to(6, 2)
        assert t.seq_len() == 5
        t.rewind_to(2, 2)
        assert (t.seq_len(), t.used_blocks(), t.free_blocks(3)) == (2, 1, 2)
        assert list(t.extend_for_append(3, 2, 1, 1)) == [2]     # blocks came back as 2, 1: block 1 first
        t.rewind_to(0, 2)
        assert t.batch is None
        t.reset()
        assert t.free_blocks(3) == 3 and t.seq_len() == 0


def test_failed_calls_leave_the_table_unchanged():
    t = BlockTable()
    t.extend_for_append(4, 2, 2, 3)
    before = (t.seq_len(), t.batch, t.used_blocks(), t.free_blocks(4), list(t.flatten_tables(2)))
    with pytest.raises(fa.InvalidArgument):
        t.extend_for_append(4, 2, 3, 1)                          # batch mismatch
    with pytest.raises(fa.InvalidArgument):
        t.extend_for_append(4, 2, 2, 2)                          # needs 2 more blocks, none free
    with pytest.raises(fa.InvalidArgument):
        t.extend_for_append(4, 2, 0, 1)                          # batch 0
    with pytest.raises(fa.InvalidArgument):
        t.rewind_to(4, 2)
    with pytest.raises(fa.InvalidArgument):
        t.flatten_tables(1)                                      # rows hold 2 blocks
    with pytest.raises(fa.InvalidArgument):
        t.extend_for_append(4, 2, 2, USIZE_MAX)                  # length overflow
    assert before == (t.seq_len(), t.batch, t.used_blocks(), t.free_blocks(4), list(t.flatten_tables(2)))
    assert list(t.extend_for_append(4, 2, 2, 0)) == []           # validated, nothing changes
    assert list(t.extend_for_append(4, 2, 2, 1)) == [3, 7]       # row 0: blocks 0,1; row 1: blocks 2,3
    # an empty append on an empty table does not fix the batch (paged_kv.rs:224-226)
    e = BlockTable()
    assert list(e.extend_for_append(4, 2, 5, 0)) == []
    assert e.batch is None


def test_flatten_pads_with_the_sentinel():
    t = BlockTable()
    assert list(t.flatten_tables(3)) == []
    t.extend_for_append(16, 4, 3, 5)
    flat = np.array(t.flatten_tables(4)).reshape(3, 4)
    assert flat[:, :2].tolist() == [[0, 1], [2, 3], [4, 5]]
    assert (flat[:, 2:] == U32MAX).all()


def test_clone_is_independent():
    t = BlockTable()
    t.extend_for_append(8, 2, 1, 3)
    c = t.clone()
    c.extend_for_append(8, 2, 1, 4)
    assert (t.seq_len(), t.used_blocks()) == (3, 2)
    assert (c.seq_len(), c.used_blocks()) == (7, 4)


def _state(t, max_blocks, width):
    try:
        flat = list(t.flatten_tables(width))
    except (fa.InvalidArgument, ob.TableError):
        flat = "too narrow"
    return (t.seq_len(), t.batch, t.used_blocks(), t.free_blocks(max_blocks), flat)


@pytest.mark.parametrize("seed", range(12))
def test_random_operation_sequences_match_the_oracle(seed):
    rng = random.Random(seed)
    block_size = rng.choice([1, 2, 4, 16])
    max_blocks = rng.randint(1, 40)
    ours, ref = BlockTable(), ob.BlockTable()
    for step in range(300):
        op = rng.random()
        if op < 0.55:
            b = ref.batch if (ref.batch is not None and rng.random() < 0.9) else rng.randint(0, 4)
            l_new = rng.choice([0, 1, 1, 1, 2, 3, block_size, block_size + 1, 7])
            try:
                want = ref.clone().extend_for_append(max_blocks, block_size, b, l_new)
                ref.extend_for_append(max_blocks, block_size, b, l_new)
            except ob.TableError:
                want = None
            if want is None:
                with pytest.raises(fa.InvalidArgument):
                    ours.extend_for_append(max_blocks, block_size, b, l_new)
            else:
                assert list(ours.extend_for_append(max_blocks, block_size, b, l_new)) == want, (seed, step)
        elif op < 0.85:
            new_len = rng.randint(0, ref.seq_len() + 1)
            try:
                ref.clone().rewind_to(new_len, block_size)
                ref.rewind_to(new_len, block_size)
                ours.rewind_to(new_len, block_size)
            except ob.TableError:
                with pytest.raises(fa.InvalidArgument):
                    ours.rewind_to(new_len, block_size)
        elif op < 0.9:
            ref.reset()
            ours.reset()
        else:
            snap_o, snap_r = ours.clone(), ref.clone()
            assert _state(snap_o, max_blocks, 64) == _state(snap_r, max_blocks, 64)
        width = rng.randint(0, 48)
        assert _state(ours, max_blocks, width) == _state(ref, max_blocks, width), (seed, step)


def test_invalid_handles_are_rejected():
    st = capi.BlockTableState()
    assert capi.lib.fa_block_table_state_get(None, 0, st) != 0
    assert capi.lib.fa_paged_cache_clear(None) != 0
