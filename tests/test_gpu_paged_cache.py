"""GPU tests of the device-resident paged KV cache (``fa_paged_cache_*``): the reference's own cache
tests (crates/autodiff/src/nn/paged_kv_device.rs:619-822) replayed against the real device, and
multi-step append -> attention runs checked against the oracle (block table restatement + paged
append / attention restatements) with rewinds, clears and snapshots in between.
"""
import os
import sys

import numpy as np
import pytest

import oracle_lib as o
from gpu_common import assert_parity, ops

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
import block_table as ob  # noqa: E402

pytestmark = pytest.mark.gpu
U32MAX = 0xFFFFFFFF


def _fa():
    import fandhe_ai_amd as fa
    return fa


def _x(b, l, e=4):
    return np.full((b, l, e), 0.5, np.float32)


def _cache(block_size=2, max_blocks=3, embed=4, dtype=None):
    fa = _fa()
    cfg = fa.PagedKvCacheConfig.new(block_size, max_blocks, embed, fa.capi.F32 if dtype is None else dtype)
    return fa.PagedKvCache.new(ops(), cfg)


def _written_slots(cache, value=0.5):
    k, v = cache.pools()
    assert np.array_equal(k, v)
    rows = k.reshape(-1, k.shape[-1])
    return [int(i) for i in np.nonzero((rows == value).all(axis=1))[0]]


def test_append_builds_row_major_slot_mapping_and_commits():
    fa = _fa()
    c = _cache()
    with pytest.raises(fa.InvalidArgument):
        c.append(_x(2, 3), _x(2, 3))                       # needs 4 blocks, 3 free
    assert c.seq_len() == 0 and c.batch() is None
    c.append(_x(1, 3), _x(1, 3))
    assert (c.seq_len(), c.num_used_blocks()) == (3, 2)
    assert _written_slots(c) == [0, 1, 2]
    c.append(_x(1, 2), _x(1, 2))
    assert _written_slots(c) == [0, 1, 2, 3, 4]
    assert c.num_free_blocks() == 0
    assert c.block_tables(3).tolist() == [[0, 1, 2]]
    c.close()


def test_append_rejects_bad_shapes_without_state_change():
    fa = _fa()
    c = _cache()
    with pytest.raises(fa.InvalidArgument):
        c.append(np.zeros((1, 2, 3), np.float32), np.zeros((1, 2, 3), np.float32))
    with pytest.raises(fa.InvalidArgument):
        c.append(np.zeros((1, 4), np.float32), np.zeros((1, 4), np.float32))
    with pytest.raises(fa.InvalidArgument):
        c.append(_x(1, 2), _x(1, 1))
    assert c.seq_len() == 0
    c.append(_x(1, 1), _x(1, 1))
    with pytest.raises(fa.InvalidArgument):
        c.append(_x(2, 1), _x(2, 1))                       # batch mismatch
    assert c.seq_len() == 1
    c.append(_x(1, 0), _x(1, 0))                           # empty append: validated only
    assert c.seq_len() == 1
    assert not c.is_poisoned()
    c.close()


def test_attention_flattens_tables_and_validates_inputs():
    fa = _fa()
    c = _cache()
    c.append(_x(1, 3), _x(1, 3))
    out = c.attention(_x(1, 3), 2, 0.5)
    assert out.shape == (1, 3, 4)
    assert np.allclose(out, 0.5)                           # all values equal: any softmax average gives 0.5
    c.rewind_to(2)
    with pytest.raises(fa.InvalidArgument):
        c.attention(_x(1, 3), 2, 1.0)                      # L_new beyond the cached length
    with pytest.raises(fa.InvalidArgument):
        c.attention(_x(1, 1), 3, 1.0)
    with pytest.raises(fa.InvalidArgument):
        c.attention(_x(1, 1), 2, float("nan"))
    with pytest.raises(fa.InvalidArgument):
        c.attention(_x(2, 1), 2, 1.0)                      # batch mismatch
    assert c.attention(_x(1, 0), 2, 1.0).shape == (1, 0, 4)
    for heads, scale in ((0, 1.0), (3, 1.0), (2, float("nan"))):
        with pytest.raises(fa.InvalidArgument):
            c.attention(_x(1, 0), heads, scale)            # the empty call keeps the argument contract
    assert not c.is_poisoned()
    c.close()


def test_rewind_and_clear_follow_reference_semantics():
    fa = _fa()
    c = _cache()
    c.append(_x(1, 5), _x(1, 5))
    assert c.num_free_blocks() == 0
    with pytest.raises(fa.InvalidArgument):
        c.rewind_to(6)
    assert c.seq_len() == 5
    c.rewind_to(2)
    assert (c.seq_len(), c.num_used_blocks(), c.num_free_blocks()) == (2, 1, 2)
    c.append(np.full((1, 1, 4), 0.25, np.float32), np.full((1, 1, 4), 0.25, np.float32))
    assert _written_slots(c, 0.25) == [2]                  # returned 2 then 1; block 1 is taken first
    c.rewind_to(0)
    assert c.batch() is None
    c.clear()
    assert (c.num_free_blocks(), c.seq_len()) == (3, 0)
    c.close()


def test_snapshot_restore_undoes_boundary_crossing_append():
    c = _cache()
    c.append(_x(1, 1), _x(1, 1))
    before = (c.seq_len(), c.num_used_blocks(), c.num_free_blocks())
    saved = c.snapshot_table()
    c.append(_x(1, 3), _x(1, 3))
    assert c.num_used_blocks() > before[1]
    c.restore_table(saved)
    assert (c.seq_len(), c.num_used_blocks(), c.num_free_blocks()) == before
    assert not c.is_poisoned()
    c.close()


def test_configs_whose_slots_exceed_32_bits_are_rejected():
    fa = _fa()
    cfg = fa.PagedKvCacheConfig.new(256, U32MAX // 2, 1)
    with pytest.raises(fa.InvalidArgument):
        fa.PagedKvCache.new(ops(), cfg)


def _run_script(cache, dtype_is_bf16, block_size, max_blocks, e_kv, heads, kv_heads, script, seed):
    """script: list of ("append", batch, l_new) / ("rewind", new_len) / ("clear",) / ("snapshot",) /
    ("restore",).  Every append is followed by attention over the appended positions."""
    fa = _fa()
    rng = o.Rng(seed)
    table, saved = ob.BlockTable(), None
    dh = e_kv // (kv_heads or heads)
    e_q = heads * dh
    np_dt = np.uint16 if dtype_is_bf16 else np.float32
    hk = np.zeros((max_blocks * block_size, e_kv), np_dt)
    hv = np.zeros_like(hk)
    cast = o.to_bf16 if dtype_is_bf16 else (lambda a: a)
    layout = o.PagedLayout(max_blocks, block_size, e_kv)
    scale = fa.default_scale(dh)
    for si, step in enumerate(script):
        if step[0] == "append":
            _, b, l_new = step
            k, v = cast(rng.randn((b, l_new, e_kv))), cast(rng.randn((b, l_new, e_kv)))
            q = cast(rng.randn((b, l_new, e_q)))
            nxt = table.clone()
            try:
                slots = nxt.extend_for_append(max_blocks, block_size, b, l_new)
            except ob.TableError:
                with pytest.raises(fa.InvalidArgument):
                    cache.append(k, v)
                continue
            cache.append(k, v)
            table = nxt
            assert o.paged_kv_append(k.reshape(-1, e_kv), v.reshape(-1, e_kv), hk, hv, slots, layout) == 0
            width = max(1, max(len(r) for r in table.tables))
            tables = np.array(table.flatten_tables(width), dtype=np.uint32).reshape(b, width)
            assert np.array_equal(cache.block_tables(width), tables)
            lens = np.full(b, table.seq_len(), np.uint32)
            oargs = o.paged_args(max_blocks, block_size, e_kv, b, l_new, heads, width, scale, kv_heads)
            pools = (hk.reshape(max_blocks, block_size, e_kv), hv.reshape(max_blocks, block_size, e_kv))
            if dtype_is_bf16:
                rc, want = o.paged_attention_bf16(q, pools[0], pools[1], tables, lens, oargs)
            else:
                rc, want = o.paged_attention_f32(q, pools[0], pools[1], tables, lens, oargs)
            assert rc == 0
            got = cache.attention(q, heads, scale, kv_heads, out_dtype=fa.capi.F32)
            assert_parity("PAGED_CACHE_PARITY", f"seed{seed}:step{si}:{step}", got, want)
        elif step[0] == "rewind":
            try:
                table.clone().rewind_to(step[1], block_size)
                table.rewind_to(step[1], block_size)
                cache.rewind_to(step[1])
            except ob.TableError:
                with pytest.raises(fa.InvalidArgument):
                    cache.rewind_to(step[1])
        elif step[0] == "clear":
            table.reset()
            cache.clear()
        elif step[0] == "snapshot":
            saved = (table.clone(), cache.snapshot_table())
        elif step[0] == "restore":
            table = saved[0].clone()
            cache.restore_table(saved[1])
        assert (cache.seq_len(), cache.batch(), cache.num_used_blocks(), cache.num_free_blocks()) == \
            (table.seq_len(), table.batch, table.used_blocks(), table.free_blocks(max_blocks))
    gk, gv = cache.pools()
    assert np.array_equal(gk.reshape(hk.shape), hk) and np.array_equal(gv.reshape(hv.shape), hv)
    assert not cache.is_poisoned()


SCRIPT_A = [("append", 2, 5), ("append", 2, 1), ("append", 2, 1), ("snapshot",), ("append", 2, 4), ("restore",),
            ("append", 2, 3), ("rewind", 4), ("append", 2, 1), ("append", 2, 7), ("append", 3, 1), ("rewind", 99),
            ("append", 2, 200), ("clear",), ("append", 3, 2), ("append", 3, 1), ("rewind", 0), ("append", 1, 9)]


@pytest.mark.parametrize("block_size,embed,heads", [(1, 8, 2), (4, 16, 2), (16, 48, 3), (256, 16, 4)])
def test_f32_cache_runs_match_the_oracle(block_size, embed, heads):
    max_blocks = max(3, 3 * ((24 + block_size - 1) // block_size) + 2)
    c = _cache(block_size, max_blocks, embed)
    _run_script(c, False, block_size, max_blocks, embed, heads, 0, SCRIPT_A, seed=block_size)
    c.close()


@pytest.mark.parametrize("heads,kv_heads", [(32, 8), (8, 2), (4, 4)])
def test_bf16_grouped_query_cache_runs_match_the_oracle(heads, kv_heads):
    """Page 16, head_dim 128: single-token appends take the decode form of the streaming kernel, longer ones
    its prefill form."""
    fa = _fa()
    e_kv, max_blocks = kv_heads * 128, 64
    c = _cache(16, max_blocks, e_kv, fa.capi.BF16)
    script = [("append", 3, 37)] + [("append", 3, 1)] * 12 + [("rewind", 20), ("append", 3, 1), ("append", 3, 2),
                                                             ("snapshot",), ("append", 3, 60), ("restore",),
                                                             ("append", 3, 1), ("clear",), ("append", 5, 1),
                                                             ("append", 5, 1), ("append", 5, 150)]
    _run_script(c, True, 16, max_blocks, e_kv, heads, kv_heads, script, seed=heads)
    c.close()


def test_cache_of_another_context_is_rejected():
    fa = _fa()
    other = fa.tape_for(fa.Device.Rocm(0))
    c = _cache()
    k = other.upload(_x(1, 1))
    with pytest.raises(fa.DeviceMismatch):
        fa.check(fa.capi.lib.fa_paged_cache_append(other._ctx, c._h, k._h, k._h, 1, 1))
    assert c.seq_len() == 0 and not c.is_poisoned()
    c.close()
