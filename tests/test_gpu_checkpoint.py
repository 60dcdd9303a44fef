"""A decoder loaded from a Llama-named safetensors checkpoint (weights stored [out, in], float) against a
decoder assembled by hand from the same weights: transposed and concatenated on the host, quantized per output
channel by the oracle, imported as codes.  The device quantizer is bit-exact against the oracle's, so both
decoders hold identical weights and their logits must be identical bit for bit, for a prompt pass and for
decode steps.  Also: the flat parameter store returns every tensor as it was stored."""
import numpy as np
import pytest
from safetensors.numpy import save as st_save

import oracle_lib as o
from decoder_common import llama_checkpoint as _checkpoint
from gpu_common import ops

pytestmark = pytest.mark.gpu


def test_loaded_decoder_equals_hand_built_decoder(tmp_path):
    import fandhe_ai_amd as fa
    be = ops()
    L, d, heads, kv, f, vocab, batch, l_new = 2, 256, 2, 1, 512, 320, 3, 21
    t = _checkpoint(5, L, d, heads, kv, f, vocab)
    path = str(tmp_path / "model.safetensors")
    with open(path, "wb") as fh:
        fh.write(st_save(t, metadata={"format": "pt"}))
    geometry = dict(max_blocks_per_seq=4, num_blocks=16, max_batch=batch)
    loaded, store = fa.safetensors_io.load_decoder(be, path, L, heads, kv, **geometry)

    # the store returns what was stored (explicitly transposed, fused projections side by side)
    p0 = "model.layers.0."
    wqkv = np.concatenate([t[p0 + "self_attn.%s_proj.weight" % n].T for n in "qkv"], axis=1)
    v = store.view("layers.0.wqkv")
    assert v.shape == wqkv.shape and v.offset % 64 == 0
    assert np.array_equal(be.download(store.buffer, v.offset, wqkv.size).reshape(wqkv.shape), wqkv)
    v = store.view("lm_head")
    assert np.array_equal(be.download(store.buffer, v.offset, vocab * d).reshape(d, vocab), t["lm_head.weight"].T)
    store.free()                                           # the decoder owns copies of all it needs

    hand = fa.Decoder(be, L, d, heads, kv, f, vocab, **geometry)

    def q(wt):                                             # [k, n] float -> imported int8 weight
        codes, scales = o.quantize_cols_i8(np.ascontiguousarray(wt, dtype=np.float32))
        return be.import_quantized_weight(codes, scales)

    for i in range(L):
        p = "model.layers.%d." % i
        hand.set_layer(i, be.upload(t[p + "input_layernorm.weight"]), be.upload(t[p + "post_attention_layernorm.weight"]),
                       q(np.concatenate([t[p + "self_attn.%s_proj.weight" % n].T for n in "qkv"], axis=1)),
                       q(t[p + "self_attn.o_proj.weight"].T),
                       q(np.concatenate([t[p + "mlp.gate_proj.weight"].T, t[p + "mlp.up_proj.weight"].T], axis=1)),
                       q(t[p + "mlp.down_proj.weight"].T))
    hand.set_head(be.upload(t["model.embed_tokens.weight"]), be.upload(t["model.norm.weight"]), q(t["lm_head.weight"].T))

    tables = np.arange(batch * 4, dtype=np.uint32).reshape(batch, 4)
    prompt = np.random.default_rng(9).integers(0, vocab, (batch, l_new)).astype(np.int32)
    outs = []
    for dec in (loaded, hand):
        dec.set_sequences(tables, np.zeros(batch, np.uint32))
        dec.prefill(prompt)
        seen = [dec.logits().copy(), dec.tokens().copy()]
        for _ in range(3):
            dec.step()
            seen += [dec.logits().copy(), dec.tokens().copy()]
        assert dec.seq_lens().tolist() == [l_new + 3] * batch
        outs.append(seen)
    for a, b in zip(*outs):
        assert np.isfinite(a).all() and a.tobytes() == b.tobytes()
    spread = outs[0][0].max() - outs[0][0].min()
    assert spread > 1.0                                    # a live model, not all-zero logits
    loaded.close()
    hand.close()


def test_checkpoint_shape_and_key_errors_surface_before_device_work():
    import fandhe_ai_amd as fa
    st = fa.safetensors_io
    be = ops()
    t = _checkpoint(6, 1, 256, 2, 1, 512, 64)
    with pytest.raises(st.SafetensorsFormat):              # wrong head count for these projections
        st.load_decoder(be, st_save(t), 1, 4, 1, max_blocks_per_seq=2, num_blocks=4, max_batch=1)
    del t["model.layers.0.mlp.down_proj.weight"]
    with pytest.raises(st.MissingKeys) as e:
        st.load_decoder(be, st_save(t), 1, 2, 1, max_blocks_per_seq=2, num_blocks=4, max_batch=1)
    assert e.value.keys == ["model.layers.0.mlp.down_proj.weight"]
    t16 = {k: a.astype(np.float16) for k, a in _checkpoint(6, 1, 256, 2, 1, 512, 64).items()}
    dec, store = st.load_decoder(be, st_save(t16), 1, 2, 1, max_blocks_per_seq=2, num_blocks=4, max_batch=1)
    dec.set_sequences(np.array([[0, 1]], np.uint32), np.zeros(1, np.uint32))
    dec.set_tokens(np.array([3], np.int32))
    dec.step()
    assert np.isfinite(dec.logits()).all()
    dec.close()
    store.free()
