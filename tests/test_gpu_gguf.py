"""A LLaMA decoder filled from a GGUF file (galois_amd/host/gguf.cpp) against the same decoder filled tensor by tensor."""
import numpy as np
import pytest

from galois_amd import host_api as g
from tests import gguf_writer as gw
from tests.test_gguf import _llama_weights, _write

pytestmark = pytest.mark.gpu

HP = dict(n_vocab=512, n_embd=256, n_head=2, n_layer=2, n_ff=512, n_ctx=64, rms_eps=1e-6, freq_base=10000.0)


def _fill(dec, w):
    dec.tensor("tok_embd").write(w["tok_embd"])
    dec.tensor("output").write(w["output"] if w["output"] is not None else w["tok_embd"])
    dec.tensor("out_norm").write(w["out_norm"])
    for i, lw in enumerate(w["layers"]):
        for n, a in lw.items():
            dec.tensor(n, i).write(a)


@pytest.mark.parametrize("tied", [False, True])
@pytest.mark.parametrize("fused", [0, 3])
def test_decoder_from_gguf_matches_hand_filled(tmp_path, tied, fused):
    rng = np.random.default_rng(11)
    w = _llama_weights(rng, HP, tied=tied)
    dev = g.Device.gpu(0)
    ref = g.LlamaDecoder(dev, **HP)
    _fill(ref, w)
    with g.GgufFile(_write(tmp_path, gw.llama_file(HP, w))) as f:
        dec = g.LlamaDecoder.from_gguf(f, dev, n_ctx_max=2048)
    assert dec.hp["n_ctx"] == HP["n_ctx"] and dec.hp["n_vocab"] == HP["n_vocab"]
    # the file may be closed once the weights are on the device
    for name, layer in (("tok_embd", -1), ("out_norm", -1), ("wq", 0), ("w_down", 1), ("ffn_norm", 1)):
        np.testing.assert_array_equal(dec.tensor(name, layer).to_cpu_tensor(), ref.tensor(name, layer).to_cpu_tensor())
    for pos, tok in enumerate([3, 77, 500]):
        ref.decode(tok, pos, fused)
        dec.decode(tok, pos, fused)
        a, b = ref.logits(), dec.logits()
        assert np.isfinite(a).all()
        np.testing.assert_array_equal(a, b)
    ref.close()
    dec.close()


def test_files_the_decoder_cannot_hold_are_refused(tmp_path):
    rng = np.random.default_rng(12)
    w = _llama_weights(rng, HP)
    dev = g.Device.gpu(0)
    e, v = HP["n_embd"], HP["n_vocab"]
    md = [("general.architecture", gw.STRING, "llama"), ("llama.block_count", gw.U32, 1),
          ("llama.embedding_length", gw.U32, e), ("llama.feed_forward_length", gw.U32, HP["n_ff"]),
          ("llama.attention.head_count", gw.U32, HP["n_head"])]
    base = [("token_embd.weight", (e, v), gw.GGML_Q4_0, w["tok_embd"]),
            ("output_norm.weight", (e,), gw.GGML_F32, w["out_norm"])]
    build = gw.build
    # output.weight stored as Q6_K (what "mostly Q4_0" files do): refused with Unimplemented
    q6k = ("output.weight", (e, v), gw.GGML_Q6_K, bytes(e * v // 256 * 210))
    with g.GgufFile(_write(tmp_path, build(md, base + [q6k]))) as f:
        with pytest.raises(g.GError) as err:
            g.LlamaDecoder.from_gguf(f, dev)
        assert err.value.kind == "Unimplemented"
    # a layer tensor is missing
    with g.GgufFile(_write(tmp_path, build(md, base))) as f:
        with pytest.raises(g.GError) as err:
            g.LlamaDecoder.from_gguf(f, dev)
        assert err.value.kind == "ShapeError" and "blk.0.attn_norm.weight" in str(err.value)
    # a norm with the wrong length
    bad_norm = [base[0], ("output_norm.weight", (e // 2,), gw.GGML_F32, w["out_norm"][:e // 2])]
    with g.GgufFile(_write(tmp_path, build(md, bad_norm))) as f:
        with pytest.raises(g.GError) as err:
            g.LlamaDecoder.from_gguf(f, dev)
        assert err.value.kind == "ShapeError"
