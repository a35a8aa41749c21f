"""GGUF reader (galois_amd/host/gguf.cpp) against files packed by tests/gguf_writer.py: metadata of every type,
tensor table, data offsets, tensors through Tensor::from_raw on the Cpu device, llama hyper-parameters, and
malformed files (every truncation point, bad magic / version / counts / offsets), which must raise, never crash."""
import struct

import numpy as np
import pytest

from galois_amd import host_api as g
from tests import gguf_writer as gw


def _write(tmp_path, data, name="m.gguf"):
    p = tmp_path / name
    p.write_bytes(data)
    return str(p)


def _q4(rng, rows, cols):
    """Random Q4_0 block bytes for a [cols, rows] tensor (finite f16 scale, random nibbles)."""
    blk = rng.integers(0, 256, (rows * cols // 32, 18), dtype=np.uint8)
    blk[:, 0], blk[:, 1] = 0x66, 0x1E
    return blk.reshape(-1)


METADATA = [("a.u8", gw.U8, 200), ("a.i8", gw.I8, -100), ("a.u16", gw.U16, 60000), ("a.i16", gw.I16, -30000),
            ("a.u32", gw.U32, 4000000000), ("a.i32", gw.I32, -2000000000), ("a.f32", gw.F32, 0.5),
            ("a.bool", gw.BOOL, 1), ("a.str", gw.STRING, "héllo wörld"), ("a.u64", gw.U64, 1 << 40),
            ("a.i64", gw.I64, -(1 << 40)), ("a.f64", gw.F64, 1e-300),
            ("a.ints", gw.ARRAY, (gw.I32, [1, -2, 3])), ("a.strs", gw.ARRAY, (gw.STRING, ["x", "", "long token"])),
            ("a.empty", gw.STRING, "")]


@pytest.mark.parametrize("version,alignment", [(3, None), (2, None), (3, 64), (3, 8)])
def test_metadata_and_tensor_table(tmp_path, version, alignment):
    rng = np.random.default_rng(1)
    f32 = rng.standard_normal((3, 5)).astype(np.float32)            # ggml shape (5, 3)
    f16 = rng.standard_normal(7).astype(np.float16)
    q4 = _q4(rng, 4, 64)                                            # ggml shape (64, 4)
    data = gw.build(METADATA, [("t.f32", (5, 3), gw.GGML_F32, f32), ("t.f16", (7,), gw.GGML_F16, f16),
                               ("t.q4", (64, 4), gw.GGML_Q4_0, q4), ("t.q6k", (256, 2), gw.GGML_Q6_K, bytes(420))],
                    version=version, alignment=alignment)
    with g.GgufFile(_write(tmp_path, data)) as f:
        al = alignment or 32
        assert f.version == version and f.alignment == al and f.data_start % al == 0
        assert f.n_kv == len(METADATA) + (alignment is not None)
        assert f.get_uint("a.u8") == 200 and f.get_uint("a.u16") == 60000 and f.get_uint("a.u32") == 4000000000
        assert f.get_uint("a.u64") == 1 << 40 and f.get_uint("a.bool") == 1
        assert f.get_uint("a.i8") is None and f.get_uint("a.i64") is None        # negative: not an unsigned value
        assert f.get_uint("a.f32") is None and f.get_uint("missing") is None
        assert f.get_float("a.f32") == 0.5 and f.get_float("a.f64") == 1e-300 and f.get_float("a.u8") is None
        assert f.get_string("a.str") == "héllo wörld" and f.get_string("a.empty") == "" and f.get_string("a.u8") is None
        assert f.get_string_array("a.strs") == ["x", "", "long token"]
        assert f.get_string_array("a.ints") is None and f.get_string_array("missing") is None
        ts = {t["name"]: t for t in f.tensors()}
        assert list(ts) == ["t.f32", "t.f16", "t.q4", "t.q6k"]
        assert ts["t.f32"]["shape"] == (5, 3) and ts["t.f32"]["nbytes"] == 60 and ts["t.f32"]["supported"]
        assert ts["t.f16"]["shape"] == (7,) and ts["t.f16"]["nbytes"] == 14
        assert ts["t.q4"]["shape"] == (64, 4) and ts["t.q4"]["nbytes"] == 8 * 18 and ts["t.q4"]["ggml_type"] == 2
        assert ts["t.q6k"]["nbytes"] == 420 and not ts["t.q6k"]["supported"]
        assert all(t["offset"] % al == 0 for t in ts.values())
        # the bytes at data_start + offset are the tensor's bytes
        for name, ref in (("t.f32", f32), ("t.f16", f16), ("t.q4", q4)):
            o = f.data_start + ts[name]["offset"]
            assert data[o:o + ts[name]["nbytes"]] == ref.tobytes()
        cpu = g.Device.cpu()
        np.testing.assert_array_equal(f.load_tensor("t.f32", cpu).to_cpu_tensor(), f32)
        np.testing.assert_array_equal(f.load_tensor("t.f16", cpu).to_cpu_tensor().reshape(-1), f16)
        np.testing.assert_array_equal(f.load_tensor("t.q4", cpu).to_cpu_tensor(), q4)
        with pytest.raises(g.GError) as e:
            f.load_tensor("t.q6k", cpu)
        assert e.value.kind == "Unimplemented"
        with pytest.raises(g.GError):
            f.load_tensor("nope", cpu)


def test_every_truncation_is_an_error(tmp_path):
    rng = np.random.default_rng(2)
    data = gw.build(METADATA[:9] + [METADATA[13]], [("t.f32", (4, 2), gw.GGML_F32, rng.standard_normal(8).astype(np.float32)),
                                                    ("t.q4", (32, 1), gw.GGML_Q4_0, _q4(rng, 1, 32))])
    with g.GgufFile(_write(tmp_path, data)) as f:
        assert len(f.tensors()) == 2
    for n in range(len(data)):
        with pytest.raises(g.GError):
            g.GgufFile(_write(tmp_path, data[:n], "cut.gguf"))


def test_malformed_headers(tmp_path):
    t = [("t", (4,), gw.GGML_F32, np.zeros(4, np.float32))]
    good = gw.build([], t)
    bad = {
        "magic": b"GGML" + good[4:],
        "version 1": gw.build([], t, version=1),
        "version 4": gw.build([], t, version=4),
        "tensor count": good[:8] + struct.pack("<Q", 1 << 60) + good[16:],
        "kv count": good[:16] + struct.pack("<Q", 1 << 60) + good[24:],
        "alignment 0": gw.build([], t, alignment=0),
        "alignment 48": gw.build([], t, alignment=48),
        "misaligned": gw.build([], t, offsets=[4]),
        "past the end": gw.build([], t)[:-1],
        "offset past the end": gw.build([], t, offsets=[1 << 40]),
        "five dims": gw.build([], [("t", (1, 1, 1, 1, 4), gw.GGML_F32, np.zeros(4, np.float32))]),
        "zero dim": gw.build([], [("t", (0,), gw.GGML_F32, b"")]),
        "overflowing shape": gw.build([], [("t", (1 << 39, 1 << 39), gw.GGML_F32, b"")]),
        "ragged blocks": gw.build([], [("t", (48, 1), gw.GGML_Q4_0, bytes(27))]),
        "duplicate": gw.build([], t + t),
        "value type": gw.build([("k", gw.U8, 1)], t).replace(b"k" + struct.pack("<I", gw.U8), b"k" + struct.pack("<I", 99)),
        "string length": gw.build([("k", gw.STRING, "abc")], t).replace(struct.pack("<Q", 3) + b"abc",
                                                                       struct.pack("<Q", 1 << 50) + b"abc"),
        "array count": gw.build([("k", gw.ARRAY, (gw.U32, [1, 2]))], t).replace(struct.pack("<IQ", gw.U32, 2),
                                                                                struct.pack("<IQ", gw.U32, 1 << 61)),
        "nested array": gw.build([("k", gw.ARRAY, (gw.U32, [1, 2]))], t).replace(struct.pack("<IQ", gw.U32, 2),
                                                                                 struct.pack("<IQ", gw.ARRAY, 2)),
    }
    with g.GgufFile(_write(tmp_path, good)):
        pass
    for what, data in bad.items():
        with pytest.raises(g.GError):
            g.GgufFile(_write(tmp_path, data, "bad.gguf"))
            pytest.fail("accepted a file with a bad " + what)
    with pytest.raises(g.GError):
        g.GgufFile(str(tmp_path / "does-not-exist.gguf"))


HP = dict(n_vocab=96, n_embd=64, n_head=2, n_layer=2, n_ff=96, n_ctx=48, rms_eps=1e-5, freq_base=10000.0)


def _llama_weights(rng, hp, tied=False):
    e, f, v = hp["n_embd"], hp["n_ff"], hp["n_vocab"]
    w = {"tok_embd": _q4(rng, v, e), "output": None if tied else _q4(rng, v, e),
         "out_norm": rng.standard_normal(e).astype(np.float32), "layers": []}
    for _ in range(hp["n_layer"]):
        w["layers"].append({"attn_norm": rng.standard_normal(e).astype(np.float32),
                            "ffn_norm": rng.standard_normal(e).astype(np.float32),
                            "wq": _q4(rng, e, e), "wk": _q4(rng, e, e), "wv": _q4(rng, e, e), "wo": _q4(rng, e, e),
                            "w_gate": _q4(rng, f, e), "w_up": _q4(rng, f, e), "w_down": _q4(rng, e, f)})
    return w


def test_llama_hparams(tmp_path):
    rng = np.random.default_rng(3)
    w = _llama_weights(rng, HP)
    with g.GgufFile(_write(tmp_path, gw.llama_file(HP, w))) as f:
        hp = f.llama_hparams(2048)
        assert {k: hp[k] for k in ("n_vocab", "n_embd", "n_head", "n_layer", "n_ff", "n_ctx")} == \
            {k: HP[k] for k in ("n_vocab", "n_embd", "n_head", "n_layer", "n_ff", "n_ctx")}
        assert hp["rms_eps"] == np.float32(1e-5) and hp["freq_base"] == 10000.0 and hp["freq_scale"] == 1.0
        assert f.llama_hparams(16)["n_ctx"] == 16                      # the caller's limit wins when smaller
        assert f.get_string("general.name") == "tiny test model"
        assert f.get_string_array("tokenizer.ggml.tokens")[95] == "<t95>"
        assert len(f.tensors()) == 3 + 9 * HP["n_layer"]
    # grouped-query attention is refused, as is another architecture
    with g.GgufFile(_write(tmp_path, gw.llama_file(dict(HP, n_head_kv=1), w))) as f:
        with pytest.raises(g.GError) as e:
            f.llama_hparams()
        assert e.value.kind == "Unimplemented"
    other = gw.build([("general.architecture", gw.STRING, "falcon")], [])
    with g.GgufFile(_write(tmp_path, other)) as f:
        with pytest.raises(g.GError) as e:
            f.llama_hparams()
        assert e.value.kind == "Unimplemented"
    # linear rope scaling becomes freq_scale = 1 / factor; other scaling types are refused
    lin = [("llama.rope.scaling.type", gw.STRING, "linear"), ("llama.rope.scaling.factor", gw.F32, 4.0)]
    with g.GgufFile(_write(tmp_path, gw.llama_file(HP, w, extra_md=lin))) as f:
        assert f.llama_hparams()["freq_scale"] == 0.25
    with g.GgufFile(_write(tmp_path, gw.llama_file(HP, w, extra_md=[("llama.rope.scale_linear", gw.F32, 2.0)]))) as f:
        assert f.llama_hparams()["freq_scale"] == 0.5
    with g.GgufFile(_write(tmp_path, gw.llama_file(HP, w, extra_md=[("llama.rope.scaling.type", gw.STRING, "yarn")]))) as f:
        with pytest.raises(g.GError) as e:
            f.llama_hparams()
        assert e.value.kind == "Unimplemented"
