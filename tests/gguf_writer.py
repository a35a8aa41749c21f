"""Minimal GGUF writer for the tests: packs metadata and tensors byte by byte from the published container layout
(magic, version, counts, key-value pairs, tensor records, padding to the alignment, tensor data), independently of
the C++ reader it is used to test."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q",
        F64: "<d"}
GGML_F32, GGML_F16, GGML_Q4_0, GGML_Q6_K = 0, 1, 2, 14


def _string(s):
    b = s.encode() if isinstance(s, str) else bytes(s)
    return struct.pack("<Q", len(b)) + b


def _value(vtype, v):
    if vtype == STRING:
        return _string(v)
    if vtype == ARRAY:
        etype, elems = v
        out = struct.pack("<IQ", etype, len(elems))
        for e in elems:
            out += _value(etype, e)
        return out
    return struct.pack(_FMT[vtype], v)


def build(metadata, tensors, version=3, alignment=None, offsets=None):
    """metadata: list of (key, type, value); tensors: list of (name, shape ne0-first, ggml_type, bytes-like).
    alignment None = leave the default (32) implicit; a number is also written as general.alignment.
    offsets: optional explicit data offsets per tensor (to build malformed files).  Returns the file's bytes."""
    metadata = list(metadata)
    if alignment is not None:
        metadata.append(("general.alignment", U32, alignment))
    al = alignment or 32
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(metadata))
    for key, vtype, v in metadata:
        head += _string(key) + struct.pack("<I", vtype) + _value(vtype, v)
    blobs, offs, pos = [], [], 0
    for i, (_, _, _, data) in enumerate(tensors):
        b = np.ascontiguousarray(data).tobytes() if not isinstance(data, (bytes, bytearray)) else bytes(data)
        off = offsets[i] if offsets is not None else pos
        offs.append(off)
        blobs.append(b)
        pos = (off + len(b) + al - 1) // al * al
    for (name, shape, ggml_type, _), off in zip(tensors, offs):
        head += _string(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape)
        head += struct.pack("<IQ", ggml_type, off)
    data_start = (len(head) + al - 1) // al * al
    out = bytearray(head) + bytearray(data_start - len(head))
    for b, off in zip(blobs, offs):
        if off > 1 << 32:  # a deliberately impossible offset: record it, place no data
            continue
        end = data_start + off + len(b)
        if len(out) < end:
            out += bytearray(end - len(out))
        out[data_start + off:end] = b
    return bytes(out)


def llama_file(hp, w, extra_md=(), **kw):
    """A llama-architecture file from hyper-parameters (as tests/test_gpu_llama.py's dicts) and weights
    {tok_embd, output, out_norm, layers: [{attn_norm, ffn_norm, wq, wk, wv, wo, w_gate, w_up, w_down}]} where the
    linear weights are Q4_0 block bytes and the norms float32."""
    e, f, v = hp["n_embd"], hp["n_ff"], hp["n_vocab"]
    md = [("general.architecture", STRING, "llama"), ("general.name", STRING, "tiny test model"),
          ("llama.block_count", U32, hp["n_layer"]), ("llama.embedding_length", U32, e),
          ("llama.feed_forward_length", U32, f), ("llama.attention.head_count", U32, hp["n_head"]),
          ("llama.attention.head_count_kv", U32, hp.get("n_head_kv", hp["n_head"])),
          ("llama.context_length", U32, hp["n_ctx"]), ("llama.rope.dimension_count", U32, e // hp["n_head"]),
          ("llama.attention.layer_norm_rms_epsilon", F32, hp["rms_eps"]), ("llama.rope.freq_base", F32, hp["freq_base"]),
          ("tokenizer.ggml.tokens", ARRAY, (STRING, ["<t%d>" % i for i in range(v)]))]
    ts = [("token_embd.weight", (e, v), GGML_Q4_0, w["tok_embd"]), ("output_norm.weight", (e,), GGML_F32, w["out_norm"])]
    if w.get("output") is not None:
        ts.append(("output.weight", (e, v), GGML_Q4_0, w["output"]))
    names = {"attn_norm": ("attn_norm", (e,), GGML_F32), "ffn_norm": ("ffn_norm", (e,), GGML_F32),
             "wq": ("attn_q", (e, e), GGML_Q4_0), "wk": ("attn_k", (e, e), GGML_Q4_0), "wv": ("attn_v", (e, e), GGML_Q4_0),
             "wo": ("attn_output", (e, e), GGML_Q4_0), "w_gate": ("ffn_gate", (e, f), GGML_Q4_0),
             "w_up": ("ffn_up", (e, f), GGML_Q4_0), "w_down": ("ffn_down", (f, e), GGML_Q4_0)}
    for i, lw in enumerate(w["layers"]):
        for n, a in lw.items():
            gn, shape, ty = names[n]
            ts.append(("blk.%d.%s.weight" % (i, gn), shape, ty, a))
    return build(md + list(extra_md), ts, **kw)
