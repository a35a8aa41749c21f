"""The LLaMA decode step issued as galois ops (galois_amd/host/llama.cpp) against the same sequence on the CPU oracle."""
import numpy as np
import pytest

import oracle
from galois_amd import host_api as g
from tests import npref

pytestmark = pytest.mark.gpu

LAYER_Q = ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down")


def _make_weights(rng, hp):
    e, f, v = hp["n_embd"], hp["n_ff"], hp["n_vocab"]
    shapes = {"wq": (e, e), "wk": (e, e), "wv": (e, e), "wo": (e, e), "w_gate": (f, e), "w_up": (f, e), "w_down": (e, f)}

    def q(rows, cols):
        return oracle.quantize_q4_0((rng.standard_normal((rows, cols)) * 0.02).astype(np.float32))

    w = {"tok_embd": q(v, e), "output": q(v, e), "out_norm": (1 + 0.1 * rng.standard_normal(e)).astype(np.float32),
         "layers": []}
    for _ in range(hp["n_layer"]):
        lw = {n: q(*shapes[n]) for n in LAYER_Q}
        lw["attn_norm"] = (1 + 0.1 * rng.standard_normal(e)).astype(np.float32)
        lw["ffn_norm"] = (1 + 0.1 * rng.standard_normal(e)).astype(np.float32)
        w["layers"].append(lw)
    return w


def _load(dec, w, kc=None, vc=None):
    for n in ("tok_embd", "output", "out_norm"):
        dec.tensor(n).write(w[n])
    for i, lw in enumerate(w["layers"]):
        for n, a in lw.items():
            dec.tensor(n, i).write(a)
        if kc is not None:   # kc[i] is [n_ctx][n_embd]; a head-major decoder keeps [n_head][n_ctx][head_dim]
            hm = getattr(dec, "kv_head_major", False)
            h = dec.hp["n_head"]
            lay = (lambda c: np.ascontiguousarray(c.reshape(c.shape[0], h, -1).transpose(1, 0, 2))) if hm else (lambda c: c)
            dec.tensor("k_cache", i).write(lay(kc[i]))
            dec.tensor("v_cache", i).write(lay(vc[i]))


def _ref_step(w, hp, kc, vc, token, n_past, round_kv=False):
    """One token through the oracle's ops; kc / vc [n_layer][n_ctx][n_embd] are updated in place.
    round_kv: the appended rows are rounded to f16 (an f16 cache) before the attention reads them."""
    e, h = hp["n_embd"], hp["n_head"]
    d, L, eps = e // h, n_past + 1, hp["rms_eps"]
    theta_scale = np.float32(hp["freq_base"]) ** np.float32(-2.0 / d)
    pos = np.array([n_past], np.int32)
    x = oracle.get_rows_q4_0(w["tok_embd"], np.array([token], np.int32))[0]
    for i, lw in enumerate(w["layers"]):
        a = oracle.mul(oracle.rms_norm(x, eps), lw["attn_norm"])
        q, k, v = (oracle.mul_mat_q4_0_f32(lw[n], a) for n in ("wq", "wk", "wv"))
        qr = oracle.rope(q.reshape(h, d), pos, 1.0, h, float(theta_scale))
        kr = oracle.rope(k.reshape(h, d), pos, 1.0, h, float(theta_scale))
        kc[i][n_past], vc[i][n_past] = kr.reshape(-1), v
        if round_kv:
            kc[i][n_past] = kc[i][n_past].astype(np.float16).astype(np.float32)
            vc[i][n_past] = vc[i][n_past].astype(np.float16).astype(np.float32)
        kview = np.lib.stride_tricks.as_strided(kc[i], (h, L, d), (d * 4, e * 4, 4))
        s = oracle.mul_mat_f32(kview, qr.reshape(h, 1, d))                       # [h, 1, L]
        p = oracle.soft_max(oracle.scale(s, float(np.float32(1.0) / np.sqrt(np.float32(d)))).reshape(h, L))
        vview = np.lib.stride_tricks.as_strided(vc[i], (h, d, L), (d * 4, 4, e * 4))
        o = oracle.mul_mat_f32(vview, p.reshape(h, 1, L)).reshape(-1)            # [h, 1, d] -> [e]
        x1 = oracle.add(oracle.mul_mat_q4_0_f32(lw["wo"], o), x)
        f = oracle.mul(oracle.rms_norm(x1, eps), lw["ffn_norm"])
        hh = oracle.mul(oracle.silu(oracle.mul_mat_q4_0_f32(lw["w_gate"], f)), oracle.mul_mat_q4_0_f32(lw["w_up"], f))
        x = oracle.add(oracle.mul_mat_q4_0_f32(lw["w_down"], hh), x1)
    return oracle.mul_mat_q4_0_f32(w["output"], oracle.mul(oracle.rms_norm(x, eps), w["out_norm"]))


SMALL = dict(n_vocab=512, n_embd=256, n_head=2, n_layer=2, n_ff=512, n_ctx=64, rms_eps=1e-6, freq_base=10000.0)


@pytest.fixture(scope="module")
def gdev():
    return g.Device.gpu(0)


def _check(got, ref, tol):
    emax, el2 = npref.rel_err(got, ref)
    assert emax < tol and el2 < tol, (emax, el2)


def test_decode_step_matches_oracle_with_a_filled_cache(gdev):
    rng = np.random.default_rng(50)
    hp = SMALL
    w = _make_weights(rng, hp)
    n_past = 37
    kc = rng.standard_normal((hp["n_layer"], hp["n_ctx"], hp["n_embd"])).astype(np.float32)
    vc = rng.standard_normal((hp["n_layer"], hp["n_ctx"], hp["n_embd"])).astype(np.float32)
    dec = g.LlamaDecoder(gdev, **hp)
    _load(dec, w, kc, vc)
    ref = _ref_step(w, hp, kc.copy(), vc.copy(), 123, n_past)
    for fused, per_layer, tail in ((0, 23, 3), (1, 20, 2), (2, 12, 1), (3, 5, 1), (4, 5, 1), (5, 4, 1)):
        _load(dec, w, kc, vc)
        dec.decode(123, n_past, fused)
        _check(dec.logits(), ref, 1e-4)
        # launches: embedding lookup + per layer + final norm and lm head (fused = 2: grouped products, 12 per layer;
        # fused = 3: attention in one launch too; fused = 5: q | k | v and the attention share a launch)
        assert dec.ops_per_step() == 1 + hp["n_layer"] * per_layer + tail
    # the step wrote row n_past of both caches and nothing else
    kc_ref, vc_ref = kc.copy(), vc.copy()
    _ref_step(w, hp, kc_ref, vc_ref, 123, n_past)
    for i in range(hp["n_layer"]):
        kg = dec.tensor("k_cache", i).to_cpu_tensor()
        vg = dec.tensor("v_cache", i).to_cpu_tensor()
        rows = np.arange(hp["n_ctx"]) != n_past
        assert np.array_equal(kg[rows], kc[i][rows]) and np.array_equal(vg[rows], vc[i][rows])
        _check(kg[n_past], kc_ref[i][n_past], 1e-4)
        _check(vg[n_past], vc_ref[i][n_past], 1e-4)
    dec.close()


def test_decode_from_an_empty_cache_over_several_tokens(gdev):
    rng = np.random.default_rng(51)
    hp = SMALL
    w = _make_weights(rng, hp)
    dec = g.LlamaDecoder(gdev, **hp)
    _load(dec, w)
    kc = np.zeros((hp["n_layer"], hp["n_ctx"], hp["n_embd"]), np.float32)
    vc = np.zeros_like(kc)
    for n_past, tok in enumerate([1, 400, 17, 17, 511, 3, 250]):
        ref = _ref_step(w, hp, kc, vc, tok, n_past)
        dec.decode(tok, n_past, (0, 3, 2, 4, 1, 5, 5)[n_past])   # every launch plan in turn, on one cache
        _check(dec.logits(), ref, 1e-4)
    dec.close()


def test_decode_with_an_f16_kv_cache(gdev):
    """KV cache in f16 (fused attention only): logits against the oracle's step run on caches rounded to f16 after
    every append, over several tokens on one cache."""
    rng = np.random.default_rng(53)
    hp = SMALL
    w = _make_weights(rng, hp)
    dec = g.LlamaDecoder(gdev, kv_f16=True, **hp)
    _load(dec, w)
    kc = np.zeros((hp["n_layer"], hp["n_ctx"], hp["n_embd"]), np.float32)
    vc = np.zeros_like(kc)
    for n_past, tok in enumerate([5, 300, 41, 41, 77, 8]):
        # the oracle's step appends f32 rows; this step's own attention must already see them rounded
        ref = _ref_step(w, hp, kc, vc, tok, n_past, round_kv=True)
        dec.decode(tok, n_past, (3, 3, 4, 3, 5, 5)[n_past])
        _check(dec.logits(), ref, 2e-4)
    kg = dec.tensor("k_cache", 1).to_cpu_tensor()
    assert kg.dtype == np.float16 and np.array_equal(kg[6:], np.zeros_like(kg[6:])) and np.any(kg[5] != 0)
    _check(kg[:6].astype(np.float32), kc[1][:6], 1e-3)
    with pytest.raises(g.GError) as e:
        dec.decode(1, 6, 2)
    assert e.value.kind == "Unimplemented"
    dec.close()


@pytest.mark.parametrize("kv_f16", [False, True])
def test_decode_with_head_major_caches(gdev, kv_f16):
    """Caches kept [n_head][n_ctx][head_dim]: every launch plan against the oracle on a filled cache (the plans built
    from single ops reach the cache through strided views), the appended rows in their head-major places."""
    rng = np.random.default_rng(57)
    hp = SMALL
    w = _make_weights(rng, hp)
    n_past = 41
    ct = np.float16 if kv_f16 else np.float32
    kc = rng.standard_normal((hp["n_layer"], hp["n_ctx"], hp["n_embd"])).astype(ct)
    vc = rng.standard_normal((hp["n_layer"], hp["n_ctx"], hp["n_embd"])).astype(ct)
    dec = g.LlamaDecoder(gdev, kv_f16=kv_f16, kv_head_major=True, **hp)
    kc_ref, vc_ref = kc.astype(np.float32), vc.astype(np.float32)
    ref = _ref_step(w, hp, kc_ref, vc_ref, 77, n_past, round_kv=kv_f16)
    for fused in ((3, 4, 5) if kv_f16 else (0, 1, 2, 3, 4, 5)):
        _load(dec, w, kc, vc)
        dec.decode(77, n_past, fused)
        _check(dec.logits(), ref, 2e-4 if kv_f16 else 1e-4)
    h, d = hp["n_head"], hp["n_embd"] // hp["n_head"]
    for i in range(hp["n_layer"]):
        kg = dec.tensor("k_cache", i).to_cpu_tensor()
        assert kg.shape == (h, hp["n_ctx"], d) and kg.dtype == ct
        kg = kg.transpose(1, 0, 2).reshape(hp["n_ctx"], -1)
        rows = np.arange(hp["n_ctx"]) != n_past
        assert np.array_equal(kg[rows], kc[i][rows])
        _check(kg[n_past].astype(np.float32), kc_ref[i][n_past], 1e-3 if kv_f16 else 1e-4)
    dec.close()


def test_graph_replays_equal_the_eager_step(gdev):
    rng = np.random.default_rng(52)
    hp = SMALL
    w = _make_weights(rng, hp)
    kc = rng.standard_normal((hp["n_layer"], hp["n_ctx"], hp["n_embd"])).astype(np.float32)
    dec = g.LlamaDecoder(gdev, **hp)
    _load(dec, w, kc, kc[::-1].copy())
    dec.decode(9, 20, 2)
    eager = dec.logits()
    dec.capture(9, 20, 2)
    for i in range(4):
        dec.replay()
        assert np.array_equal(dec.logits(), eager), i
        # eager work and synchronisation between the replays
        dec.decode(9 + i, 30 + i, False)        # appends rows the recorded step (21 keys) never reads
        assert not np.array_equal(dec.logits(), eager)
        dec.decode(9, 20, 2)                    # puts token 9 / position 20 back into the device-side inputs
    dec.close()


def test_capture_refuses_calls_that_allocate_or_block(dev):
    from galois_amd import GaloisHipError
    x = dev.upload(np.arange(8, dtype=np.float32))
    y = dev.alloc(32)
    dev.graph_begin_capture()
    try:
        for call in (lambda: dev.alloc(64), dev.synchronize, lambda: dev.download(x, np.float32, 8),
                     dev.graph_begin_capture):
            with pytest.raises(GaloisHipError) as ei:
                call()
            assert ei.value.status == -5
        dev.scale_f32(x, y, 2.0, 8)
    finally:
        graph = dev.graph_end_capture()
    assert np.array_equal(dev.download(y, np.float32, 8), np.zeros(8, np.float32))      # recorded, not run
    dev.graph_launch(graph)
    assert np.array_equal(dev.download(y, np.float32, 8), 2 * np.arange(8, dtype=np.float32))
    dev.graph_destroy(graph)


def test_full_width_layers_at_kv_length_2048(gdev):
    """Two layers at LLaMA-7B width (4096 / 32 heads / 11008 / vocab 32000) attending over 2048 cached positions,
    through every launch plan the benchmark reports (the second layer takes the first one's residual stream and, in
    the split-norm plan, its pre-weighted copy and partial sums of squares), a graph replay of the last plan, and the
    f16 KV cache."""
    rng = np.random.default_rng(53)
    hp = dict(n_vocab=32000, n_embd=4096, n_head=32, n_layer=2, n_ff=11008, n_ctx=2048, rms_eps=1e-6,
              freq_base=10000.0)
    w = _make_weights(rng, hp)
    kc = rng.standard_normal((2, 2048, 4096)).astype(np.float32)
    vc = rng.standard_normal((2, 2048, 4096)).astype(np.float32)
    dec = g.LlamaDecoder(gdev, **hp)
    ref = _ref_step(w, hp, kc.copy(), vc.copy(), 31999, 2047)
    for fused in (0, 1, 2, 3, 4, 5):
        _load(dec, w, kc, vc)
        dec.decode(31999, 2047, fused)
        _check(dec.logits(), ref, 1e-4)
    for fused in (4, 5):
        _load(dec, w, kc, vc)
        dec.capture(31999, 2047, fused)
        for _ in range(2):
            dec.replay()
            _check(dec.logits(), ref, 1e-4)
    dec.close()
    # f16 caches: the oracle's step on the f16 contents, this step's rows rounded before the attention reads them
    kc16, vc16 = kc.astype(np.float16), vc.astype(np.float16)
    dec = g.LlamaDecoder(gdev, kv_f16=True, **hp)
    ref16 = _ref_step(w, hp, kc16.astype(np.float32), vc16.astype(np.float32), 31999, 2047, round_kv=True)
    for fused in (3, 4, 5):
        _load(dec, w, kc16, vc16)
        dec.decode(31999, 2047, fused)
        _check(dec.logits(), ref16, 2e-4)
    dec.close()
    # head-major f32 caches at full width: the two shortest plans
    dec = g.LlamaDecoder(gdev, kv_head_major=True, **hp)
    for fused in (4, 5):
        _load(dec, w, kc, vc)
        dec.decode(31999, 2047, fused)
        _check(dec.logits(), ref, 1e-4)
    dec.close()


def _normal_f32(seed, count, scale, threads=8):
    """count f32 draws of N(0, scale^2) from `threads` independent streams filled in parallel."""
    from concurrent.futures import ThreadPoolExecutor
    out = np.empty(count, np.float32)
    bounds = np.linspace(0, count, threads + 1).astype(np.int64)

    def fill(t):
        g = np.random.default_rng([seed, t])
        g.standard_normal(out=out[bounds[t]:bounds[t + 1]], dtype=np.float32)
        out[bounds[t]:bounds[t + 1]] *= np.float32(scale)

    with ThreadPoolExecutor(threads) as ex:
        list(ex.map(fill, range(threads)))
    return out


def test_32_layers_at_kv_length_2048_against_the_oracle(gdev):
    """BASELINE configs[4] at its stated depth: 32 layers of distinct N(0, 0.02) weights quantized to Q4_0 (by the
    oracle, on the host), d_model 4096, 32 heads, FFN 11008, vocab 32000, one token attending over 2048 cached
    positions, against the oracle's op-by-op step in f64 dot products.  What accumulates over 225 products of the
    block-fixed-point matvec is measured here against arithmetic that does not share it, and beside it what the same
    step accumulates when the matvec runs in plain f32 multiply-add.  Every layer's cache starts
    from the same 2047 rows (the step appends its own row 2047 to each before reading it), which keeps the host side
    at two 32 MB arrays; the weights differ from layer to layer."""
    from concurrent.futures import ThreadPoolExecutor
    hp = dict(n_vocab=32000, n_embd=4096, n_head=32, n_layer=32, n_ff=11008, n_ctx=2048, rms_eps=1e-6, freq_base=10000.0)
    e, f, v, c = hp["n_embd"], hp["n_ff"], hp["n_vocab"], hp["n_ctx"]
    shapes = {"wq": (e, e), "wk": (e, e), "wv": (e, e), "wo": (e, e), "w_gate": (f, e), "w_up": (f, e), "w_down": (e, f)}
    seed = [1000]

    def q(rows, cols):   # rows quantized in parallel slabs (the oracle's quantizer is one thread per call)
        seed[0] += 1
        w = _normal_f32(seed[0], rows * cols, 0.02).reshape(rows, cols)
        slabs = np.array_split(np.arange(rows), 8)
        with ThreadPoolExecutor(8) as ex:
            parts = list(ex.map(lambda r: oracle.quantize_q4_0(w[r[0]:r[-1] + 1]), slabs))
        return np.concatenate(parts)

    rng = np.random.default_rng(77)
    print("32-layer step: drawing and quantizing weights", flush=True)
    w = {"tok_embd": q(v, e), "output": q(v, e), "out_norm": (1 + 0.1 * rng.standard_normal(e)).astype(np.float32),
         "layers": []}
    for _ in range(hp["n_layer"]):
        lw = {n: q(*shapes[n]) for n in LAYER_Q}
        lw["attn_norm"] = (1 + 0.1 * rng.standard_normal(e)).astype(np.float32)
        lw["ffn_norm"] = (1 + 0.1 * rng.standard_normal(e)).astype(np.float32)
        w["layers"].append(lw)
    kc0 = _normal_f32(5, c * e, 1.0).reshape(c, e)
    vc0 = _normal_f32(6, c * e, 1.0).reshape(c, e)
    tok, n_past = 31999, c - 1
    print("32-layer step: oracle", flush=True)
    kc_ref = [kc0.copy()] * hp["n_layer"]   # one array behind every layer: each layer rewrites row n_past before it reads
    vc_ref = [vc0.copy()] * hp["n_layer"]
    ref = _ref_step(w, hp, kc_ref, vc_ref, tok, n_past)
    assert np.all(np.isfinite(ref))
    dec = g.LlamaDecoder(gdev, **hp)
    for n in ("tok_embd", "output", "out_norm"):
        dec.tensor(n).write(w[n])
    for i, lw in enumerate(w["layers"]):
        for n, a in lw.items():
            dec.tensor(n, i).write(a)

    def load_caches():
        for i in range(hp["n_layer"]):
            dec.tensor("k_cache", i).write(kc0)
            dec.tensor("v_cache", i).write(vc0)

    worst = {}
    for fused in (0, 4, 5):
        print("32-layer step: plan %d" % fused, flush=True)
        load_caches()
        dec.decode(tok, n_past, fused)
        worst[fused] = npref.rel_err(dec.logits(), ref)
    # the one-kernel-per-op plan once more with the matvec in the reference kernel's own f32 multiply-add
    # (GALOIS_HIP_OPT_GEMV_F32_ARITHMETIC = 1): what 32 layers make of f32 rounding alone
    gdev.set_option(1, 1)
    try:
        load_caches()
        dec.decode(tok, n_past, 0)
        worst["f32_arithmetic"] = npref.rel_err(dec.logits(), ref)
    finally:
        gdev.set_option(1, 0)
    load_caches()
    dec.capture(tok, n_past, 5)
    dec.replay()
    worst["graph5"] = npref.rel_err(dec.logits(), ref)
    # the same token through the prefill pass (one row: panel matmuls with fp16 activations, the prefill attention over
    # all 2048 keys, the fused adding passes) -- the same graph with 2^-11 of rounding on every product's operands
    load_caches()
    dec.prefill([tok], n_past)
    prefill_err = npref.rel_err(dec.logits(), ref)
    dec.close()
    print("32-layer logits vs the oracle (max-rel, l2-rel):", worst, "prefill pass:", prefill_err, flush=True)
    # the prefill bar of one product is 2e-3; 32 layers of them (random weights: the errors add like a random walk)
    assert prefill_err[0] < 1e-2 and prefill_err[1] < 1e-2, prefill_err
    # The 1e-4 bar belongs to one matvec.  Through 32 layers (225 products, softmax, SwiGLU) f32 rounding alone --
    # the reference kernel's own multiply-add, measured above -- leaves the logits 1.1e-4 from the f64 step, so at
    # this depth the bar is: no plan further than 2e-4, and none more than twice as far as f32 arithmetic.
    f32_max, f32_l2 = worst["f32_arithmetic"]
    assert f32_max < 2e-4 and f32_l2 < 2e-4, worst
    for plan, (emax, el2) in worst.items():
        assert emax < 2e-4 and el2 < 2e-4, (plan, emax, el2)
        assert emax < 2 * f32_max and el2 < 2 * f32_l2, (plan, emax, el2, f32_max, f32_l2)


def _ref_tokens(w, hp, kc, vc, tokens, n_past, round_kv=False):
    """The oracle's step for each of `tokens` in turn from position n_past; the last token's logits."""
    for i, tok in enumerate(tokens):
        ref = _ref_step(w, hp, kc, vc, int(tok), n_past + i, round_kv)
    return ref


# The prefill products take their activations rounded to f16 (the Q4_0 prefill matmul and, for several rows, the f16
# matmul of an f16 cache): 2^-11 relative per element, against the decode step's exact f32 activations.
PREFILL_TOL = 3e-3


@pytest.mark.parametrize("kv_f16", [False, True])
@pytest.mark.parametrize("n_head", [2, 4, 128])
def test_prefill_matches_the_oracle_token_by_token(gdev, kv_f16, n_head):
    """Two prefill calls (an empty cache, then a filled one; 20 and 9 tokens: neither a multiple of the panel's 16
    rows) and a decode step on the caches they left, each against the oracle's one-token step run over the same tokens.
    Heads of 128 (n_head = 2) take the attention as one launch, heads of 64 as the op sequence; heads of 2 also take
    the two rotations and the cache append as single ops."""
    rng = np.random.default_rng(57)
    hp = dict(SMALL, n_head=n_head)
    w = _make_weights(rng, hp)
    dec = g.LlamaDecoder(gdev, kv_f16=kv_f16, **hp)
    _load(dec, w)
    kc = np.zeros((hp["n_layer"], hp["n_ctx"], hp["n_embd"]), np.float32)
    vc = np.zeros_like(kc)
    toks = rng.integers(0, hp["n_vocab"], 30).astype(np.int32)
    ref = _ref_tokens(w, hp, kc, vc, toks[:20], 0, kv_f16)
    dec.prefill(toks[:20], 0)
    _check(dec.logits(), ref, PREFILL_TOL)
    # library calls: embedding lookup, per layer 14 with the op-sequence attention and 8 with the attention in one
    # launch (heads of 2: 15, and two more for the copies into f16 caches), then the last row's copy, norm and lm head
    per_layer = {2: 8, 4: 14, 128: 15 + (2 if kv_f16 else 0)}[n_head]
    assert dec.ops_per_prefill() == 1 + hp["n_layer"] * per_layer + 3
    ref = _ref_tokens(w, hp, kc, vc, toks[20:29], 20, kv_f16)
    dec.prefill(toks[20:29], 20)
    _check(dec.logits(), ref, PREFILL_TOL)
    for i in range(hp["n_layer"]):
        kg = dec.tensor("k_cache", i).to_cpu_tensor().astype(np.float32)
        vg = dec.tensor("v_cache", i).to_cpu_tensor().astype(np.float32)
        assert not kg[29:].any() and not vg[29:].any()
        _check(kg[:29], kc[i][:29], PREFILL_TOL)
        _check(vg[:29], vc[i][:29], PREFILL_TOL)
    ref = _ref_step(w, hp, kc, vc, int(toks[29]), 29, kv_f16)
    if kv_f16 and n_head == 128:
        dec.close()          # an f16 cache decodes through the fused attention only (heads of 64 or 128)
        return
    dec.decode(int(toks[29]), 29, {2: 5, 4: 4, 128: 1}[n_head])
    _check(dec.logits(), ref, PREFILL_TOL)
    dec.close()


def test_prefill_of_one_token_and_its_refusals(gdev):
    rng = np.random.default_rng(58)
    hp = SMALL
    w = _make_weights(rng, hp)
    dec = g.LlamaDecoder(gdev, **hp)
    _load(dec, w)
    kc = np.zeros((hp["n_layer"], hp["n_ctx"], hp["n_embd"]), np.float32)
    vc = np.zeros_like(kc)
    ref = _ref_step(w, hp, kc, vc, 7, 0)
    dec.prefill([7], 0)
    _check(dec.logits(), ref, PREFILL_TOL)
    # a full context in one call
    toks = rng.integers(0, hp["n_vocab"], hp["n_ctx"] - 1).astype(np.int32)
    ref = _ref_tokens(w, hp, kc, vc, toks, 1)
    dec.prefill(toks, 1)
    _check(dec.logits(), ref, PREFILL_TOL)
    for bad in (([], 0), ([1, 2], hp["n_ctx"] - 1), ([1], -1), ([hp["n_vocab"]], 0)):
        with pytest.raises(g.GError) as e:
            dec.prefill(*bad)
        assert e.value.kind == "ShapeError"
    dec.close()
    hm = g.LlamaDecoder(gdev, kv_head_major=True, **hp)
    with pytest.raises(g.GError) as e:
        hm.prefill([1, 2, 3], 0)
    assert e.value.kind == "Unimplemented"
    hm.close()
    narrow = g.LlamaDecoder(gdev, **dict(hp, n_embd=128, n_head=1))
    with pytest.raises(g.GError) as e:
        narrow.prefill([1, 2, 3], 0)
    assert e.value.kind == "Unimplemented"
    narrow.close()


@pytest.mark.parametrize("kv_f16", [False, True])
def test_prefill_at_full_width_whole_in_chunks_and_token_by_token(gdev, kv_f16):
    """Two layers at LLaMA-7B width, 600 tokens (not a multiple of any tile): one prefill call, the same tokens as a
    chunk of 512 and a chunk of 88 behind it, and the same tokens decoded one by one (the decode step is held to the
    oracle above).  Chunking changes which shapes the launches take (rows per workgroup, shares of k), not what a row
    is: logits and cache rows agree to 1e-3 between the two prefills, and to the prefill bar with the decode."""
    rng = np.random.default_rng(61)
    hp = dict(n_vocab=32000, n_embd=4096, n_head=32, n_layer=2, n_ff=11008, n_ctx=1024, rms_eps=1e-6, freq_base=10000.0)
    w = _make_weights(rng, hp)
    toks = rng.integers(0, hp["n_vocab"], 600).astype(np.int32)
    zeros = np.zeros((hp["n_layer"], hp["n_ctx"], hp["n_embd"]), np.float16 if kv_f16 else np.float32)
    dec = g.LlamaDecoder(gdev, kv_f16=kv_f16, **hp)

    def caches():
        return [(dec.tensor("k_cache", i).to_cpu_tensor().astype(np.float32)[:600],
                 dec.tensor("v_cache", i).to_cpu_tensor().astype(np.float32)[:600]) for i in range(hp["n_layer"])]

    _load(dec, w, zeros, zeros)
    dec.prefill(toks, 0)
    whole, whole_kv = dec.logits().copy(), caches()
    assert np.all(np.isfinite(whole))
    _load(dec, w, zeros, zeros)
    dec.prefill(toks[:512], 0)
    dec.prefill(toks[512:], 512)
    _check(dec.logits(), whole, 1e-3)
    for (k1, v1), (k2, v2) in zip(caches(), whole_kv):
        _check(k1, k2, 1e-3)
        _check(v1, v2, 1e-3)
    _load(dec, w, zeros, zeros)
    for i, t in enumerate(toks):
        dec.decode(int(t), i, 5)
    _check(dec.logits(), whole, PREFILL_TOL)
    for (k1, v1), (k2, v2) in zip(caches(), whole_kv):
        _check(k1, k2, PREFILL_TOL)
        _check(v1, v2, PREFILL_TOL)
    dec.close()
