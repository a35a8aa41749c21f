#!/usr/bin/env python3
"""Writes tests/golden/kat.json: hand-derived known-answer vectors for the Q4_0 path.

galois's own tests hold no golden vectors for this path (they only print), so the
expected values here come from the block layout / closed forms worked by hand with
Python integers and ``math`` -- never from the C oracle or the HIP kernels.  Every
case says how its answer was derived.  Run:  python tests/golden/make_fixtures.py
"""
import json
import math
import os
import struct

HERE = os.path.dirname(os.path.abspath(__file__))


def f16_bits(v):
    return struct.unpack("<H", struct.pack("<e", v))[0]


def block(d, nibbles):
    """18 bytes: f16 d (little endian), then qs[j] = w[j] | w[j+16] << 4."""
    assert len(nibbles) == 32 and all(0 <= n <= 15 for n in nibbles)
    b = list(struct.pack("<e", d))
    b += [nibbles[j] | (nibbles[j + 16] << 4) for j in range(16)]
    return b


def f32(v):
    return struct.unpack("<f", struct.pack("<f", v))[0]


cases = {}

# --- layout: d = 1.0, qs[j] = j | (15-j)<<4  -> weight j = j-8, weight j+16 = 7-j
nib = list(range(16)) + [15 - j for j in range(16)]
cases["layout_ramp"] = {
    "why": "d=1.0 (0x3C00); low nibble of byte j is j, high nibble is 15-j; value=(nibble-8)*d",
    "block": block(1.0, nib),
    "values": [float(n - 8) for n in nib],
}

# --- quantizer KATs (canonical ggml quantize_row_q4_0)
q = {}
q["zeros"] = {
    "why": "max=+0 -> d = 0/-8 = -0.0 (f16 0x8000), id=0 -> every q = trunc(0+8.5) = 8 -> bytes 0x88",
    "x": [0.0] * 32,
    "block": block(-0.0, [8] * 32),
}
x = [float(j - 8) for j in range(16)] + [float(7 - j) for j in range(16)]
q["ramp_neg_max"] = {
    "why": "first |x|=8 is -8 -> d=-8/-8=1, id=1, q=trunc(x+8.5)=x+8",
    "x": x,
    "block": block(1.0, [int(v) + 8 for v in x]),
}
x = [float(8 - j) for j in range(16)] + [float(j - 7) for j in range(15)] + [-8.0]
# max=+8 (index 0 wins the tie with -8 at index 31: strict '<') -> d=-1, id=-1, q=trunc(-x+8.5);
# x=-8 -> 16.5 -> 16 -> clamped to 15
qq = [min(15, int(-v + 8.5)) for v in x]
q["pos_max_tie_clamp"] = {
    "why": "max=+8 first wins tie -> d=-1; the later -8 maps to 16 and is clamped to 15",
    "x": x,
    "block": block(-1.0, qq),
}
x = [0.0] * 32
x[3] = 1.0
q["single_one"] = {
    "why": "max=1 -> d=-0.125 (f16 0xB000), id=-8: the 1.0 -> trunc(0.5)=0, zeros -> 8",
    "x": x,
    "block": block(-0.125, [0 if j == 3 else 8 for j in range(32)]),
}
x = [0.0] * 32
x[17] = -0.1
d32 = f32(f32(-0.1) / -8.0)
q["f16_scale_rounding"] = {
    "why": "max=-0.1f -> d=f32(0.0125) stored as RNE f16; element -> trunc(-8+8.5)=0; zeros -> 8",
    "x": [f32(v) for v in x],
    "block": block(d32, [0 if j == 17 else 8 for j in range(32)]),
}
# which d the reciprocal is taken of: max = -1.0003f gives d = 0.12503..., which is stored as f16 0.125; the rule takes
# id = 1 / d from the f32 d (7.9976...), so 0.4375 -> trunc(0.4375 * id + 8.5) = trunc(11.998..) = 11, whereas a
# reciprocal of the stored f16 d (exactly 8) would give trunc(12.0) = 12
x = [0.0] * 32
x[0], x[1] = f32(-1.0003), 0.4375
d32 = f32(x[0] / -8.0)
id32 = f32(1.0 / d32)
q1 = int(f32(f32(x[1] * id32) + 8.5))
q0 = int(f32(f32(x[0] * id32) + 8.5))
d16 = struct.unpack("<e", struct.pack("<e", d32))[0]
assert d16 == 0.125 and (q0, q1) == (0, 11) and int(f32(f32(x[1] * f32(1.0 / d16)) + 8.5)) == 12
q["reciprocal_of_the_f32_scale"] = {
    "why": "id = 1/d uses the unrounded f32 d: 0.4375 lands on nibble 11; 1/f16(d) = 8 would give 12",
    "x": x,
    "block": block(d32, [q0, q1] + [8] * 30),
}
cases["quantize_q4_0"] = q

# --- Q8_0 KATs (BlockQ8_0::from_f32): amax=127 -> d=1, id=1, q = round-half-away(x)
x = [-127.0, 2.5, -2.5, 0.5, -0.5, 1.49, -1.51, 126.5] + [float(j) for j in range(8, 32)]
exp = [-127, 3, -3, 1, -1, 1, -2, 127] + list(range(8, 32))
cases["quantize_q8_0"] = {
    "half_away": {
        "why": "amax=127 -> d=1.0 exactly; f32::round is half away from zero",
        "x": x,
        "d_bits": f16_bits(1.0),
        "q": exp,
    },
    "zeros": {"why": "amax=0 -> d=0, id=0, q=0", "x": [0.0] * 32, "d_bits": 0, "q": [0] * 32},
}

# --- dot / GEMV KATs on the ramp block
ramp_vals = cases["layout_ramp"]["values"]
cases["gemv"] = {
    "why": "W row0 = ramp block (d=1), row1 = all-0x88 block with d=1 (all weights 0); K=32, N=2",
    "W": [cases["layout_ramp"]["block"], block(1.0, [8] * 32)],
    "cases": [
        {"x": [1.0] * 32, "y": [sum(ramp_vals), 0.0]},
        {"x": [1.0 if k == 5 else 0.0 for k in range(32)], "y": [ramp_vals[5], 0.0]},
        {"x": [1.0 if k == 20 else 0.0 for k in range(32)], "y": [ramp_vals[20], 0.0]},
        {"x": [float(k) for k in range(32)], "y": [float(sum(k * v for k, v in enumerate(ramp_vals))), 0.0]},
    ],
}

# --- row ops
ln = math.log
cases["soft_max"] = {
    "why": "exp([0, ln2, -inf, ln3]) = [1,2,0,3] / 6",
    "x": [0.0, f32(ln(2.0)), "-inf", f32(ln(3.0))],
    "y": [math.exp(0.0), math.exp(f32(ln(2.0))), 0.0, math.exp(f32(ln(3.0)))],
}
s = sum(cases["soft_max"]["y"])
cases["soft_max"]["y"] = [v / s for v in cases["soft_max"]["y"]]

row = [3.0, 4.0] + [0.0] * 30
eps = f32(1e-6)
sc = 1.0 / math.sqrt(25.0 / 32.0 + eps)
cases["rms_norm"] = {
    "why": "mean(x^2) = 25/32; y = x / sqrt(25/32 + eps); constant row c -> c/sqrt(c^2+eps)",
    "eps": eps,
    "x": [row, [2.0] * 32],
    "y": [[v * sc for v in row], [2.0 / math.sqrt(4.0 + eps)] * 32],
}

fs = f32(math.pi / 2)
cases["rope"] = {
    "why": "one head, 4 dims, theta_scale=0.5: pair i rotates by pos*freq_scale*0.5^i; pos 0 is identity",
    "ncols": 4, "p_delta_rows": 1, "freq_scale": fs, "theta_scale": 0.5,
    "pos": [0, 1, 2],
    "x": [[1.0, 2.0, 3.0, 4.0], [1.0, 0.0, 0.0, 1.0], [1.0, 1.0, 2.0, 0.0]],
}
ys = []
for p, xr in zip(cases["rope"]["pos"], cases["rope"]["x"]):
    out = []
    for i in range(2):
        th = p * fs * (0.5 ** i)
        x0, x1 = xr[2 * i], xr[2 * i + 1]
        out += [x0 * math.cos(th) - x1 * math.sin(th), x0 * math.sin(th) + x1 * math.cos(th)]
    ys.append(out)
cases["rope"]["y"] = ys

with open(os.path.join(HERE, "kat.json"), "w") as f:
    json.dump(cases, f, indent=1)
print("wrote", os.path.join(HERE, "kat.json"))
