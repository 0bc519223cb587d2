"""Writes tests/golden/rounding_cases.json: small inputs on which each rounding point of the reference's fused decode
kernels (lfm25_cuda_kernels.py:32-44 RMSNorm, :58-65 SwiGLU, :75-100 conv update, :113-140 QK-norm + RoPE) decides
the bf16 result.

Every case is computed here with scalar numpy float32 arithmetic (each operation rounds to fp32, as the kernels' fp32
registers do) and an integer round-to-nearest-even to bf16 — no torch, nothing from `oracle/`.  For each rounding
point the search keeps the first input whose result changes when that one rounding is left out; the fixture stores
the input, the result with every rounding (`expected`) and the result without that one (`without`), so a restatement
that drops or misplaces the rounding fails the case.  Two of the cases are worked by hand in
tests/test_oracle_rounding.py.

    python tests/golden/make_rounding_cases.py
"""
import json
import os
import struct

import numpy as np

f32 = np.float32


def bf(x):
    """fp32 -> bf16 (round to nearest, ties to even) -> fp32."""
    bits = struct.unpack("<I", struct.pack("<f", float(f32(x))))[0]
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return f32(struct.unpack("<f", struct.pack("<I", bits))[0])


def rsqrt(x):
    return f32(1.0) / np.sqrt(f32(x))


def rms(x, r, w, eps, skip=None):
    h = [f32(a) + f32(b) for a, b in zip(x, r)]
    if skip != "add":
        h = [bf(v) for v in h]
    total = f32(0)
    for v in h:
        total = total + v * v
    inv = rsqrt(total / f32(len(h)) + f32(eps))
    n = [v * inv for v in h]
    if skip != "norm":
        n = [bf(v) for v in n]
    return [float(bf(a * f32(b))) for a, b in zip(n, w)], [float(bf(v)) for v in h]


def swiglu(g, u, skip=None):
    a = f32(g) / (f32(1) + np.exp(-f32(g)))
    if skip != "act":
        a = bf(a)
    return float(bf(a * f32(u)))


def conv(b, c, x, s1, s2, w, skip=None):
    bx = f32(b) * f32(x)
    if skip != "bx":
        bx = bf(bx)
    p0, p1, p2 = f32(s1) * f32(w[0]), f32(s2) * f32(w[1]), bx * f32(w[2])
    if skip != "p0":
        p0 = bf(p0)
    if skip != "p1":
        p1 = bf(p1)
    if skip != "p2":
        p2 = bf(p2)
    total = p0 + p1 + p2
    if skip != "sum":
        total = bf(total)
    return float(bf(f32(c) * total)), float(bf(bx))


def qk_head(x, w, cos, sin, eps, skip=None):
    """One head of D dims: x, w [D]; cos, sin [D/2] fp32 table rows."""
    d = len(x)
    total = f32(0)
    for v in x:
        total = total + f32(v) * f32(v)
    inv = rsqrt(total / f32(d) + f32(eps))
    n = [f32(v) * inv for v in x]
    if skip != "norm":
        n = [bf(v) for v in n]
    n = [a * f32(b) for a, b in zip(n, w)]
    if skip != "weight":
        n = [bf(v) for v in n]
    out = []
    for i in range(d):
        c, s = f32(cos[i % (d // 2)]), f32(sin[i % (d // 2)])
        if skip != "table":
            c, s = bf(c), bf(s)
        left, right = n[i] * c, n[(i + d // 2) % d] * s
        if skip != "left":
            left = bf(left)
        if skip != "right":
            right = bf(right)
        out.append(float(bf(left - right if i < d // 2 else left + right)))
    return out


VALUES = [float(bf(v)) for v in (1.0, 1.0078125, 1.5, 1.7421875, 2.25, 3.0, 0.3330078125, 0.7109375, 5.0, 7.0, 0.1, 1.3, 2.7,
                                 -1.1, -0.6, 0.9)]


def main():
    rng = np.random.default_rng(0)
    pick = lambda n: [VALUES[i] for i in rng.integers(0, len(VALUES), n)]
    cases = {}
    for skip in ("add", "norm"):
        while True:
            x, r, w = pick(8), [v * 2.0 ** -7 for v in pick(8)], pick(8)
            (a, summed), (b, _) = rms(x, r, w, 1e-5), rms(x, r, w, 1e-5, skip)
            if a != b:
                cases["rms_" + skip] = dict(x=x, residual=r, weight=w, eps=1e-5, expected=a, summed=summed, without=b)
                break
    # the two cases worked by hand in tests/test_oracle_rounding.py are fixed inputs, not search results
    g, u = 1.0, 1.0078125
    cases["swiglu_act"] = dict(gate=g, up=u, expected=swiglu(g, u), without=swiglu(g, u, "act"))
    hand = dict(b=5.0, c=0.8984375, x=1.0, s1=7.0, s2=0.7109375, w=[1.0, 5.0, 2.703125])
    for skip in ("bx", "p0", "p1", "p2", "sum"):
        while True:
            b_, c_, x_, s1, s2 = pick(5)
            w = pick(3)
            if skip == "p2":
                b_, c_, x_, s1, s2, w = hand["b"], hand["c"], hand["x"], hand["s1"], hand["s2"], hand["w"]
            (a, newest), (other, _) = conv(b_, c_, x_, s1, s2, w), conv(b_, c_, x_, s1, s2, w, skip)
            if a != other:
                cases["conv_" + skip] = dict(b=b_, c=c_, x=x_, state=[0.5, s1, s2], weight=w, expected=a,
                                             new_state=[s1, s2, newest], without=other)
                break
    dim, theta = 64, 1e6
    for skip in ("norm", "weight", "table", "left", "right"):
        while True:
            x, w = pick(dim), pick(dim)
            position = int(rng.integers(1, 200))
            inv = [f32(1.0) / (f32(theta) ** (f32(2 * i) / f32(dim))) for i in range(dim // 2)]
            cos = [float(np.cos(f32(position) * v, dtype=f32)) for v in inv]
            sin = [float(np.sin(f32(position) * v, dtype=f32)) for v in inv]
            a, b = qk_head(x, w, cos, sin, 1e-5), qk_head(x, w, cos, sin, 1e-5, skip)
            if a != b:
                cases["qk_" + skip] = dict(x=x, weight=w, cos=cos, sin=sin, eps=1e-5, expected=a, without=b)
                break
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rounding_cases.json")
    with open(path, "w") as f:
        json.dump(cases, f, indent=1)
    print(path, sorted(cases))


if __name__ == "__main__":
    main()
