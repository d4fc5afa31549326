"""Writes the committed fixtures under tests/golden/.  Run from the repo root:  python tests/golden/make_golden.py

attn_small_f64.npz : inputs (storage bits) and fp64 brute-force attention outputs + logsumexp for three small
                     cases, computed here with numpy only (no oracle code, no reference code).
inputs_kat.npz     : first outputs of the seeded input generator, from the pure-Python re-implementation below
                     (Philox4x32-10 + Box-Muller in double), which tests compare bit-for-bit with the C generator.
"""
import math
import os
import struct

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
M32 = 0xFFFFFFFF


def philox4x32_10(ctr, key):
    c0, c1, c2, c3 = ctr
    k0, k1 = key
    for _ in range(10):
        p0 = 0xD2511F53 * c0
        p1 = 0xCD9E8D57 * c2
        c0, c1, c2, c3 = ((p1 >> 32) ^ c1 ^ k0) & M32, p1 & M32, ((p0 >> 32) ^ c3 ^ k1) & M32, p0 & M32
        k0 = (k0 + 0x9E3779B9) & M32
        k1 = (k1 + 0xBB67AE85) & M32
    return c0, c1, c2, c3


def f32(x):
    return struct.unpack("<f", struct.pack("<f", x))[0]


def normal(seed, tensor, index):
    group = index >> 2
    r = philox4x32_10((group & M32, group >> 32, tensor, 0), (seed & M32, seed >> 32))
    pair = (index & 3) >> 1
    u1 = (r[2 * pair] + 0.5) / 4294967296.0
    u2 = (r[2 * pair + 1] + 0.5) / 4294967296.0
    rad = math.sqrt(-2.0 * math.log(u1))
    ang = 6.283185307179586476925286766559 * u2
    return f32(rad * (math.sin(ang) if index & 1 else math.cos(ang)))


def row_selected(seed, tensor, row, fraction):
    r = philox4x32_10((row & M32, row >> 32, tensor, 1), (seed & M32, seed >> 32))
    return float(r[0]) < fraction * 4294967296.0


def to_bits(x, dtype):
    x = np.asarray(x, dtype=np.float32)
    if dtype == 0:
        return x.astype(np.float16).view(np.uint16)
    u = x.view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def to_f64(bits, dtype):
    if dtype == 0:
        return bits.view(np.float16).astype(np.float64)
    return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def gen(shape, dtype, seed, tensor, sigma=1.0, fraction=0.0, mult=1.0):
    B, H, S, D = shape
    out = np.empty(B * H * S * D, dtype=np.float32)
    for row in range(B * H * S):
        m = np.float32(sigma) * np.float32(mult) if row_selected(seed, tensor, row, fraction) else np.float32(sigma)
        for t in range(D):
            out[row * D + t] = np.float32(normal(seed, tensor, row * D + t)) * m
    return to_bits(out, dtype).reshape(shape)


def attention_f64(q, k, v, dtype, scale, causal, wl, wr):
    qf, kf, vf = (to_f64(x, dtype) for x in (q, k, v))
    S = q.shape[2]
    s = np.einsum("bhid,bhjd->bhij", qf, kf) * np.float64(np.float32(scale))
    i, j = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
    masked = np.zeros((S, S), dtype=bool)
    if causal:
        masked |= j > i
    if wl >= 0:
        masked |= i - j > wl
    if wr >= 0:
        masked |= j - i > wr
    s = np.where(masked, -np.inf, s)
    mx = s.max(axis=-1, keepdims=True)
    e = np.exp(s - mx)
    l = e.sum(axis=-1, keepdims=True)
    return np.einsum("bhij,bhjd->bhid", e / l, vf), (mx + np.log(l))[..., 0]


def main():
    cases = {
        # name: shape, dtype, causal, wl, wr, scale, seed
        "nc_f16": ((1, 1, 128, 64), 0, 0, -1, -1, 0.125, 101),
        "causal_f16": ((1, 1, 256, 64), 0, 1, -1, -1, 0.125, 102),
        "window_bf16": ((1, 1, 256, 128), 1, 1, 100, -1, 1.0 / math.sqrt(128), 103),
    }
    out = {}
    for name, (shape, dtype, causal, wl, wr, scale, seed) in cases.items():
        q, k, v = (gen(shape, dtype, seed, t) for t in range(3))
        o, lse = attention_f64(q, k, v, dtype, scale, bool(causal), wl, wr)
        out.update({f"{name}_q": q, f"{name}_k": k, f"{name}_v": v, f"{name}_o": o, f"{name}_lse": lse,
                    f"{name}_cfg": np.array([dtype, causal, wl, wr, np.float32(scale)], dtype=np.float64)})
    np.savez_compressed(os.path.join(HERE, "attn_small_f64.npz"), **out)

    kat = {}
    for seed, tensor in ((26, 0), (26, 1), (27, 2), (0x1234567890ABCDEF, 0)):
        kat[f"normal_{seed}_{tensor}"] = np.array([normal(seed, tensor, n) for n in range(64)], dtype=np.float32)
    big = (1 << 34) + 5
    kat["normal_26_2_big_index"] = np.array([normal(26, 2, big + n) for n in range(8)], dtype=np.float32)
    kat["rows_selected_31_0_f0.01"] = np.array([r for r in range(20000) if row_selected(31, 0, r, 0.01)], dtype=np.int64)
    kat["c5_q_bits"] = gen((1, 1, 16, 8), 0, 31, 0, 0.5, 0.25, 8.0)
    np.savez_compressed(os.path.join(HERE, "inputs_kat.npz"), **kat)


if __name__ == "__main__":
    main()
