"""Pins the CPU oracle (oracle/fa_oracle.c) against things other than itself.

The reference holds no golden vectors for this path, so the checks are: the literal restatement of the
reference's loop structure vs the streamed evaluation (bit-exact), the bit-level conversions vs numpy/torch,
closed forms and invariants chosen so that a dropped scale, a wrong mask edge, a transposed operand or a
missing rounding step fails at least one of them, brute-force fp64 fixtures under tests/golden, and torch's
scaled_dot_product_attention."""
import ctypes
import os

import numpy as np
import pytest

import oracle_binding as ob
from parity_util import numpy_keep_mask, numpy_philox4x32_10

F16, BF16 = ob.F16, ob.BF16
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def rand_bits(rng, shape, dtype, sigma=1.0):
    return ob.from_f32(rng.standard_normal(shape).astype(np.float32) * np.float32(sigma), dtype)


# ---------------------------------------------------------------- conversions
def test_f16_roundtrip_exhaustive():
    L = ob.lib()
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    for b, r in zip(bits[::7].tolist() + [0x0001, 0x03ff, 0x0400, 0x7bff, 0x7c00, 0xfc00, 0x8000], ref[::7].tolist() + [None] * 7):
        x = L.fa_oracle_f16_to_f32(b)
        if r is not None and not np.isnan(r):
            assert np.float32(x) == np.float32(r)
        if not np.isnan(x):
            assert L.fa_oracle_f32_to_f16(x) == b


def test_f32_to_f16_matches_numpy_rne():
    L = ob.lib()
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.standard_normal(4000).astype(np.float32),
        (rng.standard_normal(2000) * 1e-5).astype(np.float32),          # subnormal halves
        (rng.standard_normal(500) * 7e4).astype(np.float32),            # overflow edge
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                  1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 1.0 + 2.0 ** -11 + 2.0 ** -20, 2.0 ** -14, 2.0 ** -14 - 2.0 ** -26],
                 dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.fa_oracle_f32_to_f16(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_bf16_matches_torch_rne():
    import torch
    L = ob.lib()
    rng = np.random.default_rng(1)
    xs = np.concatenate([rng.standard_normal(4000).astype(np.float32) * 3,
                         np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, 0.0, -0.0, 3.3895e38], dtype=np.float32)])
    want = torch.from_numpy(xs).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([L.fa_oracle_f32_to_bf16(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(ob.from_f32(xs, BF16), want)
    back = np.array([L.fa_oracle_bf16_to_f32(int(b)) for b in want], dtype=np.float32)
    assert np.array_equal(back, ob.to_f32(want, BF16))


# ---------------------------------------------------------------- structure: literal vs streamed
@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("causal,wl,wr,alibi", [(False, -1, -1, False), (True, -1, -1, False), (False, 5, 5, False),
                                                (True, 7, -1, False), (False, 3, 11, True), (True, -1, -1, True)])
def test_streamed_equals_literal_bit_exact(dtype, causal, wl, wr, alibi):
    rng = np.random.default_rng(5)
    shape = (2, 3, 40, 24)
    q, k, v = (rand_bits(rng, shape, dtype) for _ in range(3))
    slopes = (-(2.0 ** (-8.0 / 3 * (np.arange(3) + 1)))).astype(np.float32) if alibi else None   # main.cu:41
    lit = ob.literal(q, k, v, dtype, None, causal, wl, wr, slopes)
    lit_scalar = ob.literal(q, k, v, dtype, None, causal, wl, wr, slopes, scalar=True)
    o, _ = ob.full(q, k, v, dtype, None, causal, wl, wr, slopes)
    o_scalar, _ = ob.full(q, k, v, dtype, None, causal, wl, wr, slopes, scalar=True)
    assert np.array_equal(lit, lit_scalar)
    assert np.array_equal(o, lit)           # AVX2/F16C fast path == reference loop structure
    assert np.array_equal(o_scalar, lit)    # bit-level scalar path too


def test_row_subset_equals_full():
    rng = np.random.default_rng(6)
    shape = (1, 2, 96, 32)
    q, k, v = (rand_bits(rng, shape, F16) for _ in range(3))
    o, lse = ob.full(q, k, v, F16, None, True, 20, -1)
    idx = np.array([191, 0, 95, 96, 7, 7, 150], dtype=np.int64)     # unsorted, repeated
    o_s, lse_s = ob.rows(q, k, v, idx, F16, None, True, 20, -1)
    assert np.array_equal(o_s, o.reshape(-1, 32)[idx])
    assert np.array_equal(lse_s, lse.reshape(-1)[idx])


# ---------------------------------------------------------------- the verifier's roundings, by an independent literal
# reference src/main.cu:189-263 restated with library half arithmetic only: numpy's float16 multiply IS the
# half x half -> half product of main.cu:193 and :259 (numpy computes it in fp32 and rounds once), torch's CPU
# bfloat16 multiply is the same for bf16; the sums are sequential fp32 adds in index order; expf is libm's.
# Nothing here calls into oracle/; a rounding dropped on either side of the softmax changes output bits.
def _libm_expf():
    import ctypes.util
    m = ctypes.CDLL(ctypes.util.find_library("m") or "libm.so.6")
    m.expf.restype = ctypes.c_float
    m.expf.argtypes = [ctypes.c_float]
    return m.expf


def _storage_mul(a32, b32, dtype):
    """Elementwise product of storage-type values (given as float32), rounded to the storage type, widened."""
    if dtype == F16:
        return (a32.astype(np.float16) * b32.astype(np.float16)).astype(np.float32)
    import torch
    ta, tb = torch.from_numpy(np.ascontiguousarray(a32)).to(torch.bfloat16), torch.from_numpy(np.ascontiguousarray(b32)).to(torch.bfloat16)
    return (ta * tb).to(torch.float32).numpy()


def _storage_round(x32, dtype):
    if dtype == F16:
        return x32.astype(np.float16).astype(np.float32)
    import torch
    return torch.from_numpy(np.ascontiguousarray(x32)).to(torch.bfloat16).to(torch.float32).numpy()


def independent_verifier(qb, kb, vb, dtype, scale, causal, window):
    """O bits [B,H,S,D] by the sequence of main.cu:176-266 (window < 0: none; symmetric, main.cu:220-229)."""
    expf = _libm_expf()
    B, H, S, D = qb.shape
    q, k, v = (ob.to_f32(x, dtype) for x in (qb, kb, vb))
    out = np.empty((B, H, S, D), dtype=np.uint16)
    scale = np.float32(scale)
    for b in range(B):
        for h in range(H):
            sc = np.zeros((S, S), dtype=np.float32)
            for t in range(D):                                      # main.cu:192-194, fp32 sum in index order
                sc = sc + _storage_mul(np.broadcast_to(q[b, h, :, t, None], (S, S)), np.broadcast_to(k[b, h, None, :, t], (S, S)), dtype)
            sc = sc * scale                                          # main.cu:195
            i, j = np.arange(S)[:, None], np.arange(S)[None, :]
            if causal:
                sc = np.where(j > i, np.float32(-np.inf), sc)        # main.cu:210-218
            if window >= 0:
                sc = np.where(np.abs(i - j) > window, np.float32(-np.inf), sc)   # main.cu:220-229
            p = np.zeros((S, S), dtype=np.float32)
            for r in range(S):                                      # main.cu:232-252
                mx = np.float32(-np.inf)
                for c in range(S):
                    mx = max(mx, sc[r, c])
                tot = np.float32(0.0)
                e = np.zeros(S, dtype=np.float32)
                for c in range(S):
                    e[c] = np.float32(expf(float(np.float32(sc[r, c] - mx))))
                    tot = np.float32(tot + e[c])
                p[r] = e / tot
            o = np.zeros((S, D), dtype=np.float32)
            for c in range(S):                                      # main.cu:255-263: half(p) * v as a half product
                o = o + _storage_mul(np.broadcast_to(p[:, c, None], (S, D)), np.broadcast_to(v[b, h, None, c, :], (S, D)), dtype)
            out[b, h] = ob.from_f32(o, dtype)                        # main.cu:261
    return out


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("causal,window", [(False, -1), (True, -1), (False, 3), (True, 5)])
def test_verifier_roundings_against_independent_half_arithmetic(dtype, causal, window):
    rng = np.random.default_rng(259 + 2 * int(causal) + window)
    shape = (1, 2, 24, 16)
    # values of full significand width, so p * v is inexact in the storage type almost everywhere; the second
    # head has the reference's own input distribution, U[0, 10) (main.cu:69-70)
    q, k, v = (rand_bits(rng, shape, dtype) for _ in range(3))
    for x in (q, k, v):
        x[0, 1] = ob.from_f32(rng.uniform(0.0, 10.0, size=shape[2:]).astype(np.float32), dtype)
    scale = 1.0 / np.sqrt(shape[3])
    want = independent_verifier(q, k, v, dtype, scale, causal, window)
    # the check has teeth: without the product rounding, or without rounding p, other bits come out
    lit = ob.literal(q, k, v, dtype, scale, causal, window, window)
    o, _ = ob.full(q, k, v, dtype, scale, causal, window, window)
    o_scalar, _ = ob.full(q, k, v, dtype, scale, causal, window, window, scalar=True)
    assert np.array_equal(lit, want)
    assert np.array_equal(o, want)
    assert np.array_equal(o_scalar, want)


def test_independent_half_arithmetic_is_sensitive_to_each_rounding():
    """The independent literal itself: leaving out the p -> half rounding or the half product changes bits,
    so agreement above cannot come from an insensitive input."""
    rng = np.random.default_rng(7)
    S, D = 24, 16
    p = rng.uniform(0, 1, (S, S)).astype(np.float32)
    p /= p.sum(1, keepdims=True)
    v = rng.standard_normal((S, D)).astype(np.float16).astype(np.float32)

    def pv(round_p, round_prod):
        o = np.zeros((S, D), dtype=np.float32)
        for c in range(S):
            pc = _storage_round(p[:, c, None], F16) if round_p else p[:, c, None]
            pr = pc * v[None, c, :]
            o = o + (_storage_round(pr, F16) if round_prod else pr)
        return ob.from_f32(o, F16)
    base = pv(True, True)
    assert not np.array_equal(base, pv(False, True))
    assert not np.array_equal(base, pv(True, False))


# ---------------------------------------------------------------- mask predicate, exhaustively
@pytest.mark.parametrize("causal,wl,wr", [(False, -1, -1), (True, -1, -1), (False, 4, 4), (True, 9, -1), (False, 0, 3),
                                          (False, -1, 0), (False, 6, -1), (True, 0, -1)])
def test_mask_predicate_via_one_hot_values(causal, wl, wr):
    """Q = 0 makes the softmax uniform over visible keys; V = identity makes O_ij = [j visible]/n_i, so the
    oracle's mask is read off its output and compared with the reference predicates
    (main.cu:213 j>i, main.cu:224 |i-j|>w, one-sided here)."""
    S = D = 48
    q = np.zeros((1, 1, S, D), dtype=np.uint16)
    k = rand_bits(np.random.default_rng(2), (1, 1, S, D), F16)
    v = ob.from_f32(np.eye(S, dtype=np.float32).reshape(1, 1, S, D), F16)
    o, lse = ob.full(q, k, v, F16, 0.25, causal, wl, wr)
    i, j = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
    vis = np.ones((S, S), dtype=bool)
    if causal:
        vis &= ~(j > i)
    if wl >= 0:
        vis &= ~(i - j > wl)
    if wr >= 0:
        vis &= ~(j - i > wr)
    n = vis.sum(axis=1)
    got = ob.to_f32(o, F16)[0, 0]
    assert np.array_equal(got > 0, vis)
    want = vis * ob.to_f32(ob.from_f32((1.0 / n).astype(np.float32), F16), F16)[:, None]
    assert np.array_equal(got, want.astype(np.float32))
    assert np.allclose(lse[0, 0], np.log(n), rtol=0, atol=2e-7 * np.log(S) + 1e-7)


# ---------------------------------------------------------------- closed forms
def test_constant_values_give_that_constant():
    rng = np.random.default_rng(3)
    shape = (1, 2, 64, 16)
    q, k = rand_bits(rng, shape, F16), rand_bits(rng, shape, F16)
    v = ob.from_f32(np.full(shape, 0.75, dtype=np.float32), F16)
    for causal, wl in ((False, -1), (True, -1), (True, 5)):
        o, _ = ob.full(q, k, v, F16, None, causal, wl, -1)
        # sum_j half(half(p_j)*0.75) differs from 0.75 only by the roundings of p: well inside 1e-3
        assert np.max(np.abs(ob.to_f32(o, F16) - 0.75)) <= 1e-3


def test_causal_row0_is_v0_and_lse_is_its_score():
    rng = np.random.default_rng(4)
    for dtype in (F16, BF16):
        shape = (2, 2, 32, 16)
        q, k, v = (rand_bits(rng, shape, dtype) for _ in range(3))
        scale = np.float32(0.3)
        o, lse = ob.full(q, k, v, dtype, scale, True)
        assert np.array_equal(o[:, :, 0, :], v[:, :, 0, :])
        qf, kf = ob.to_f32(q, dtype)[:, :, 0, :], ob.to_f32(k, dtype)[:, :, 0, :]
        prods = ob.to_f32(ob.from_f32(qf * kf, dtype), dtype)      # each product rounded to storage, main.cu:193
        acc = np.zeros(prods.shape[:2], dtype=np.float32)
        for t in range(prods.shape[-1]):
            acc = acc + prods[..., t]
        assert np.array_equal(lse[:, :, 0], acc * scale)           # max + logf(1) = the score itself


def test_zero_queries_average_visible_values():
    rng = np.random.default_rng(7)
    shape = (1, 1, 128, 32)
    q = np.zeros(shape, dtype=np.uint16)
    k, v = rand_bits(rng, shape, F16), rand_bits(rng, shape, F16)
    vf = ob.to_f32(v, F16)[0, 0].astype(np.float64)
    o, lse = ob.full(q, k, v, F16, None, True, 31, -1)
    for i in (0, 1, 30, 31, 32, 100, 127):
        lo = max(0, i - 31)
        assert abs(lse[0, 0, i] - np.log(i - lo + 1)) < 1e-6
        assert np.max(np.abs(ob.to_f32(o, F16)[0, 0, i] - vf[lo:i + 1].mean(axis=0))) < 2e-3


def test_dominant_key_selects_its_value():
    rng = np.random.default_rng(8)
    shape = (1, 1, 64, 32)
    q, k, v = (rand_bits(rng, shape, F16) for _ in range(3))
    kf = ob.to_f32(k, F16)
    kf[0, 0, 17] = 6.0 * ob.to_f32(q, F16)[0, 0, 40]          # key 17 aligned with query 40
    k = ob.from_f32(kf, F16)
    o, _ = ob.full(q, k, v, F16, 1.0)
    assert np.max(np.abs(ob.to_f32(o, F16)[0, 0, 40] - ob.to_f32(v, F16)[0, 0, 17])) < 2e-3


def test_equal_keys_give_uniform_weights():
    rng = np.random.default_rng(9)
    shape = (1, 1, 64, 32)
    q, v = rand_bits(rng, shape, F16), rand_bits(rng, shape, F16)
    k = np.broadcast_to(rand_bits(rng, (1, 1, 1, 32), F16), shape).copy()
    o, lse = ob.full(q, k, v, F16)
    mean = ob.to_f32(v, F16)[0, 0].astype(np.float64).mean(axis=0)
    assert np.max(np.abs(ob.to_f32(o, F16)[0, 0] - mean)) < 2e-3
    _, lse1 = ob.rows(q[:, :, :, :], k[:, :, :1, :].copy().reshape(1, 1, 1, 32).repeat(64, axis=2), v, np.arange(64), F16)
    assert np.allclose(lse[0, 0], lse1, atol=1e-6)


# ---------------------------------------------------------------- invariants
def test_key_shift_moves_lse_only():
    rng = np.random.default_rng(10)
    shape = (1, 2, 96, 16)
    q, k, v = (rand_bits(rng, shape, F16, 0.5) for _ in range(3))
    k = ob.from_f32(np.round(ob.to_f32(k, F16) * 64) / 64, F16)              # coarse grid: the shift below is exact
    cvec = np.array([0.5, -0.25] * 8, dtype=np.float32)
    k2 = ob.from_f32(ob.to_f32(k, F16) + cvec, F16)
    assert np.array_equal(ob.to_f32(k2, F16), ob.to_f32(k, F16) + cvec)      # the shift is exact in fp16 here
    idx = np.arange(2 * 96)
    o1, l1 = ob.rows_f64(q, k, v, idx, F16, None, True)
    o2, l2 = ob.rows_f64(q, k2, v, idx, F16, None, True)
    shift = (ob.to_f32(q, F16).astype(np.float64) @ cvec.astype(np.float64)).reshape(-1) * np.float32(1 / np.sqrt(16))
    assert np.allclose(l2 - l1, shift, atol=1e-12)
    assert np.allclose(o1, o2, atol=1e-12)


def test_key_permutation_invariance_non_causal():
    rng = np.random.default_rng(11)
    shape = (1, 1, 128, 32)
    q, k, v = (rand_bits(rng, shape, BF16) for _ in range(3))
    perm = rng.permutation(128)
    o1, l1 = ob.full(q, k, v, BF16)
    o2, l2 = ob.full(q, k[:, :, perm].copy(), v[:, :, perm].copy(), BF16)
    assert np.allclose(l1, l2, atol=5e-6)
    assert np.max(np.abs(ob.to_f32(o1, BF16) - ob.to_f32(o2, BF16))) <= 1.6e-2


def test_lse_bounds_and_output_hull():
    rng = np.random.default_rng(12)
    shape = (1, 2, 160, 32)
    q, k, v = (rand_bits(rng, shape, F16) for _ in range(3))
    idx = np.arange(2 * 160)
    o, lse = ob.rows_f64(q, k, v, idx, F16, None, True, 50, -1)
    s = np.einsum("hid,hjd->hij", ob.to_f32(q, F16)[0].astype(np.float64), ob.to_f32(k, F16)[0].astype(np.float64)) * np.float32(1 / np.sqrt(32))
    vf = ob.to_f32(v, F16)[0].astype(np.float64)
    for h in range(2):
        for i in range(160):
            lo = max(0, i - 50)
            row = s[h, i, lo:i + 1]
            L = lse[h * 160 + i]
            assert row.max() - 1e-12 <= L <= row.max() + np.log(len(row)) + 1e-12
            assert np.all(o[h * 160 + i] <= vf[h, lo:i + 1].max(axis=0) + 1e-12)
            assert np.all(o[h * 160 + i] >= vf[h, lo:i + 1].min(axis=0) - 1e-12)


# ---------------------------------------------------------------- independent implementations
def numpy_attention_f64(q, k, v, dtype, scale, causal, wl, wr):
    qf, kf, vf = (ob.to_f32(x, dtype).astype(np.float64) for x in (q, k, v))
    S = q.shape[2]
    s = np.einsum("bhid,bhjd->bhij", qf, kf) * np.float64(np.float32(scale))
    i, j = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
    m = np.zeros((S, S), dtype=bool)
    if causal:
        m |= j > i
    if wl >= 0:
        m |= i - j > wl
    if wr >= 0:
        m |= j - i > wr
    s = np.where(m, -np.inf, s)
    mx = s.max(axis=-1, keepdims=True)
    e = np.exp(s - mx)
    l = e.sum(axis=-1, keepdims=True)
    return np.einsum("bhij,bhjd->bhid", e / l, vf), (mx + np.log(l))[..., 0]


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("causal,wl,wr", [(False, -1, -1), (True, -1, -1), (True, 24, -1), (False, 16, 16)])
def test_against_numpy_f64_and_torch_sdpa(dtype, causal, wl, wr):
    import torch
    rng = np.random.default_rng(13)
    shape = (2, 2, 128, 64)
    q, k, v = (rand_bits(rng, shape, dtype) for _ in range(3))
    scale = 1 / np.sqrt(64)
    o_np, lse_np = numpy_attention_f64(q, k, v, dtype, scale, causal, wl, wr)
    idx = np.arange(2 * 2 * 128)
    o64, lse64 = ob.rows_f64(q, k, v, idx, dtype, None, causal, wl, wr)
    assert np.allclose(o64.reshape(shape), o_np, atol=1e-12)
    assert np.allclose(lse64.reshape(shape[:3]), lse_np, atol=1e-12)
    # third-party library cross-check (not reference code)
    tq, tk, tv = (torch.from_numpy(ob.to_f32(x, dtype).astype(np.float64)) for x in (q, k, v))
    S = 128
    i, j = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
    vis = np.ones((S, S), dtype=bool)
    if causal:
        vis &= j <= i
    if wl >= 0:
        vis &= i - j <= wl
    if wr >= 0:
        vis &= j - i <= wr
    o_t = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=torch.from_numpy(vis), scale=float(np.float32(scale)))
    assert np.allclose(o64.reshape(shape), o_t.numpy(), atol=1e-10)
    # the faithful path stays within the stated tolerance of the exact result
    o, lse = ob.full(q, k, v, dtype, None, causal, wl, wr)
    tol = 2e-3 if dtype == F16 else 1.6e-2
    assert np.max(np.abs(ob.to_f32(o, dtype) - o_np)) <= tol
    assert np.max(np.abs(lse - lse_np)) <= (2e-3 if dtype == F16 else 8e-3)   # bf16 products carry 2^-9 relative error


# ---------------------------------------------------------------- ALiBi (main.cu:200-207)
@pytest.mark.parametrize("causal", [False, True])
def test_alibi_closed_form_zero_queries(causal):
    """Q = 0 leaves only the bias: p_ij = exp(-slope_h |i-j|) / Z_i over the visible keys, and V = identity
    makes O = P.  A bias with the wrong sign, a missing |.|, the wrong head's slope or a bias applied after the
    mask's -inf would all change these numbers."""
    H, S = 3, 48
    slopes = np.array([0.5, -0.0625, 0.0], dtype=np.float32)      # both signs and a zero
    q = np.zeros((1, H, S, S), dtype=np.uint16)
    k = rand_bits(np.random.default_rng(3), (1, H, S, S), F16)
    v = np.broadcast_to(ob.from_f32(np.eye(S, dtype=np.float32), F16), (1, H, S, S)).copy()
    o, lse = ob.full(q, k, v, F16, None, causal, -1, -1, slopes)
    o64, lse64 = ob.rows_f64(q, k, v, np.arange(H * S), F16, None, causal, -1, -1, slopes)
    i, j = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
    for h in range(H):
        w = np.exp(-np.float64(slopes[h]) * np.abs(i - j))
        if causal:
            w = np.where(j <= i, w, 0.0)
        # normalise against the row maximum like a softmax does (exp(+big) overflows nothing here, S is small)
        Z = w.sum(axis=1, keepdims=True)
        assert np.allclose(o64.reshape(H, S, S)[h], w / Z, atol=1e-12)
        assert np.allclose(lse64.reshape(H, S)[h], np.log(Z[:, 0]), atol=1e-12)
        assert np.max(np.abs(ob.to_f32(o, F16)[0, h] - w / Z)) <= 6e-4       # p rounded to fp16: half an ulp below 1
        assert np.max(np.abs(lse[0, h] - np.log(Z[:, 0]))) <= 1e-5


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("causal,wl,wr", [(False, -1, -1), (True, -1, -1), (True, 24, -1), (False, 16, 16)])
def test_alibi_against_numpy_f64_and_torch_sdpa(dtype, causal, wl, wr):
    import torch
    rng = np.random.default_rng(17)
    shape = (2, 4, 128, 64)
    B, H, S, D = shape
    q, k, v = (rand_bits(rng, shape, dtype) for _ in range(3))
    slopes = np.array([2.0 ** -1, 2.0 ** -3, -(2.0 ** -4), 2.0 ** -8], dtype=np.float32)
    idx = np.arange(B * H * S)
    o64, lse64 = ob.rows_f64(q, k, v, idx, dtype, None, causal, wl, wr, slopes)
    i, j = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
    vis = np.ones((S, S), dtype=bool)
    if causal:
        vis &= j <= i
    if wl >= 0:
        vis &= i - j <= wl
    if wr >= 0:
        vis &= j - i <= wr
    bias = -slopes.astype(np.float64)[None, :, None, None] * np.abs(i - j)[None, None]
    bias = np.where(vis[None, None], bias, -np.inf)
    # numpy fp64, written out
    qf, kf, vf = (ob.to_f32(x, dtype).astype(np.float64) for x in (q, k, v))
    s = np.einsum("bhid,bhjd->bhij", qf, kf) * np.float64(np.float32(1 / np.sqrt(D))) + bias
    mx = s.max(axis=-1, keepdims=True)
    e = np.exp(s - mx)
    l = e.sum(axis=-1, keepdims=True)
    o_np, lse_np = np.einsum("bhij,bhjd->bhid", e / l, vf), (mx + np.log(l))[..., 0]
    assert np.allclose(o64.reshape(shape), o_np, atol=1e-12)
    assert np.allclose(lse64.reshape(shape[:3]), lse_np, atol=1e-12)
    # a third-party library with the bias as an additive float mask
    o_t = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(qf), torch.from_numpy(kf), torch.from_numpy(vf),
        attn_mask=torch.from_numpy(np.broadcast_to(bias, (B, H, S, S)).copy()), scale=float(np.float32(1 / np.sqrt(D))))
    assert np.allclose(o64.reshape(shape), o_t.numpy(), atol=1e-10)
    # the reference-order fp32 path stays close to the exact result (a steep slope concentrates the softmax on a
    # few keys, where the verifier's rounding of every p*v product to the storage type shows: up to 3e-3 in fp16)
    o, lse = ob.full(q, k, v, dtype, None, causal, wl, wr, slopes)
    assert np.max(np.abs(ob.to_f32(o, dtype) - o_np)) <= (3e-3 if dtype == F16 else 1.6e-2)
    assert np.max(np.abs(lse - lse_np)) <= (2e-3 if dtype == F16 else 8e-3)


# ---------------------------------------------------------------- dropout (flash_forward.h:248-265)
def test_dropout_philox_known_answers_and_mask_definition():
    L = ob.lib()

    def philox(ctr, key):
        c, k, o = (ctypes.c_uint32 * 4)(*ctr), (ctypes.c_uint32 * 2)(*key), (ctypes.c_uint32 * 4)()
        L.fa_oracle_philox4x32_10(c, k, o)
        return tuple(o)
    # Random123 known answers for Philox4x32-10
    f = 0xFFFFFFFF
    assert philox((0, 0, 0, 0), (0, 0)) == (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)
    assert philox((f, f, f, f), (f, f)) == (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)
    assert philox((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0)) == \
        (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)
    assert tuple(int(x) for x in numpy_philox4x32_10((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0))) == \
        (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)
    # the C decision function against the numpy one, all (i, j) of a 96 x 96 block, two heads, two thresholds
    for seed, bh, thr in ((48, 0, 26), (0x1234567890ABCDEF, 5, 128)):
        want = numpy_keep_mask(seed, bh, 96, thr)
        got = np.array([[L.fa_oracle_dropout_keep(seed, bh, i, j, thr) for j in range(96)] for i in range(96)], dtype=bool)
        assert np.array_equal(got, want)
        assert abs(want.mean() - (1 - thr / 256)) < 4 * np.sqrt(thr / 256 * (1 - thr / 256) / want.size)


@pytest.mark.parametrize("causal", [False, True])
def test_dropout_mask_read_back_through_identity_values(causal):
    """Q = 0 makes P uniform over the n_i visible keys; V = identity then gives O_ij = keep_ij / (n_i (1-p)):
    the mask the oracle applied is read off its output and compared with the numpy definition, and the
    logsumexp must be that of the run without dropout."""
    H, S, thr, seed = 2, 64, 77, 0xC0FFEE
    q = np.zeros((1, H, S, S), dtype=np.uint16)
    k = rand_bits(np.random.default_rng(3), (1, H, S, S), F16)
    v = np.broadcast_to(ob.from_f32(np.eye(S, dtype=np.float32), F16), (1, H, S, S)).copy()
    o64, lse64 = ob.rows_f64(q, k, v, np.arange(H * S), F16, None, causal, -1, -1, None, dropout=(thr, seed))
    o, lse = ob.full(q, k, v, F16, None, causal, -1, -1, None, dropout=(thr, seed))
    _, lse_plain = ob.full(q, k, v, F16, None, causal, -1, -1)
    assert np.array_equal(lse, lse_plain)
    i, j = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
    vis = (j <= i) if causal else np.ones((S, S), dtype=bool)
    n = vis.sum(axis=1, keepdims=True)
    for h in range(H):
        want = np.where(vis & numpy_keep_mask(seed, h, S, thr), 1.0 / (n * (1 - thr / 256)), 0.0)
        assert np.allclose(o64.reshape(H, S, S)[h], want, atol=1e-12)
        assert np.max(np.abs(ob.to_f32(o, F16)[0, h] - want)) <= 1e-3 * np.maximum(want.max(), 1.0)


def test_dropout_threshold_zero_is_no_dropout_and_streamed_equals_literal():
    rng = np.random.default_rng(21)
    shape = (1, 2, 72, 32)
    q, k, v = (rand_bits(rng, shape, F16) for _ in range(3))
    o0, l0 = ob.full(q, k, v, F16, None, True, -1, -1)
    o1, l1 = ob.full(q, k, v, F16, None, True, -1, -1, None, dropout=(0, 12345))
    assert np.array_equal(o0, o1) and np.array_equal(l0, l1)
    for dtype in (F16, BF16):
        lit = ob.literal(q, k, v, dtype, None, True, 40, -1, None, dropout=(60, 9))
        o, _ = ob.full(q, k, v, dtype, None, True, 40, -1, None, dropout=(60, 9))
        o_s, _ = ob.full(q, k, v, dtype, None, True, 40, -1, None, scalar=True, dropout=(60, 9))
        assert np.array_equal(o, lit) and np.array_equal(o_s, lit)


def test_golden_fixture_f64():
    """tests/golden/attn_small_f64.npz was written by tests/golden/make_golden.py with a numpy fp64 brute force
    (no oracle code involved)."""
    z = np.load(os.path.join(GOLDEN, "attn_small_f64.npz"))
    for name in ("nc_f16", "causal_f16", "window_bf16"):
        q, k, v = z[f"{name}_q"], z[f"{name}_k"], z[f"{name}_v"]
        dtype, causal, wl, wr, scale = (int(x) if n < 4 else float(x) for n, x in enumerate(z[f"{name}_cfg"]))
        B, H, S, D = q.shape
        idx = np.arange(B * H * S)
        o64, lse64 = ob.rows_f64(q, k, v, idx, dtype, scale, bool(causal), wl, wr)
        assert np.allclose(o64.reshape(q.shape), z[f"{name}_o"], atol=1e-12)
        assert np.allclose(lse64.reshape(B, H, S), z[f"{name}_lse"], atol=1e-12)
        o, lse = ob.full(q, k, v, dtype, scale, bool(causal), wl, wr)
        assert np.max(np.abs(ob.to_f32(o, dtype) - z[f"{name}_o"])) <= (2e-3 if dtype == F16 else 1.6e-2)
        assert np.max(np.abs(lse - z[f"{name}_lse"])) <= (2e-3 if dtype == F16 else 8e-3)


def test_bad_arguments_are_rejected():
    q = np.zeros((1, 1, 8, 8), dtype=np.uint16)
    import ctypes
    c = ob.Cfg(1, 1, 8, 8, 7, 1.0, 0, -1, -1, None)     # bad dtype
    assert ob.lib().fa_oracle_full(ctypes.byref(c), q.ctypes.data, q.ctypes.data, q.ctypes.data, q.ctypes.data, None, 1) == -1
    c = ob.Cfg(1, 1, 8, 8, 0, 1.0, 0, -1, -1, None)
    idx = np.array([8], dtype=np.int64)                  # out of range row
    assert ob.lib().fa_oracle_rows(ctypes.byref(c), q.ctypes.data, q.ctypes.data, q.ctypes.data, idx.ctypes.data, 1, None, None, 1) == -1
