"""Query rows that see only a few keys.

Under a causal-type mask the rows with at most 32 visible keys are computed in the arithmetic of the
reference's CPU verifier (every q*k and p*v product rounded to the storage type, reference src/main.cu:193,259)
unless fa_fwd_params.exact_first_rows is set.  Checked here: those rows agree with the oracle bit for bit
(up to the last-place difference between the device's and the host's expf, which survives the rounding of p
only rarely); the same holds when the queries are the last rows of a longer key sequence; with
exact_first_rows the whole output meets the usual tolerance against exact (fp64) attention; and for masks
that leave EVERY row with only a few keys (windows narrower than 32), where no row takes the verifier's
arithmetic unless it is among the first 32, the documented bound holds: the tolerance, or one output ulp
where the output is so large that one ulp exceeds it."""
import numpy as np
import pytest

from parity_util import TOL, assert_within, errors, from_torch, make_inputs, to_torch

pytestmark = pytest.mark.gpu


def ulp(x, dtype):
    """Spacing of the storage type at |x| (fp16: 11-bit significand, bf16: 8-bit)."""
    bits = 10 if dtype == 0 else 7
    e = np.floor(np.log2(np.maximum(np.abs(x), 2.0 ** -14)))
    return 2.0 ** (e - bits)


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("shape,wl,seed,sched", [((2, 4, 256, 128), -1, 29, 0), ((1, 8, 384, 64), -1, 7, 0), ((1, 4, 256, 128), 9, 3, 0),
                                                 ((2, 32, 1024, 128), -1, 29, 0),
                                                 # the path dealt in one, two and four parts, in workgroups of 128 and of 256
                                                 # rows, under every schedule (several passes over the resident grid included)
                                                 ((1, 4, 128, 64), -1, 5, 0), ((1, 4, 512, 128), -1, 6, 2), ((4, 64, 2048, 64), -1, 28, 0),
                                                 ((4, 64, 2048, 64), 40, 28, 3), ((8, 80, 768, 128), -1, 9, 2), ((8, 80, 512, 64), -1, 10, 3),
                                                 ((8, 80, 256, 64), -1, 11, 1),
                                                 # other lengths (the general kernels deal the rows the same way): two, four
                                                 # and eight parts, one block alone, every schedule
                                                 ((2, 8, 200, 128), -1, 12, 0), ((4, 64, 500, 64), -1, 13, 2), ((4, 64, 1000, 128), -1, 14, 0),
                                                 ((4, 64, 2047, 64), 100, 15, 2), ((2, 16, 1100, 128), -1, 16, 3), ((8, 80, 300, 64), -1, 17, 1),
                                                 ((1, 4, 100, 128), -1, 18, 0)])
def test_first_rows_are_the_verifiers_bits(fa, oracle, dtype, shape, wl, seed, sched):
    B, H, S, D = shape
    q, k, v = make_inputs(fa, shape, dtype, seed)
    o, lse = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype), causal=True, window_left=wl, sched=sched)
    rows = np.array([bh * S + r for bh in range(B * H) for r in range(32)], dtype=np.int64)
    o_ref, lse_ref = oracle.rows(q, k, v, rows, dtype, None, True, wl, -1)
    got = from_torch(o).reshape(-1, D)[rows]
    differ = np.count_nonzero(got != o_ref)
    # the same sequence of operations; only expf may differ in the last place between device and host
    assert differ <= max(1, got.size // 2000), f"{differ} of {got.size} elements differ"
    # where they differ, p moved by one place of the storage type: one ulp of the output, or of 1 where the
    # output is a small difference of larger terms
    d = np.abs(oracle.to_f32(got, dtype).astype(np.float64) - oracle.to_f32(o_ref, dtype))
    assert np.all(d <= ulp(np.maximum(np.abs(oracle.to_f32(o_ref, dtype)), 1.0), dtype) * 1.0001)
    assert np.max(np.abs(lse.cpu().numpy().reshape(-1)[rows] - lse_ref)) <= 1e-5


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("S,S_kv", [(128, 131), (64, 80), (200, 231), (5, 36), (300, 301)])
def test_first_rows_behind_a_few_earlier_keys(fa, oracle, dtype, S, S_kv):
    """Queries at the end of a slightly longer key sequence (query i at position i + S_kv - S): the rows at
    positions below 32 still see few keys and still take the verifier's arithmetic."""
    H, D = 3, 128
    q_full, k, v = make_inputs(fa, (1, H, S_kv, D), dtype, 41 + S)
    q = np.ascontiguousarray(q_full[:, :, S_kv - S:, :])
    o, lse = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype), causal=True)
    rows = np.array([h * S_kv + r for h in range(H) for r in range(S_kv - S, S_kv)], dtype=np.int64)
    o_ref, lse_ref = oracle.rows(q_full, k, v, rows, dtype, None, True, -1, -1)
    got = oracle.to_f32(from_torch(o), dtype).reshape(-1, D)
    err = errors(got, oracle.to_f32(o_ref, dtype), lse.cpu().numpy().reshape(-1), lse_ref)
    print(S, S_kv, dtype, err)
    assert_within(err, dtype, f"S={S} S_kv={S_kv}")
    few = np.array([n for n, r in enumerate(rows) if r % S_kv < 32])
    if few.size:
        differ = np.count_nonzero(from_torch(o).reshape(-1, D)[few] != o_ref[few])
        assert differ <= max(1, few.size * D // 2000)


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("causal,wl,wr", [(True, 0, -1), (True, 4, -1), (True, 15, -1), (False, 0, 0), (False, 4, 4),
                                          (False, 15, 15), (False, 15, 3)])
def test_narrow_windows_documented_bound(fa, oracle, dtype, causal, wl, wr):
    """Every row sees at most 31 keys.  Rows beyond the first 32 (and all rows of a two-sided window) accumulate
    exact products while the verifier rounds each one, and with so few keys an output can be several units
    large: the stated bound is the tolerance or one output ulp, whichever is larger, and the usual rel-L2."""
    shape = (1, 4, 512, 128)
    q, k, v = make_inputs(fa, shape, dtype, 77 + wl)
    o_ref, lse_ref = oracle.full(q, k, v, dtype, None, causal, wl, wr)
    o, lse = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype),
                                        causal=causal, window_left=wl, window_right=wr)
    ref = oracle.to_f32(o_ref, dtype)
    got = oracle.to_f32(from_torch(o), dtype)
    err = errors(got, ref, lse.cpu().numpy(), lse_ref)
    print(dtype, causal, wl, wr, err)
    assert err["nonfinite"] == 0
    bound = np.maximum(TOL[dtype]["max_abs"], ulp(ref, dtype) * 1.0001)
    assert np.all(np.abs(got.astype(np.float64) - ref) <= bound)
    assert err["rel_l2"] <= TOL[dtype]["rel_l2"] and err["lse_abs"] <= TOL[dtype]["lse_abs"]


@pytest.mark.parametrize("dtype", [0, 1])
def test_exact_first_rows_against_fp64(fa, oracle, dtype):
    """exact_first_rows = 1: no row takes the verifier's rounded products; the whole output, first rows
    included, is within the usual tolerance of exact attention, and the logsumexp of the
    first rows is the exact one (what fa_bwd recomputes P from)."""
    shape = (2, 4, 256, 128)
    B, H, S, D = shape
    q, k, v = make_inputs(fa, shape, dtype, 29)
    rows = np.arange(B * H * S, dtype=np.int64)
    o64, lse64 = oracle.rows_f64(q, k, v, rows, dtype, None, True, -1, -1)
    o, lse = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype), causal=True,
                                        exact_first_rows=True)
    got = oracle.to_f32(from_torch(o), dtype).reshape(-1, D)
    # p rounded to the storage type before the second product, one rounding of the result
    err = errors(got, o64.astype(np.float32), lse.cpu().numpy().reshape(-1), lse64.astype(np.float32))
    print(dtype, err)
    assert_within(err, dtype, "exact_first_rows vs fp64")
    assert err["rel_l2"] <= (4e-4 if dtype == 0 else 3e-3)
    assert err["lse_abs"] <= 2e-5
    # and it differs from the default path where the verifier's rounding matters
    o_default, _ = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype), causal=True)
    assert np.count_nonzero(from_torch(o_default).reshape(-1, D)[:32] != from_torch(o).reshape(-1, D)[:32]) > 0
