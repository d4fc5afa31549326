"""Seeded counter-based input generator (flash-attn-rtx5060_amd/host/fa_inputs.c): Philox known answers,
bit-for-bit agreement with the independent pure-Python implementation that wrote tests/golden/inputs_kat.npz,
conversions, and sample statistics."""
import ctypes
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def philox(H, ctr, key):
    c = (ctypes.c_uint32 * 4)(*ctr)
    k = (ctypes.c_uint32 * 2)(*key)
    o = (ctypes.c_uint32 * 4)()
    H.fa_philox4x32_10(c, k, o)
    return tuple(o)


def test_philox4x32_10_known_answers(fa):
    """Known-answer vectors of Philox4x32-10 as published with Random123 (kat_vectors)."""
    H = fa.host_lib()
    assert philox(H, (0, 0, 0, 0), (0, 0)) == (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)
    f = 0xffffffff
    assert philox(H, (f, f, f, f), (f, f)) == (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)
    assert philox(H, (0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0)) == \
        (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)


def test_generator_matches_python_fixture_bit_for_bit(fa):
    H = fa.host_lib()
    z = np.load(os.path.join(GOLDEN, "inputs_kat.npz"))
    for seed, tensor in ((26, 0), (26, 1), (27, 2), (0x1234567890ABCDEF, 0)):
        got = np.array([H.fa_input_normal(seed, tensor, n) for n in range(64)], dtype=np.float32)
        assert np.array_equal(got.view(np.uint32), z[f"normal_{seed}_{tensor}"].view(np.uint32))
    big = (1 << 34) + 5
    got = np.array([H.fa_input_normal(26, 2, big + n) for n in range(8)], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32), z["normal_26_2_big_index"].view(np.uint32))
    sel = np.array([r for r in range(20000) if H.fa_input_row_selected(31, 0, r, 0.01)], dtype=np.int64)
    assert np.array_equal(sel, z["rows_selected_31_0_f0.01"])
    assert 120 <= len(sel) <= 280            # about 1 % of 20000
    q = fa.fill_normal(16, 8, 0, 31, 0, 0.5, 0.25, 8.0, nthreads=3)
    assert np.array_equal(q.reshape(1, 1, 16, 8), z["c5_q_bits"])


def test_fill_is_a_pure_function_of_the_index(fa):
    a = fa.fill_normal(64, 128, 0, 26, 1, nthreads=1)
    b = fa.fill_normal(64, 128, 0, 26, 1, nthreads=8)
    c = fa.fill_normal(32, 128, 0, 26, 1, nthreads=5)
    assert np.array_equal(a, b) and np.array_equal(a[:32], c)
    assert not np.array_equal(a, fa.fill_normal(64, 128, 0, 26, 2))      # tensors differ
    assert not np.array_equal(a, fa.fill_normal(64, 128, 0, 27, 1))      # seeds differ


def test_sample_statistics(fa):
    for dtype in (0, 1):
        x = fa.fill_normal(4096, 128, dtype, 29, 0)
        f = x.view(np.float16).astype(np.float64) if dtype == 0 else (x.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        assert abs(f.mean()) < 5e-3 and abs(f.std() - 1.0) < 5e-3
        assert abs(np.mean(f ** 3)) < 2e-2 and abs(np.mean(f ** 4) - 3.0) < 5e-2
    y = fa.fill_normal(20000, 8, 0, 31, 0, 0.5, 0.01, 8.0).view(np.float16).astype(np.float64)
    H = fa.host_lib()
    sel = np.array([bool(H.fa_input_row_selected(31, 0, r, 0.01)) for r in range(20000)])
    assert abs(y[~sel].std() - 0.5) < 5e-3 and abs(y[sel].std() - 4.0) < 0.15


def test_host_conversions_match_numpy_and_oracle(fa, oracle):
    H, O = fa.host_lib(), oracle.lib()
    rng = np.random.default_rng(3)
    xs = np.concatenate([rng.standard_normal(3000).astype(np.float32) * 2, (rng.standard_normal(1000) * 1e-5).astype(np.float32),
                         np.array([0.0, -0.0, 65504.0, 65520.0, 1e9, 2.0 ** -24, 2.0 ** -25, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11], dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([H.fa_f32_to_f16_bits(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)
    for x in xs[:500]:
        assert H.fa_f32_to_bf16_bits(float(x)) == O.fa_oracle_f32_to_bf16(float(x))
    for b in range(0, 65536, 11):
        f = np.array([b], dtype=np.uint16).view(np.float16).astype(np.float32)[0]
        g = H.fa_f16_bits_to_f32(b)
        assert (np.isnan(f) and np.isnan(g)) or np.float32(g) == f
