"""GPU parity: the HIP forward pass, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Tolerances are stated in parity_util.TOL."""
import numpy as np
import pytest

from parity_util import assert_within, errors, from_torch, make_inputs, sample_rows, to_torch

pytestmark = pytest.mark.gpu

SMALL = [
    # shape (B,H,S,D), dtype, causal, wl, wr
    ((1, 4, 256, 64), 0, False, -1, -1),      # config 1
    ((1, 2, 256, 64), 0, True, -1, -1),
    ((1, 2, 512, 128), 0, False, -1, -1),
    ((1, 2, 512, 128), 0, True, -1, -1),
    ((2, 2, 384, 128), 0, True, -1, -1),      # S not a multiple of the 256-row block
    ((1, 2, 640, 64), 1, True, -1, -1),
    ((1, 2, 1024, 128), 1, True, 200, -1),    # left window + causal
    ((1, 2, 1024, 128), 0, False, 128, 128),  # the reference's symmetric local window
    ((1, 2, 1024, 64), 0, False, 100, 37),
    ((1, 1, 1024, 128), 1, False, -1, 0),     # right window 0 == causal
    ((1, 2, 768, 128), 0, True, 0, -1),       # each query sees only itself
]


@pytest.mark.parametrize("shape,dtype,causal,wl,wr", SMALL)
def test_small_full_tensor(fa, oracle, shape, dtype, causal, wl, wr):
    q, k, v = make_inputs(fa, shape, dtype, seed=1234 + shape[2] + dtype)
    o_ref, lse_ref = oracle.full(q, k, v, dtype, None, causal, wl, wr)
    o, lse = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype),
                                        causal=causal, window_left=wl, window_right=wr)
    err = errors(oracle.to_f32(from_torch(o), dtype), oracle.to_f32(o_ref, dtype), lse.cpu().numpy(), lse_ref)
    print(shape, dtype, causal, wl, wr, err)
    assert_within(err, dtype, f"{shape} dtype={dtype} causal={causal} w=({wl},{wr})")
