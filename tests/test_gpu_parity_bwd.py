"""GPU parity of the backward pass (fa_bwd, include/fa_bwd.h) against the fp64 gradient oracle.  The reference
has no backward pass; the oracle is pinned by torch autograd in fp64 and by finite differences of the forward
oracle (test_oracle_bwd.py).

The GPU works from the storage-type O and the fp32 logsumexp of its own forward pass, rounds P and dS to the
storage type for the matrix units and the three gradients to the storage type on the way out.  The bar, per
gradient: rel-L2 <= 1e-3 (fp16) / 8e-3 (bf16), max-abs <= 2e-3 / 1.6e-2 times max(1, max |gradient|): the forward
pass's bars, the absolute one scaled because gradients, unlike O, are not bounded by the inputs (measured:
rel-L2 3e-4 / 2.5e-3, max-abs 8e-4 / 5e-3 of the largest gradient)."""
import numpy as np
import pytest

from parity_util import from_torch, make_inputs, to_torch

pytestmark = pytest.mark.gpu

CASES = [
    # shape, dtype, causal, wl, wr
    ((1, 2, 128, 64), 0, False, -1, -1),
    ((1, 2, 128, 128), 0, True, -1, -1),
    ((2, 3, 256, 128), 0, True, -1, -1),
    ((1, 2, 384, 64), 0, True, -1, -1),
    ((1, 3, 512, 128), 0, False, -1, -1),
    ((1, 2, 640, 128), 0, True, 100, -1),
    ((1, 2, 512, 64), 0, False, 70, 50),
    ((1, 2, 512, 128), 0, False, -1, 33),
    ((2, 2, 384, 128), 1, True, -1, -1),
    ((1, 2, 256, 64), 1, False, -1, -1),
    ((1, 2, 768, 128), 1, False, 128, 0),
]


def grad_errors(got, want):
    got, want = got.astype(np.float64), want.astype(np.float64)
    return {"max_abs": float(np.max(np.abs(got - want))), "rel_l2": float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30)),
            "max_ref": float(np.max(np.abs(want))), "nonfinite": int(np.size(got) - np.isfinite(got).sum())}


def check(err, dtype, what):
    rel, mx = (1e-3, 2e-3) if dtype == 0 else (8e-3, 1.6e-2)
    assert err["nonfinite"] == 0, (what, err)
    assert err["rel_l2"] <= rel, (what, err)
    assert err["max_abs"] <= mx * max(1.0, err["max_ref"]), (what, err)


@pytest.mark.parametrize("shape,dtype,causal,wl,wr", CASES)
def test_gradients_against_the_fp64_oracle(fa, oracle, shape, dtype, causal, wl, wr):
    import torch
    q, k, v = make_inputs(fa, shape, dtype, seed=500 + shape[2])
    do, _, _ = make_inputs(fa, shape, dtype, seed=501 + shape[2])
    dq_ref, dk_ref, dv_ref = oracle.bwd_f64(q, k, v, do, dtype, None, causal, wl, wr)
    tq, tk, tv, tdo = (to_torch(x, dtype) for x in (q, k, v, do))
    o, lse = fa.flash_attention_forward(tq, tk, tv, causal=causal, window_left=wl, window_right=wr)
    dq, dk, dv = fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, causal=causal, window_left=wl, window_right=wr)
    torch.cuda.synchronize()
    for name, got, want in (("dQ", dq, dq_ref), ("dK", dk, dk_ref), ("dV", dv, dv_ref)):
        err = grad_errors(oracle.to_f32(from_torch(got), dtype), want)
        print(shape, dtype, causal, wl, wr, name, err, flush=True)
        check(err, dtype, name)


def test_against_torch_autograd_on_the_gpu(fa):
    """A larger problem than the CPU oracle finishes quickly: torch's fp32 attention and autograd on the GPU."""
    import torch
    B, H, S, D = 2, 4, 2048, 128
    g = torch.Generator(device="cuda").manual_seed(5)
    q, k, v, do = (torch.randn((B, H, S, D), device="cuda", generator=g).half() for _ in range(4))
    o, lse = fa.flash_attention_forward(q, k, v, causal=True)
    dq, dk, dv = fa.flash_attention_backward(q, k, v, o, lse, do, causal=True)
    qf, kf, vf = (t.float().requires_grad_(True) for t in (q, k, v))
    ref = torch.nn.functional.scaled_dot_product_attention(qf, kf, vf, is_causal=True)
    ref.backward(do.float())
    torch.cuda.synchronize()
    for name, got, want in (("dQ", dq, qf.grad), ("dK", dk, kf.grad), ("dV", dv, vf.grad)):
        err = grad_errors(got.float().cpu().numpy(), want.cpu().numpy())
        print("torch autograd", name, err, flush=True)
        check(err, 0, name)


def test_backward_refuses_what_it_does_not_cover(fa):
    import ctypes
    import torch
    t = torch.zeros((1, 1, 128, 64), dtype=torch.float16, device="cuda")
    lse = torch.zeros((1, 1, 128), dtype=torch.float32, device="cuda")
    L = fa.lib()
    ws = torch.empty(1024, dtype=torch.uint8, device="cuda")

    def params(S=128, d=64, ws_bytes=1024):
        ptr = t.data_ptr()
        return fa.make_bwd_params(1, 1, S, d, ptr, ptr, ptr, ptr, ptr, lse.data_ptr(), ptr, ptr, ptr,
                                  workspace_ptr=ws.data_ptr(), workspace_bytes=ws_bytes)
    assert L.fa_bwd_validate(ctypes.byref(params())) == fa.FA_OK
    assert L.fa_bwd(ctypes.byref(params(S=100)), None) == fa.FA_ERR_SEQLEN_MULTIPLE
    assert L.fa_bwd(ctypes.byref(params(d=96)), None) == fa.FA_ERR_HEAD_DIM
    assert L.fa_bwd(ctypes.byref(params(ws_bytes=511)), None) == fa.FA_ERR_WORKSPACE
    p = params(); p.dK = 0
    assert L.fa_bwd(ctypes.byref(p), None) == fa.FA_ERR_NULL_POINTER
