"""The checking build of the forward kernels (libfa_fwd_gfx950_check.so, -DFA_CHECK_RING): every wave asserts in
every iteration, in front of its work and again behind it, that the LDS stages it reads hold the key tiles the
iteration expects (the invariants of the global->LDS ring that replaces the reference's mbarrier ring,
flash_forward.h:95-111).  The product library carries none of this code.  Here: the checks run, find nothing, and the
outputs are the product library's bits, over the kernel flavours and schedules; and a library whose ring is broken
on purpose (a K tile requested into the stage that is being read) is caught by the same checks."""
import ctypes
import os

import numpy as np
import pytest

from parity_util import make_inputs, to_torch

pytestmark = pytest.mark.gpu


def load(fa, name):
    import torch  # noqa: F401  (PyTorch's HIP runtime first, as for the product library)
    path = os.path.join(os.path.dirname(fa.LIB_PATH), name)
    assert os.path.exists(path), f"{path} is missing: run make -C flash-attn-rtx5060_amd"
    L = ctypes.CDLL(path)
    L.fa_fwd.argtypes = [ctypes.POINTER(fa.FaFwdParams), ctypes.c_void_p]
    L.fa_debug_ring_counts.argtypes = [ctypes.POINTER(ctypes.c_ulonglong)] * 2
    return L


def counts(L):
    c, v = ctypes.c_ulonglong(0), ctypes.c_ulonglong(0)
    assert L.fa_debug_ring_counts(ctypes.byref(c), ctypes.byref(v)) == 0
    return c.value, v.value


CASES = [
    # B, H, Hk, S, Skv, D, dtype, causal, wl, wr, bshd, dropout, splits
    (1, 4, 4, 256, 256, 64, 0, False, -1, -1, False, 0.0, 1),        # c1's shape: the 4-wave, 2-stage kernel
    (2, 64, 64, 2048, 2048, 64, 0, True, -1, -1, False, 0.0, 1),     # 8-wave, 3 stages, several items per workgroup
    (2, 32, 32, 4096, 4096, 128, 0, True, -1, -1, False, 0.0, 1),
    (1, 32, 32, 4096, 4096, 128, 1, True, 512, -1, False, 0.0, 1),   # window: waves of a block walk different tile ranges
    (1, 16, 16, 2048, 2048, 128, 0, False, 100, 300, False, 0.0, 1),
    (2, 32, 8, 2048, 2048, 128, 0, True, -1, -1, True, 0.0, 1),      # strided flavour, grouped heads, [B,S,H,D]
    (1, 8, 2, 1000, 1500, 64, 1, True, -1, -1, True, 0.0, 1),        # general flavour: ragged lengths
    (2, 8, 8, 1024, 1024, 128, 0, True, -1, -1, False, 0.2, 1),      # dropout flavour
    (4, 8, 2, 3, 4096, 128, 0, True, -1, -1, False, 0.0, 4),         # key splits, packed heads
]


@pytest.mark.parametrize("case", CASES)
def test_ring_invariants_hold(fa, case):
    import torch
    B, H, Hk, S, Skv, D, dtype, causal, wl, wr, bshd, dropout, splits = case
    L = load(fa, "libfa_fwd_gfx950_check.so")
    g = torch.Generator(device="cuda").manual_seed(B * 1000 + S)
    tdt = torch.bfloat16 if dtype else torch.float16

    def make(h, s):
        t = torch.randn((B, s, h, D) if bshd else (B, h, s, D), device="cuda", generator=g).to(tdt)
        return t.transpose(1, 2) if bshd else t
    q, k, v = make(H, S), make(Hk, Skv), make(Hk, Skv)
    counts(L)                                       # start from zero
    for sched in (1, 2, 3):
        want, want_lse = fa.flash_attention_forward(q, k, v, causal=causal, window_left=wl, window_right=wr, sched=sched,
                                                    dropout_prob=dropout, seed=7, splits=splits)
        out = torch.full_like(want, float("nan"))
        lse = torch.full_like(want_lse, float("nan"))
        st = lambda t: tuple(t.stride()[:3])
        p = fa.make_params(B, H, S, D, q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), None, causal, wl, wr,
                           dtype, sched, 0, 0 if Hk == H else Hk, st(q), st(k), st(v), st(out), dropout_prob=dropout, seed=7,
                           S_kv=0 if Skv == S else Skv)
        ws = None
        if splits > 1:
            p.split_num = splits
            need = fa.lib().fa_fwd_workspace_bytes(ctypes.byref(p))
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            p.workspace, p.workspace_bytes = ws.data_ptr(), need
        assert L.fa_fwd(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
        checked, bad = counts(L)
        print(case, "sched", sched, "comparisons", checked, "violations", bad, flush=True)
        assert checked > 0 and bad == 0
        assert torch.equal(out.contiguous().view(torch.int16), want.contiguous().view(torch.int16)) and torch.equal(lse, want_lse)


def test_a_broken_ring_is_caught(fa):
    """The negative control: the same checks in a library whose steady iterations request every K tile into the stage
    that is being read.  No access leaves the workgroup's LDS; the result is merely wrong, and the checks say so."""
    import torch
    L = load(fa, "libfa_fwd_gfx950_check_broken.so")
    shape, dtype = (1, 32, 4096, 128), 0
    q, k, v = (to_torch(x, dtype) for x in make_inputs(fa, shape, dtype, seed=77))
    out = torch.empty_like(q)
    lse = torch.empty(shape[:3], dtype=torch.float32, device="cuda")
    p = fa.make_params(*shape, q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), causal=True, dtype=dtype)
    counts(L)
    assert L.fa_fwd(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    checked, bad = counts(L)
    print("broken ring: comparisons", checked, "violations", bad, flush=True)
    assert checked > 0 and bad > 0
