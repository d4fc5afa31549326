"""fa_fwd_split_static: the forward pass with key splits for callers that cannot allocate.  Its partial
results live in a file-scope device array instead of a caller's workspace; the kernels are fa_fwd's, so the
results must be the same bits.  Two calls in a row share the array; the second is smaller, so stale partial
rows of the first lie beyond (and between) what it writes."""
import ctypes

import numpy as np
import pytest

from parity_util import from_torch, make_inputs, to_torch

pytestmark = pytest.mark.gpu


def run_pair(fa, shape_q, S_kv, n_kv_heads, dtype, splits, causal, seed):
    import torch
    B, H, S, D = shape_q
    q_full, _, _ = make_inputs(fa, (B, H, S_kv, D), dtype, seed)
    _, k, v = make_inputs(fa, (B, n_kv_heads, S_kv, D), dtype, seed + 1)
    q = to_torch(np.ascontiguousarray(q_full[:, :, S_kv - S:, :]), dtype)
    k, v = to_torch(k, dtype), to_torch(v, dtype)
    L = fa.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for static in (False, True):
        o = torch.full_like(q, float("nan"))
        lse = torch.full((B, H, S), float("nan"), dtype=torch.float32, device="cuda")
        p = fa.make_params(B, H, S, D, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                           causal=causal, dtype=dtype, n_kv_heads=0 if n_kv_heads == H else n_kv_heads,
                           S_kv=0 if S_kv == S else S_kv, split_num=splits)
        need = L.fa_fwd_workspace_bytes(ctypes.byref(p))
        assert 0 < need <= L.fa_fwd_static_scratch_bytes()
        if static:
            assert L.fa_fwd_split_static(ctypes.byref(p), stream) == fa.FA_OK      # workspace fields stay NULL / 0
        else:
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            p.workspace, p.workspace_bytes = ws.data_ptr(), need
            assert L.fa_fwd(ctypes.byref(p), stream) == fa.FA_OK
        torch.cuda.synchronize()
        outs.append((from_torch(o), lse.cpu().numpy()))
    (o_ws, lse_ws), (o_st, lse_st) = outs
    assert np.isfinite(lse_st).all() and not np.isnan(o_st.view(np.float16 if dtype == 0 else np.uint16).astype(np.float32)).any()
    assert np.array_equal(o_ws, o_st) and np.array_equal(lse_ws, lse_st)
    return o_st, lse_st


def test_static_scratch_matches_workspace_twice_in_a_row(fa, oracle):
    # first call: decoding-shaped, grouped heads, 8 splits (1.06 MB of partial results)
    run_pair(fa, (4, 32, 1, 128), 4096, 8, 0, 8, True, seed=5)
    # second call: smaller in every dimension, other dtype; it must not see the first call's leftovers
    o, lse = run_pair(fa, (2, 8, 3, 64), 1000, 8, 1, 3, True, seed=9)
    # and it is right, not merely equal: against the oracle on the square problem's last rows
    B, H, S, D, S_kv = 2, 8, 3, 64, 1000
    q_full, _, _ = make_inputs(fa, (B, H, S_kv, D), 1, 9)
    _, k, v = make_inputs(fa, (B, H, S_kv, D), 1, 10)
    rows = np.array([bh * S_kv + r for bh in range(B * H) for r in range(S_kv - S, S_kv)], dtype=np.int64)
    o_ref, lse_ref = oracle.rows(q_full, k, v, rows, 1, None, True, -1, -1)
    d = np.abs(oracle.to_f32(o, 1).reshape(-1, D) - oracle.to_f32(o_ref, 1))
    assert d.max() <= 1.6e-2 and np.abs(lse.reshape(-1) - lse_ref).max() <= 8e-3
    # a square causal problem split five ways through the same entry point
    run_pair(fa, (1, 4, 640, 128), 640, 4, 0, 5, True, seed=11)


def test_static_scratch_refuses_what_does_not_fit(fa):
    import torch
    L = fa.lib()
    B, H, S, D, S_kv = 8, 32, 128, 128, 8192
    t = torch.zeros(16, dtype=torch.float16, device="cuda")
    p = fa.make_params(B, H, S, D, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), S_kv=S_kv, split_num=16)
    assert L.fa_fwd_workspace_bytes(ctypes.byref(p)) > L.fa_fwd_static_scratch_bytes()
    assert L.fa_fwd_split_static(ctypes.byref(p), None) == fa.FA_ERR_SCRATCH_LIMIT
