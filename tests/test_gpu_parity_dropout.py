"""GPU parity of dropout (reference src/flash_forward.h:248-265; the reference's own verifier skips dropout
runs, src/main.cu:102).  The kept keys are a counter-based function of (seed, head, query, key) that the CPU
oracle and a numpy implementation replay, so the GPU output is compared element by element, not statistically."""
import numpy as np
import pytest

from parity_util import assert_within, errors, from_torch, make_inputs, numpy_keep_mask, sample_rows, to_torch

pytestmark = pytest.mark.gpu

CASES = [
    # shape, dtype, causal, wl, wr, p, seed
    ((1, 4, 256, 64), 0, False, -1, -1, 0.1, 48),
    ((2, 2, 512, 128), 0, True, -1, -1, 0.1, 48),
    ((1, 2, 384, 128), 0, True, -1, -1, 0.5, 0x123456789ABCDEF),
    ((1, 3, 640, 64), 1, True, 100, -1, 0.25, 7),
    ((1, 2, 1024, 128), 1, False, 128, 128, 0.1, 8),
    ((2, 3, 333, 128), 0, True, -1, -1, 0.2, 9),          # ragged length
    ((1, 2, 200, 64), 0, False, -1, -1, 0.9, 10),         # almost everything dropped
]


@pytest.mark.parametrize("shape,dtype,causal,wl,wr,p,seed", CASES)
def test_small_full_tensor_dropout(fa, oracle, shape, dtype, causal, wl, wr, p, seed):
    thr = fa.lib().fa_dropout_threshold(p)
    q, k, v = make_inputs(fa, shape, dtype, seed=900 + shape[2])
    o_ref, lse_ref = oracle.full(q, k, v, dtype, None, causal, wl, wr, None, dropout=(thr, seed))
    o, lse = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype), causal=causal,
                                        window_left=wl, window_right=wr, dropout_prob=p, seed=seed)
    err = errors(oracle.to_f32(from_torch(o), dtype), oracle.to_f32(o_ref, dtype), lse.cpu().numpy(), lse_ref)
    print(shape, dtype, causal, wl, wr, p, err)
    # kept probabilities are multiplied by 1/(1-p), and so is every rounding difference
    scale = 256.0 / (256 - thr)
    assert err["nonfinite"] == 0
    assert err["max_abs"] <= (2e-3 if dtype == 0 else 1.6e-2) * scale, err
    assert err["rel_l2"] <= (1e-3 if dtype == 0 else 8e-3) * scale, err
    assert err["lse_abs"] <= (2e-3 if dtype == 0 else 8e-3), err
    # a different seed gives a different result, the same seed the same bits
    o2, _ = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype), causal=causal,
                                       window_left=wl, window_right=wr, dropout_prob=p, seed=seed)
    o3, _ = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype), causal=causal,
                                       window_left=wl, window_right=wr, dropout_prob=p, seed=seed + 1)
    import torch
    torch.cuda.synchronize()
    assert torch.equal(o.view(torch.int16), o2.view(torch.int16))
    assert not torch.equal(o.view(torch.int16), o3.view(torch.int16))


def test_dropout_mask_read_back_on_gpu(fa):
    """Q = 0 and V[j, t] = [j mod D == t]: O[i, t] = sum of keep_ij / (n_i (1-p)) over the visible keys
    j = t (mod D).  numpy evaluates that from the published definition of the decision, no oracle code involved;
    run at S = 1024 so that queries, key blocks and heads all vary."""
    import torch
    B, H, S, D, p, seed = 2, 3, 1024, 64, 0.3, 0xDEADBEEF
    thr = fa.lib().fa_dropout_threshold(p)
    q = torch.zeros((B, H, S, D), dtype=torch.float16, device="cuda")
    k = torch.randn((B, H, S, D), dtype=torch.float16, device="cuda")
    onehot = np.zeros((S, D))
    onehot[np.arange(S), np.arange(S) % D] = 1.0
    v = torch.from_numpy(onehot.astype(np.float16)).cuda().expand(B, H, S, D).contiguous()
    i, j = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
    for causal in (False, True):
        o, lse = fa.flash_attention_forward(q, k, v, causal=causal, dropout_prob=p, seed=seed)
        torch.cuda.synchronize()
        o, lse = o.float().cpu().numpy(), lse.cpu().numpy()
        vis = (j <= i) if causal else np.ones((S, S), dtype=bool)
        n = vis.sum(axis=1, keepdims=True)
        for bh in range(B * H):
            keep = numpy_keep_mask(seed, bh, S, thr)
            want = np.where(vis & keep, 1.0 / (n * (1 - thr / 256)), 0.0) @ onehot
            got = o.reshape(B * H, S, D)[bh]
            assert np.max(np.abs(got - want)) <= 2e-3 * max(1.0, want.max()), (causal, bh)
            assert np.max(np.abs(lse.reshape(B * H, S)[bh] - np.log(n[:, 0]))) <= 1e-3


def test_dropout_on_the_headline_shape(fa, oracle):
    """c3's shape with p = 0.1: sampled rows against the oracle, through run_flash_attention's argument list
    (Is_dropout = 1, seed 48 as in the reference's main(), main.cu:93)."""
    import torch
    shape = (2, 32, 8192, 128)
    B, H, S, D = shape
    q, k, v = make_inputs(fa, shape, 0, seed=29)
    tq, tk, tv = (to_torch(x, 0) for x in (q, k, v))
    o = torch.full_like(tq, float("nan"))
    lse = torch.empty((B, H, S), dtype=torch.float32, device="cuda")
    assert fa.run_flash_attention(B, H, S, D, tq, tk, tv, o, lse, None, True, True, False, False, 0, None, 0.1, None) == fa.FA_OK
    thr = fa.lib().fa_dropout_threshold(0.1)
    rows = sample_rows(shape, 1024, 29)
    o_ref, lse_ref = oracle.rows(q, k, v, rows, 0, None, True, -1, -1, None, dropout=(thr, 48))
    err = errors(oracle.to_f32(from_torch(o), 0).reshape(-1, D)[rows], oracle.to_f32(o_ref, 0),
                 lse.cpu().numpy().reshape(-1)[rows], lse_ref)
    print("c3 dropout", err)
    assert bool(torch.isfinite(o.float()).all())
    assert err["max_abs"] <= 2e-3 * 256 / (256 - thr) and err["rel_l2"] <= 1e-3 * 256 / (256 - thr) and err["lse_abs"] <= 2e-3, err
