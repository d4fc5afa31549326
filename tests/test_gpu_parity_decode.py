"""GPU parity for query and key lengths that differ (the queries are the last S of S_kv positions: decoding,
chunked prefill) and for key splits merged by a second kernel (the reference's dead `split_num` field,
include/utils.h:164).

The oracle evaluates square problems only.  Rows are independent, so a problem with S queries at positions
S_kv - S .. S_kv - 1 is exactly rows S_kv - S .. S_kv - 1 of the square S_kv problem whose first query rows
hold anything at all: the tests pad Q in front and ask the oracle for those rows."""
import numpy as np
import pytest

from parity_util import assert_within, errors, from_torch, make_inputs, to_torch

pytestmark = pytest.mark.gpu


def oracle_rect(oracle, q, k, v, dtype, causal, wl, wr, slopes=None, dropout=(0, 0)):
    """q [B,H,S,D], k/v [B,Hk,Skv,D] (numpy bits) -> (O [B,H,S,D] bits, lse [B,H,S])."""
    B, H, S, D = q.shape
    Skv = k.shape[2]
    rep = H // k.shape[1]
    kf, vf = (np.repeat(x, rep, axis=1) if rep > 1 else x for x in (k, v))
    off = Skv - S
    assert off >= 0
    qpad = np.zeros((B, H, Skv, D), dtype=np.uint16)
    qpad[:, :, off:, :] = q
    rows = (np.arange(B * H)[:, None] * Skv + off + np.arange(S)[None, :]).reshape(-1).astype(np.int64)
    o, lse = oracle.rows(qpad, kf, vf, rows, dtype, None, causal, wl, wr, slopes, dropout=dropout)
    return o.reshape(B, H, S, D), lse.reshape(B, H, S)


RECT = [
    # B, H, Hk, S, Skv, D, dtype, causal, wl, wr
    (2, 4, 4, 1, 1000, 128, 0, True, -1, -1),        # one new token against a long cache
    (2, 8, 2, 1, 4096, 128, 0, True, -1, -1),        # ... with grouped K/V heads
    (1, 4, 4, 7, 777, 64, 0, True, -1, -1),
    (1, 4, 1, 16, 2048, 128, 1, True, -1, -1),
    (2, 2, 2, 128, 1024, 128, 0, True, -1, -1),      # chunked prefill: 128 new queries
    (1, 2, 2, 200, 1500, 64, 0, True, 300, -1),      # ... with a left window
    (1, 3, 3, 100, 612, 128, 0, False, -1, -1),      # cross attention, no mask
    (1, 2, 2, 256, 1024, 128, 1, False, 64, 64),     # two-sided window around the shifted diagonal
    (1, 2, 2, 300, 300, 128, 0, True, -1, -1),       # equal lengths through the same path
]


@pytest.mark.parametrize("B,H,Hk,S,Skv,D,dtype,causal,wl,wr", RECT)
@pytest.mark.parametrize("splits", [1, 3, "auto"])
def test_query_and_key_lengths_differ(fa, oracle, B, H, Hk, S, Skv, D, dtype, causal, wl, wr, splits):
    import torch
    q, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed=1000 + S)
    _, k, v = make_inputs(fa, (B, Hk, Skv, D), dtype, seed=1001 + Skv)
    o_ref, lse_ref = oracle_rect(oracle, q, k, v, dtype, causal, wl, wr)
    o, lse = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype), causal=causal,
                                        window_left=wl, window_right=wr, splits=splits)
    torch.cuda.synchronize()
    err = errors(oracle.to_f32(from_torch(o), dtype), oracle.to_f32(o_ref, dtype), lse.cpu().numpy(), lse_ref)
    print((B, H, Hk, S, Skv, D), dtype, causal, wl, wr, "splits", splits, err)
    assert_within(err, dtype, f"S={S} Skv={Skv} splits={splits}")


@pytest.mark.parametrize("splits", [2, 5, 64])
def test_splits_on_a_square_causal_problem(fa, oracle, splits):
    """Splits whose key range lies entirely behind the diagonal of a row are empty for that row (logsumexp -inf,
    weight 0 in the merge); the first rows of every head still come out in the reference's arithmetic."""
    import torch
    shape, dtype = (1, 3, 1024, 128), 0
    q, k, v = make_inputs(fa, shape, dtype, seed=77)
    o_ref, lse_ref = oracle.full(q, k, v, dtype, None, True, -1, -1)
    tq, tk, tv = (to_torch(x, dtype) for x in (q, k, v))
    o, lse = fa.flash_attention_forward(tq, tk, tv, causal=True, splits=splits)
    torch.cuda.synchronize()
    err = errors(oracle.to_f32(from_torch(o), dtype), oracle.to_f32(o_ref, dtype), lse.cpu().numpy(), lse_ref)
    print("square causal, splits", splits, err)
    assert_within(err, dtype, f"square causal splits={splits}")
    # rows 0..31 are computed by the same code as without splits and pass through the merge unchanged
    o1, _ = fa.flash_attention_forward(tq, tk, tv, causal=True)
    torch.cuda.synchronize()
    assert torch.equal(o[:, :, :32].view(torch.int16), o1[:, :, :32].view(torch.int16))


def test_everything_with_splits(fa, oracle):
    """Short queries against long keys with grouped heads, [B,S,H,D] storage, ALiBi, a left window and dropout,
    split four ways."""
    import torch
    B, H, Hk, S, Skv, D, dtype = 2, 8, 2, 40, 1111, 128, 0
    q, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed=31)
    _, k, v = make_inputs(fa, (B, Hk, Skv, D), dtype, seed=32)
    slopes = np.power(2.0, -8.0 / H * (np.arange(H) + 1)).astype(np.float32)
    p, seed = 0.2, 99
    thr = fa.lib().fa_dropout_threshold(p)
    o_ref, lse_ref = oracle_rect(oracle, q, k, v, dtype, True, 500, -1, slopes, dropout=(thr, seed))
    tq, tk, tv = (to_torch(x, dtype).transpose(1, 2).contiguous().transpose(1, 2) for x in (q, k, v))
    o, lse = fa.flash_attention_forward(tq, tk, tv, causal=True, window_left=500, splits=4, dropout_prob=p, seed=seed,
                                        alibi_slopes=torch.from_numpy(slopes).cuda())
    torch.cuda.synchronize()
    err = errors(oracle.to_f32(from_torch(o.contiguous()), dtype), oracle.to_f32(o_ref, dtype), lse.cpu().numpy(), lse_ref)
    print("everything with splits", err)
    grow = 256.0 / (256 - thr)
    assert err["nonfinite"] == 0 and err["max_abs"] <= 2e-3 * grow and err["rel_l2"] <= 1e-3 * grow and err["lse_abs"] <= 2e-3, err


def test_rows_without_any_key(fa):
    """More queries than keys under a causal mask: the first S - S_kv queries sit before key 0 and see nothing;
    they come out as O = 0 and logsumexp = -inf instead of NaN."""
    import torch
    B, H, S, Skv, D = 1, 2, 192, 64, 64
    q = torch.randn((B, H, S, D), dtype=torch.float16, device="cuda")
    k = torch.randn((B, H, Skv, D), dtype=torch.float16, device="cuda")
    v = torch.randn((B, H, Skv, D), dtype=torch.float16, device="cuda")
    o, lse = fa.flash_attention_forward(q, k, v, causal=True)
    torch.cuda.synchronize()
    blind = S - Skv
    assert bool((o[:, :, :blind] == 0).all()) and bool(torch.isinf(lse[:, :, :blind]).all()) and bool((lse[:, :, :blind] < 0).all())
    ref = torch.nn.functional.scaled_dot_product_attention(q[:, :, blind:].float(), k.float(), v.float(), is_causal=True)
    assert float((o[:, :, blind:].float() - ref).abs().max()) <= 2e-3


def test_workspace_is_required_and_checked(fa):
    import ctypes
    import torch
    q = torch.zeros((1, 2, 1, 64), dtype=torch.float16, device="cuda")
    k = torch.zeros((1, 2, 1024, 64), dtype=torch.float16, device="cuda")
    o = torch.zeros_like(q)
    p = fa.make_params(1, 2, 1, 64, q.data_ptr(), k.data_ptr(), k.data_ptr(), o.data_ptr(), S_kv=1024, split_num=4, causal=True)
    L = fa.lib()
    need = L.fa_fwd_workspace_bytes(ctypes.byref(p))
    assert need == 4 * 1 * 2 * 1 * 65 * 4
    assert L.fa_fwd(ctypes.byref(p), None) == fa.FA_ERR_WORKSPACE
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    p.workspace, p.workspace_bytes = ws.data_ptr(), need - 1
    assert L.fa_fwd(ctypes.byref(p), None) == fa.FA_ERR_WORKSPACE
    p.workspace_bytes = need
    assert L.fa_fwd(ctypes.byref(p), None) == fa.FA_OK
    torch.cuda.synchronize()
    assert L.fa_fwd_suggest_splits(ctypes.byref(p)) >= 2
