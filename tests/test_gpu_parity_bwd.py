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
    assert err["rel_l2"] <= rel or err["max_abs"] <= 1e-5, (what, err)      # (a gradient that is exactly 0 has no relative error)
    assert err["max_abs"] <= mx * max(1.0, err["max_ref"]), (what, err)


@pytest.mark.parametrize("shape,dtype,causal,wl,wr", CASES)
def test_gradients_against_the_fp64_oracle(fa, oracle, shape, dtype, causal, wl, wr):
    import torch
    q, k, v = make_inputs(fa, shape, dtype, seed=500 + shape[2])
    do, _, _ = make_inputs(fa, shape, dtype, seed=501 + shape[2])
    dq_ref, dk_ref, dv_ref = oracle.bwd_f64(q, k, v, do, dtype, None, causal, wl, wr)
    tq, tk, tv, tdo = (to_torch(x, dtype) for x in (q, k, v, do))
    o, lse = fa.flash_attention_forward(tq, tk, tv, causal=causal, window_left=wl, window_right=wr, exact_first_rows=True)
    # (the seven-product form: fa_bwd_dq and fa_bwd_dkdv; the five-product form has its own test below)
    dq, dk, dv = fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, causal=causal, window_left=wl, window_right=wr, five_products=False)
    torch.cuda.synchronize()
    for name, got, want in (("dQ", dq, dq_ref), ("dK", dk, dk_ref), ("dV", dv, dv_ref)):
        err = grad_errors(oracle.to_f32(from_torch(got), dtype), want)
        print(shape, dtype, causal, wl, wr, name, err, flush=True)
        check(err, dtype, name)


FIVE_CASES = [
    # shape, dtype, causal, wl, wr: the reference's layout (S a multiple of 128), every kind of band
    ((1, 2, 128, 64), 0, False, -1, -1),
    ((2, 2, 256, 128), 0, True, -1, -1),
    ((1, 2, 384, 64), 1, True, -1, -1),
    ((1, 2, 640, 128), 0, True, 100, -1),
    ((1, 2, 512, 64), 0, False, 70, 50),
    ((1, 2, 512, 128), 0, False, -1, 32),      # a right window that ends on a 32-key block edge
    ((1, 2, 512, 128), 1, False, -1, 33),
    ((1, 1, 384, 64), 0, False, 31, 0),
    ((1, 1, 384, 128), 0, False, 0, 0),        # the diagonal alone
    ((1, 2, 768, 128), 1, False, 128, 0),
    ((1, 2, 1024, 128), 0, False, 5, 200),
]


@pytest.mark.parametrize("shape,dtype,causal,wl,wr", FIVE_CASES)
def test_five_product_form_against_the_fp64_oracle(fa, oracle, shape, dtype, causal, wl, wr):
    """fa_bwd with the large workspace (fa_bwd_fast_workspace_bytes): the key-owning kernel writes its dS blocks and
    dQ is one product over them.  Through the C ABI, with the workspace filled with NaN beforehand: a block read
    without having been written (the two kernels must agree on which blocks exist under every mask) poisons dQ."""
    import ctypes
    import torch
    B, H, S, D = shape
    q, k, v = make_inputs(fa, shape, dtype, seed=700 + S)
    do, _, _ = make_inputs(fa, shape, dtype, seed=701 + S)
    dq_ref, dk_ref, dv_ref = oracle.bwd_f64(q, k, v, do, dtype, None, causal, wl, wr)
    tq, tk, tv, tdo = (to_torch(x, dtype) for x in (q, k, v, do))
    o, lse = fa.flash_attention_forward(tq, tk, tv, causal=causal, window_left=wl, window_right=wr, exact_first_rows=True)
    dq, dk, dv = (torch.full_like(tq, float("nan")) for _ in range(3))
    p = fa.make_bwd_params(B, H, S, D, tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), o.data_ptr(), tdo.data_ptr(), lse.data_ptr(),
                           dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), causal=causal, window_left=wl, window_right=wr, dtype=dtype)
    L = fa.lib()
    small, need = L.fa_bwd_workspace_bytes(ctypes.byref(p)), L.fa_bwd_fast_workspace_bytes(ctypes.byref(p))
    assert need >= small + B * H * S * S * 2
    ws = torch.full((need // 4 + 1,), float("nan"), dtype=torch.float32, device="cuda")
    p.workspace, p.workspace_bytes = ws.data_ptr(), need
    assert L.fa_bwd(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == fa.FA_OK
    torch.cuda.synchronize()
    for name, got, want in (("dQ", dq, dq_ref), ("dK", dk, dk_ref), ("dV", dv, dv_ref)):
        err = grad_errors(oracle.to_f32(from_torch(got), dtype), want)
        print("five products", shape, dtype, causal, wl, wr, name, err, flush=True)
        check(err, dtype, name)
    # the same bits on a second run
    dq2, dk2, dv2 = (torch.full_like(tq, float("nan")) for _ in range(3))
    p.dQ, p.dK, p.dV = dq2.data_ptr(), dk2.data_ptr(), dv2.data_ptr()
    ws.fill_(float("nan"))
    assert L.fa_bwd(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == fa.FA_OK
    torch.cuda.synchronize()
    for a_, b_ in ((dq, dq2), (dk, dk2), (dv, dv2)):
        assert torch.equal(a_.view(torch.int16), b_.view(torch.int16))


def test_five_product_workspace_is_offered_for_regular_lengths_only(fa):
    """As many keys as queries, in any storage order and with any grouping of K/V heads (the dS blocks are per QUERY
    head); lengths a multiple of 128 also with dropout or with ALiBi (not both at once), other lengths without."""
    import ctypes
    L = fa.lib()
    ok = dict(B=2, N=4, S=1024, d=128)
    small = L.fa_bwd_workspace_bytes(ctypes.byref(fa.make_bwd_params(**ok)))
    large = ((small + 255) // 256) * 256 + 2 * 4 * 1024 * 1024 * 2
    assert L.fa_bwd_fast_workspace_bytes(ctypes.byref(fa.make_bwd_params(**ok))) == large
    for same in (dict(n_kv_heads=2), dict(n_kv_heads=1), dict(strides={"q": (4 * 1024 * 128, 128, 4 * 128)}), dict(dropout_prob=0.1),
                 dict(alibi_ptr=256)):
        assert L.fa_bwd_fast_workspace_bytes(ctypes.byref(fa.make_bwd_params(**{**ok, **same}))) == large, same
    ragged = dict(B=2, N=4, S=1000, d=128)
    small_r = L.fa_bwd_workspace_bytes(ctypes.byref(fa.make_bwd_params(**ragged)))
    # (32 blocks of 32 queries or keys per side, in four squares of eight: as many as S = 1024 has)
    assert L.fa_bwd_fast_workspace_bytes(ctypes.byref(fa.make_bwd_params(**ragged))) == ((small_r + 255) // 256) * 256 + 2 * 4 * 1024 * 1024 * 2
    for other in (dict(S=1000, dropout_prob=0.1), dict(S=1000, alibi_ptr=256), dict(S_kv=2048), dict(alibi_ptr=256, dropout_prob=0.1)):
        assert L.fa_bwd_fast_workspace_bytes(ctypes.byref(fa.make_bwd_params(**{**ok, **other}))) == 0, other


@pytest.mark.parametrize("B,H,Hk,S,D,dtype,causal,bshd", [(2, 16, 16, 8192, 64, 0, True, False), (6, 16, 8, 4096, 128, 1, True, True),
                                                          (3, 24, 24, 2048, 128, 0, False, False)])
def test_five_product_form_in_chunks_of_heads(fa, B, H, Hk, S, D, dtype, causal, bshd):
    """A workspace that holds the dS blocks of some of the heads only: the key-owning and the query-owning kernel run
    once per chunk of heads.  Same bits as with the full workspace (every head's arithmetic is the same), with the
    smallest workspace the form accepts and with one in between whose last chunk is a partial one; one byte less than
    the smallest selects the seven-product form."""
    import ctypes
    import torch
    g = torch.Generator(device="cuda").manual_seed(77)
    dt = torch.bfloat16 if dtype else torch.float16
    q, do = (torch.randn((B, H, S, D), device="cuda", generator=g).to(dt) for _ in range(2))
    k, v = (torch.randn((B, Hk, S, D), device="cuda", generator=g).to(dt) for _ in range(2))
    if bshd:
        q, k, v, do = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (q, k, v, do))
    o, lse = fa.flash_attention_forward(q, k, v, causal=causal, exact_first_rows=True)
    full = fa.flash_attention_backward(q, k, v, o, lse, do, causal=causal, five_products=True, poison_workspace=True)
    strides = {n: tuple(t.stride()[:3]) for n, t in (("q", q), ("k", k), ("v", v), ("o", o), ("do", do), ("dq", q), ("dk", k), ("dv", v))}
    p = fa.make_bwd_params(B, H, S, D, causal=causal, dtype=dtype, n_kv_heads=Hk, strides=strides)
    L = fa.lib()
    small, least, most = (int(f(ctypes.byref(p))) for f in (L.fa_bwd_workspace_bytes, L.fa_bwd_min_fast_workspace_bytes, L.fa_bwd_fast_workspace_bytes))
    assert small < least < most
    for limit in (least, (least + most) // 2):
        assert limit < most
        got = fa.flash_attention_backward(q, k, v, o, lse, do, causal=causal, five_products="auto", poison_workspace=True, workspace_limit=limit)
        torch.cuda.synchronize()
        for name, x, y in zip(("dQ", "dK", "dV"), full, got):
            assert torch.equal(x.contiguous().view(torch.int16), y.contiguous().view(torch.int16)), (name, limit)
    seven = fa.flash_attention_backward(q, k, v, o, lse, do, causal=causal, five_products=False)
    below = fa.flash_attention_backward(q, k, v, o, lse, do, causal=causal, five_products="auto", workspace_limit=least - 1)
    torch.cuda.synchronize()
    for name, x, y in zip(("dQ", "dK", "dV"), seven, below):
        assert torch.equal(x.contiguous().view(torch.int16), y.contiguous().view(torch.int16)), name


FIVE_STRIDED = [
    # B, H, Hk, S, D, dtype, causal, wl, wr, bshd: regular lengths through the strided kernels
    (2, 4, 2, 512, 128, 0, True, -1, -1, True),
    (1, 4, 4, 384, 64, 1, True, 100, -1, True),
    (1, 6, 2, 256, 64, 0, False, -1, -1, False),
    (1, 2, 1, 640, 128, 1, False, 64, 64, True),
    (1, 8, 2, 768, 128, 0, True, -1, -1, True),
    (2, 3, 1, 384, 128, 0, False, 0, 40, False),
]


@pytest.mark.parametrize("B,H,Hk,S,D,dtype,causal,wl,wr,bshd", FIVE_STRIDED)
def test_five_product_form_in_strided_layouts_and_with_grouped_heads(fa, oracle, B, H, Hk, S, D, dtype, causal, wl, wr, bshd):
    """[B,S,H,D] storage and K/V heads shared by groups of query heads: the key-owning workgroup writes the dS blocks
    of every query head of its group."""
    five_product_case(fa, oracle, B, H, Hk, S, D, dtype, causal, wl, wr, bshd, False)


FIVE_RAGGED = [
    # B, H, Hk, S, D, dtype, causal, wl, wr, bshd: any length with as many keys, through the general kernels
    (1, 2, 2, 100, 64, 0, True, -1, -1, False),
    (2, 4, 2, 333, 128, 0, True, -1, -1, False),
    (1, 2, 1, 300, 128, 1, False, -1, -1, True),
    (1, 2, 2, 1000, 128, 0, True, -1, -1, False),       # the last 32-key block of the last tile holds 8 keys
    (1, 3, 3, 970, 64, 0, True, 200, -1, True),         # ... holds none: its wave of the key-owning kernel has no key
    (1, 2, 2, 1, 128, 0, True, -1, -1, False),
    (2, 2, 1, 33, 64, 1, False, 5, 7, False),
    (1, 4, 2, 577, 128, 0, False, 100, 60, True),
]


@pytest.mark.parametrize("B,H,Hk,S,D,dtype,causal,wl,wr,bshd", FIVE_RAGGED)
def test_five_product_form_at_any_length(fa, oracle, B, H, Hk, S, D, dtype, causal, wl, wr, bshd):
    """Lengths that are not a multiple of 128 (as many keys as queries): the general kernels write and read the dS
    blocks too.  Lanes of the key-owning kernel whose key lies past the end store zeros, 32-key blocks without any
    key are neither written nor read, query rows past the end are masked to zero: with a NaN-filled workspace."""
    five_product_case(fa, oracle, B, H, Hk, S, D, dtype, causal, wl, wr, bshd, False)


ALIBI_REGULAR = [
    # B, H, Hk, S, D, dtype, causal, wl, wr, bshd: regular lengths with ALiBi slopes of both signs
    (1, 4, 4, 384, 128, 0, True, -1, -1, False),
    (2, 4, 2, 512, 128, 1, True, 200, -1, True),
    (1, 2, 2, 256, 64, 0, False, -1, -1, False),
    (1, 6, 2, 640, 64, 0, False, 50, 30, True),
    (1, 2, 1, 768, 128, 0, False, -1, -1, True),
]


@pytest.mark.parametrize("B,H,Hk,S,D,dtype,causal,wl,wr,bshd", ALIBI_REGULAR)
def test_alibi_on_regular_lengths_in_both_forms(fa, oracle, B, H, Hk, S, D, dtype, causal, wl, wr, bshd):
    """ALiBi on regular lengths runs kernels of its own (not the general ones), in both storage orders, with the
    five-product form: the bias enters the score the key-owning kernel recomputes, dS carries it from there."""
    five_product_case(fa, oracle, B, H, Hk, S, D, dtype, causal, wl, wr, bshd, True)


def five_product_case(fa, oracle, B, H, Hk, S, D, dtype, causal, wl, wr, bshd, alibi):
    """The five-product form against the fp64 oracle, with a NaN-filled workspace, twice with the same bits; the
    seven-product form of the same call meets the same bars."""
    import torch
    q, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed=720 + S)
    do, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed=721 + S)
    _, k, v = make_inputs(fa, (B, Hk, S, D), dtype, seed=722 + S)
    slopes = (np.power(2.0, -8.0 / H * (np.arange(H) + 1)) * np.where(np.arange(H) % 2, -0.5, 1.0)).astype(np.float32) if alibi else None
    dq_ref, dk_ref, dv_ref = oracle_bwd_general(oracle, q, k, v, do, dtype, causal, wl, wr, slopes)
    tq, tk, tv, tdo = (to_torch(x, dtype) for x in (q, k, v, do))
    if bshd:
        tq, tk, tv, tdo = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (tq, tk, tv, tdo))
    kw = dict(causal=causal, window_left=wl, window_right=wr, alibi_slopes=None if slopes is None else torch.from_numpy(slopes).cuda())
    o, lse = fa.flash_attention_forward(tq, tk, tv, exact_first_rows=True, **kw)
    five = fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, five_products=True, poison_workspace=True, **kw)
    seven = fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, five_products=False, **kw)
    again = fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, five_products=True, poison_workspace=True, **kw)
    torch.cuda.synchronize()
    for name, got, want, other, rerun, like in zip(("dQ", "dK", "dV"), five, (dq_ref, dk_ref, dv_ref), seven, again, (tq, tk, tv)):
        assert got.stride() == like.stride()
        err = grad_errors(oracle.to_f32(from_torch(got.contiguous()), dtype), want)
        print("five products, strided", (B, H, Hk, S, D), dtype, causal, wl, wr, bshd, name, err, flush=True)
        check(err, dtype, name)
        assert torch.equal(got.contiguous().view(torch.int16), rerun.contiguous().view(torch.int16)), name
        # (the seven-product form sums delta and dQ in other orders: close, not equal)
        close = grad_errors(oracle.to_f32(from_torch(other.contiguous()), dtype), want)
        check(close, dtype, name + " (seven products)")


@pytest.mark.parametrize("dtype", [0, 1])
def test_default_forward_feeding_the_backward_pass(fa, oracle, dtype):
    """fa_bwd.h asks for a forward pass with exact_first_rows = 1.  A C caller that forgets (the default forward
    writes the first 32 rows of a causal head in the CPU verifier's rounded-product arithmetic, and fa_bwd
    recomputes P from exact scores) must still get gradients inside the ordinary bars: stated bound, rows 0-31 of
    dQ and all of dK, dV within rel-L2 1e-3 / 8e-3 and max-abs 2e-3 / 1.6e-2 of the largest gradient; dQ rows
    from 32 on do not change by a bit (a row of dQ depends on its own O row and logsumexp only)."""
    import torch
    shape = (1, 2, 256, 128)
    q, k, v = make_inputs(fa, shape, dtype, seed=901)
    do, _, _ = make_inputs(fa, shape, dtype, seed=902)
    dq_ref, dk_ref, dv_ref = oracle.bwd_f64(q, k, v, do, dtype, None, True, -1, -1)
    tq, tk, tv, tdo = (to_torch(x, dtype) for x in (q, k, v, do))
    grads = {}
    for exact in (False, True):
        o, lse = fa.flash_attention_forward(tq, tk, tv, causal=True, exact_first_rows=exact)
        grads[exact] = fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, causal=True)
    torch.cuda.synchronize()
    for name, got, want in zip(("dQ", "dK", "dV"), grads[False], (dq_ref, dk_ref, dv_ref)):
        err = grad_errors(oracle.to_f32(from_torch(got), dtype), want)
        print("default forward", dtype, name, err, flush=True)
        check(err, dtype, name)
    first = grad_errors(oracle.to_f32(from_torch(grads[False][0][:, :, :32].contiguous()), dtype), dq_ref[:, :, :32])
    print("default forward", dtype, "dQ rows 0-31", first, flush=True)
    check(first, dtype, "dQ rows 0-31")
    assert torch.equal(grads[False][0][:, :, 32:], grads[True][0][:, :, 32:])


def test_against_torch_autograd_on_the_gpu(fa):
    """A larger problem than the CPU oracle finishes quickly: torch's fp32 attention and autograd on the GPU."""
    import torch
    B, H, S, D = 2, 4, 2048, 128
    g = torch.Generator(device="cuda").manual_seed(5)
    q, k, v, do = (torch.randn((B, H, S, D), device="cuda", generator=g).half() for _ in range(4))
    o, lse = fa.flash_attention_forward(q, k, v, causal=True, exact_first_rows=True)
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

    def params(S=128, d=64, ws_bytes=1024, **kw):
        ptr = t.data_ptr()
        return fa.make_bwd_params(1, 1, S, d, ptr, ptr, ptr, ptr, ptr, lse.data_ptr(), ptr, ptr, ptr,
                                  workspace_ptr=ws.data_ptr(), workspace_bytes=ws_bytes, **kw)
    assert L.fa_bwd_validate(ctypes.byref(params())) == fa.FA_OK
    assert L.fa_bwd(ctypes.byref(params(d=96)), None) == fa.FA_ERR_HEAD_DIM
    assert L.fa_bwd(ctypes.byref(params(ws_bytes=1023)), None) == fa.FA_ERR_WORKSPACE
    assert L.fa_bwd(ctypes.byref(params(n_kv_heads=2)), None) == fa.FA_ERR_LAYOUT
    assert L.fa_bwd(ctypes.byref(params(strides=dict(dq=(0, 0, 60)))), None) == fa.FA_ERR_LAYOUT
    p = params(); p.dK = 0
    assert L.fa_bwd(ctypes.byref(p), None) == fa.FA_ERR_NULL_POINTER

def oracle_bwd_general(oracle, q, k, v, do, dtype, causal, wl, wr, slopes, dropout=(0, 0)):
    """q, do [B,H,S,D], k, v [B,Hk,Skv,D] (storage bits) -> fp64 dq [B,H,S,D], dk, dv [B,Hk,Skv,D].
    The oracle differentiates square problems with one K/V head per query head.  Grouped heads: repeat K and V
    and sum their gradients over the group.  S < Skv: the queries are the last S rows of the square Skv problem
    whose first rows carry dO = 0 (such a row contributes nothing to dK or dV and rows do not interact)."""
    B, H, S, D = q.shape
    Hk, Skv = k.shape[1], k.shape[2]
    rep, off = H // Hk, Skv - S
    assert off >= 0
    kf, vf = (np.repeat(x, rep, axis=1) if rep > 1 else x for x in (k, v))
    qpad = np.zeros((B, H, Skv, D), dtype=np.uint16)
    dopad = np.zeros((B, H, Skv, D), dtype=np.uint16)
    qpad[:, :, off:], dopad[:, :, off:] = q, do
    dq, dk, dv = oracle.bwd_f64(qpad, kf, vf, dopad, dtype, None, causal, wl, wr, slopes, dropout=dropout)
    return dq[:, :, off:], dk.reshape(B, Hk, rep, Skv, D).sum(axis=2), dv.reshape(B, Hk, rep, Skv, D).sum(axis=2)


GENERAL = [
    # B, H, Hk, S, Skv, D, dtype, causal, wl, wr, alibi, bshd
    (1, 2, 2, 100, 100, 64, 0, True, -1, -1, False, False),        # ragged length
    (2, 4, 2, 333, 333, 128, 0, True, -1, -1, False, False),       # ... with grouped K/V heads
    (1, 4, 1, 256, 256, 128, 0, False, -1, -1, False, True),       # one K/V head, [B,S,H,D] storage
    (1, 2, 2, 200, 456, 128, 0, True, -1, -1, False, False),       # more keys than queries, causal
    (1, 3, 3, 77, 300, 64, 1, False, -1, -1, False, True),         # cross attention, bf16
    (1, 4, 2, 384, 384, 128, 0, True, -1, -1, True, False),        # ALiBi with grouped heads
    (1, 2, 2, 190, 190, 64, 0, False, 50, 30, True, True),         # ALiBi, two-sided window, [B,S,H,D]
    (1, 8, 2, 512, 640, 128, 1, True, 200, -1, False, True),
    (1, 2, 2, 1, 500, 128, 0, True, -1, -1, False, False),         # a single query
    (1, 2, 1, 300, 300, 128, 0, True, -1, -1, False, False),
    (1, 2, 2, 256, 256, 64, 0, True, -1, -1, True, False),         # ALiBi on a shape the plain kernels cover
    # the reference's lengths with other strides or grouped heads: the strided kernels
    (2, 4, 2, 512, 512, 128, 0, True, -1, -1, False, True),
    (1, 4, 4, 384, 384, 64, 1, True, 100, -1, False, True),
    (1, 6, 2, 256, 256, 64, 0, False, -1, -1, False, False),
    (1, 2, 1, 640, 640, 128, 1, False, 64, 64, False, True),
]


@pytest.mark.parametrize("B,H,Hk,S,Skv,D,dtype,causal,wl,wr,alibi,bshd", GENERAL)
def test_general_layouts_against_the_fp64_oracle(fa, oracle, B, H, Hk, S, Skv, D, dtype, causal, wl, wr, alibi, bshd):
    import torch
    q, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed=700 + S)
    do, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed=701 + S)
    _, k, v = make_inputs(fa, (B, Hk, Skv, D), dtype, seed=702 + Skv)
    slopes = (np.power(2.0, -8.0 / H * (np.arange(H) + 1)) * np.where(np.arange(H) % 2, -0.5, 1.0)).astype(np.float32) if alibi else None
    dq_ref, dk_ref, dv_ref = oracle_bwd_general(oracle, q, k, v, do, dtype, causal, wl, wr, slopes)
    tq, tk, tv, tdo = (to_torch(x, dtype) for x in (q, k, v, do))
    if bshd:
        tq, tk, tv, tdo = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (tq, tk, tv, tdo))
    ts = None if slopes is None else torch.from_numpy(slopes).cuda()
    o, lse = fa.flash_attention_forward(tq, tk, tv, causal=causal, window_left=wl, window_right=wr, alibi_slopes=ts)
    dq, dk, dv = fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, causal=causal, window_left=wl, window_right=wr, alibi_slopes=ts)
    torch.cuda.synchronize()
    assert dq.stride() == tq.stride() and dk.stride() == tk.stride() and dv.stride() == tv.stride()
    for name, got, want in (("dQ", dq, dq_ref), ("dK", dk, dk_ref), ("dV", dv, dv_ref)):
        err = grad_errors(oracle.to_f32(from_torch(got.contiguous()), dtype), want)
        print((B, H, Hk, S, Skv, D), dtype, causal, wl, wr, alibi, bshd, name, err, flush=True)
        check(err, dtype, name)


@pytest.mark.parametrize("five", [False, True])
@pytest.mark.parametrize("D,dtype,causal,wl", [(128, 0, True, -1), (64, 1, False, -1), (128, 1, True, 200), (64, 0, True, -1)])
def test_storage_order_changes_no_bit_of_the_gradients(fa, D, dtype, causal, wl, five):
    """[B,S,H,D] storage goes through the strided kernels, [B,H,S,D] through the plain ones: same values, same
    arithmetic in the same order, so dQ, dK and dV have to agree bit for bit, in the seven-product form and in the
    five-product form (which sums dQ in another order than the seven-product one, but in the same order in both
    layouts)."""
    import torch
    B, H, S = 2, 3, 768
    q, k, v = make_inputs(fa, (B, H, S, D), dtype, seed=910 + D)
    do, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed=911 + D)
    dense = [to_torch(x, dtype) for x in (q, k, v, do)]
    bshd = [t.transpose(1, 2).contiguous().transpose(1, 2) for t in dense]
    got = []
    for tq, tk, tv, tdo in (dense, bshd):
        o, lse = fa.flash_attention_forward(tq, tk, tv, causal=causal, window_left=wl)
        got.append(fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, causal=causal, window_left=wl, five_products=five))
    torch.cuda.synchronize()
    assert got[1][0].stride() == bshd[0].stride()
    for name, a, b in zip(("dQ", "dK", "dV"), got[0], got[1]):
        assert torch.equal(a.view(torch.int16), b.contiguous().view(torch.int16)), name


def test_queries_without_any_key_get_zero_gradients(fa):
    """More queries than keys under a causal mask: the first S - S_kv queries see nothing (O = 0, logsumexp
    -inf in the forward pass); their dQ is 0, they add nothing to dK and dV, and nothing is NaN."""
    import torch
    B, H, S, Skv, D = 1, 2, 192, 64, 64
    g = torch.Generator(device="cuda").manual_seed(11)
    q, do = (torch.randn((B, H, S, D), device="cuda", generator=g).half() for _ in range(2))
    k, v = (torch.randn((B, H, Skv, D), device="cuda", generator=g).half() for _ in range(2))
    o, lse = fa.flash_attention_forward(q, k, v, causal=True)
    dq, dk, dv = fa.flash_attention_backward(q, k, v, o, lse, do, causal=True)
    torch.cuda.synchronize()
    blind = S - Skv
    assert bool((dq[:, :, :blind] == 0).all())
    qf, kf, vf = (t.float().requires_grad_(True) for t in (q[:, :, blind:], k, v))
    torch.nn.functional.scaled_dot_product_attention(qf, kf, vf, is_causal=True).backward(do[:, :, blind:].float())
    for name, got, want in (("dQ", dq[:, :, blind:], qf.grad), ("dK", dk, kf.grad), ("dV", dv, vf.grad)):
        err = grad_errors(got.float().cpu().numpy(), want.cpu().numpy())
        print("blind rows", name, err, flush=True)
        check(err, 0, name)


DROPOUT = [
    # B, H, Hk, S, Skv, D, dtype, causal, wl, wr, alibi, bshd, p, seed
    (1, 2, 2, 256, 256, 64, 0, False, -1, -1, False, False, 0.1, 48),
    (2, 2, 2, 384, 384, 128, 0, True, -1, -1, False, False, 0.1, 48),
    (1, 4, 2, 333, 333, 128, 0, True, -1, -1, False, True, 0.25, 0x123456789ABCDEF),     # grouped heads, ragged, [B,S,H,D]
    (1, 2, 2, 200, 456, 128, 1, True, -1, -1, False, False, 0.5, 7),                     # more keys than queries, bf16
    (1, 2, 1, 190, 190, 64, 0, False, 50, 30, True, False, 0.2, 8),                      # ALiBi, window, one K/V head
    (1, 3, 3, 640, 640, 128, 0, True, 100, -1, True, False, 0.9, 9),                     # almost everything dropped
    # regular lengths without ALiBi: kernels of their own, with a five-product form
    (2, 4, 2, 512, 512, 128, 1, True, -1, -1, False, True, 0.3, 10),                      # grouped heads, [B,S,H,D]
    (1, 2, 2, 640, 640, 64, 0, False, 64, 40, False, False, 0.1, 11),
    (1, 3, 1, 384, 384, 128, 0, True, 200, -1, False, True, 0.6, 12),
]


@pytest.mark.parametrize("five", [False, True])
@pytest.mark.parametrize("B,H,Hk,S,Skv,D,dtype,causal,wl,wr,alibi,bshd,p,seed", DROPOUT)
def test_dropout_gradients_against_the_fp64_oracle(fa, oracle, B, H, Hk, S, Skv, D, dtype, causal, wl, wr, alibi, bshd, p, seed, five):
    """The backward pass replays the forward's keep decisions from (seed, head, query position, key); the oracle
    does the same on the CPU.  Kept probabilities are multiplied by 1/(1-p), and so is every rounding error.
    Both forms: with five products (regular lengths without ALiBi; the others run seven either way) only the
    key-owning kernel replays the decisions, and the workspace is filled with NaN first."""
    import torch
    thr = fa.lib().fa_dropout_threshold(p)
    q, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed=800 + S)
    do, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed=801 + S)
    _, k, v = make_inputs(fa, (B, Hk, Skv, D), dtype, seed=802 + Skv)
    slopes = np.power(2.0, -8.0 / H * (np.arange(H) + 1)).astype(np.float32) if alibi else None
    dq_ref, dk_ref, dv_ref = oracle_bwd_general(oracle, q, k, v, do, dtype, causal, wl, wr, slopes, dropout=(thr, seed))
    tq, tk, tv, tdo = (to_torch(x, dtype) for x in (q, k, v, do))
    if bshd:
        tq, tk, tv, tdo = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (tq, tk, tv, tdo))
    ts = None if slopes is None else torch.from_numpy(slopes).cuda()
    kw = dict(causal=causal, window_left=wl, window_right=wr, alibi_slopes=ts, dropout_prob=p, seed=seed)
    o, lse = fa.flash_attention_forward(tq, tk, tv, **kw)
    dq, dk, dv = fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, five_products=five, poison_workspace=True, **kw)
    dq2, dk2, dv2 = fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, five_products=five, poison_workspace=True, **kw)
    torch.cuda.synchronize()
    grow = 256.0 / (256 - thr)
    rel, mx = (1e-3, 2e-3) if dtype == 0 else (8e-3, 1.6e-2)
    for name, got, again, want in (("dQ", dq, dq2, dq_ref), ("dK", dk, dk2, dk_ref), ("dV", dv, dv2, dv_ref)):
        err = grad_errors(oracle.to_f32(from_torch(got.contiguous()), dtype), want)
        print((B, H, Hk, S, Skv, D), dtype, causal, wl, wr, alibi, bshd, p, name, err, flush=True)
        assert err["nonfinite"] == 0 and err["rel_l2"] <= rel * grow and err["max_abs"] <= mx * grow * max(1.0, err["max_ref"]), (name, err)
        assert torch.equal(got.view(torch.int16), again.view(torch.int16))        # no atomics: the same bits every time


def torch_grads_f64(q, k, v, do, causal, wl, wr):
    """fp64 autograd on the CPU for any S and S_kv (query i at key position i + S_kv - S; a query that sees no
    key has output 0).  q, do [B,H,S,D], k, v [B,Hk,Skv,D] torch tensors."""
    import torch
    B, H, S, D = q.shape
    Hk, Skv = k.shape[1], k.shape[2]
    qf, kf, vf = (t.detach().double().cpu().requires_grad_(True) for t in (q, k, v))
    kr, vr = (t.repeat_interleave(H // Hk, dim=1) for t in (kf, vf))
    pos = torch.arange(S)[:, None] + (Skv - S)
    j = torch.arange(Skv)[None, :]
    vis = torch.ones((S, Skv), dtype=torch.bool)
    if causal:
        vis &= j <= pos
    if wl >= 0:
        vis &= pos - j <= wl
    if wr >= 0:
        vis &= j - pos <= wr
    s = torch.einsum("bhid,bhjd->bhij", qf, kr) * float(np.float32(1.0 / np.sqrt(D)))
    s = s.masked_fill(~vis, float("-inf"))
    p = torch.nan_to_num(torch.softmax(s, dim=-1), nan=0.0)       # rows without any key
    (torch.einsum("bhij,bhjd->bhid", p, vr) * do.detach().double().cpu()).sum().backward()
    return qf.grad.numpy(), kf.grad.numpy(), vf.grad.numpy()


TINY = [
    # B, H, Hk, S, Skv, D, dtype, causal, wl, wr
    (1, 1, 1, 1, 1, 64, 0, True, -1, -1),
    (1, 3, 3, 5, 5, 128, 0, True, -1, -1),
    (2, 5, 5, 31, 33, 64, 0, False, -1, -1),
    (1, 2, 2, 65, 64, 128, 0, True, -1, -1),          # one query before the first key
    (1, 4, 2, 300, 70, 64, 0, False, -1, -1),         # cross attention with more queries than keys
    (1, 2, 2, 257, 100, 128, 1, True, 40, -1),        # causal window, queries before the first key, bf16
    (1, 9, 3, 129, 513, 64, 0, False, 10, 10),        # nine heads: the last group of eight is a single head
    (3, 1, 1, 64, 64, 128, 0, True, 0, -1),           # window 0: every query sees only itself
    (16, 24, 8, 128, 128, 64, 0, True, -1, -1),       # many small heads: 384 work items of one block each
    (1, 2, 2, 2048, 2048, 128, 1, True, 256, -1),     # a sliding window much shorter than the sequence, bf16
]


@pytest.mark.parametrize("B,H,Hk,S,Skv,D,dtype,causal,wl,wr", TINY)
def test_small_and_odd_shapes_against_torch_autograd_f64(fa, B, H, Hk, S, Skv, D, dtype, causal, wl, wr):
    import torch
    g = torch.Generator(device="cuda").manual_seed(100 + S)
    dt = torch.bfloat16 if dtype else torch.float16
    q, do = (torch.randn((B, H, S, D), device="cuda", generator=g).to(dt) for _ in range(2))
    k, v = (torch.randn((B, Hk, Skv, D), device="cuda", generator=g).to(dt) for _ in range(2))
    o, lse = fa.flash_attention_forward(q, k, v, causal=causal, window_left=wl, window_right=wr)
    dq, dk, dv = fa.flash_attention_backward(q, k, v, o, lse, do, causal=causal, window_left=wl, window_right=wr)
    torch.cuda.synchronize()
    for name, got, want in zip(("dQ", "dK", "dV"), (dq, dk, dv), torch_grads_f64(q, k, v, do, causal, wl, wr)):
        err = grad_errors(got.float().cpu().numpy(), want)
        print((B, H, Hk, S, Skv, D), dtype, causal, wl, wr, name, err, flush=True)
        check(err, dtype, name)


def test_autograd_wrapper_trains_like_torch_attention(fa):
    """fa.flash_attention under torch autograd: [B,S,H,D] storage, grouped K/V heads, a loss that is not a plain
    sum, compared with torch's scaled_dot_product_attention differentiated in fp32."""
    import torch
    B, S, H, Hk, D = 2, 512, 8, 2, 128
    g = torch.Generator(device="cuda").manual_seed(21)
    base = [torch.randn((B, S, n, D), device="cuda", generator=g).half() for n in (H, Hk, Hk)]
    w = torch.randn((B, H, S, D), device="cuda", generator=g).half()
    q, k, v = (t.transpose(1, 2).detach().requires_grad_(True) for t in base)
    out = fa.flash_attention(q, k, v, causal=True)
    ((out.float() * w.float()).sum() + 0.5 * (out.float() ** 2).sum()).backward()
    qf, kf, vf = (t.transpose(1, 2).detach().float().requires_grad_(True) for t in base)
    ref = torch.nn.functional.scaled_dot_product_attention(qf, kf.repeat_interleave(H // Hk, 1), vf.repeat_interleave(H // Hk, 1), is_causal=True)
    ((ref * w.float()).sum() + 0.5 * (ref ** 2).sum()).backward()
    torch.cuda.synchronize()
    assert float((out.detach().float() - ref.detach()).abs().max()) <= 2e-3
    for name, got, want in (("dQ", q.grad, qf.grad), ("dK", k.grad, kf.grad), ("dV", v.grad, vf.grad)):
        err = grad_errors(got.float().cpu().numpy(), want.cpu().numpy())
        print("autograd wrapper", name, err, flush=True)
        # the loss gradient dO = w + out is itself rounded to fp16 on the way into fa_bwd
        assert err["nonfinite"] == 0 and err["rel_l2"] <= 2e-3 and err["max_abs"] <= 4e-3 * max(1.0, err["max_ref"]), (name, err)


def test_gradients_with_outlier_query_rows(fa, oracle):
    """c5's input recipe on a small shape: sigma 0.5 and a seeded 5 % of the query rows multiplied by 8, so that
    some rows have one dominant key (P close to one-hot, large logsumexp) next to ordinary ones."""
    import torch
    shape, dtype = (1, 4, 512, 128), 0
    q, k, v = make_inputs(fa, shape, dtype, 31, 0.5, 0.05, 8.0)
    do, _, _ = make_inputs(fa, shape, dtype, seed=32)
    dq_ref, dk_ref, dv_ref = oracle.bwd_f64(q, k, v, do, dtype, None, True, -1, -1)
    tq, tk, tv, tdo = (to_torch(x, dtype) for x in (q, k, v, do))
    o, lse = fa.flash_attention_forward(tq, tk, tv, causal=True)
    dq, dk, dv = fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, causal=True)
    torch.cuda.synchronize()
    assert float(lse.max()) > 8.0          # the outlier rows are there
    for name, got, want in (("dQ", dq, dq_ref), ("dK", dk, dk_ref), ("dV", dv, dv_ref)):
        err = grad_errors(oracle.to_f32(from_torch(got), dtype), want)
        print("outlier rows", name, err, flush=True)
        check(err, dtype, name)
