"""GPU parity beyond the reference's only layout (contiguous [B,H,S,D], S % 128 == 0, reference
src/main.cu:182, src/flash_forward.h:134): any sequence length, strided tensors ([B,S,H,D], padded rows),
query heads sharing K/V heads.  The oracle always works on contiguous [B,H,S,D] copies of the same values."""
import numpy as np
import pytest

from parity_util import assert_within, errors, from_torch, make_inputs, sample_rows, to_torch

pytestmark = pytest.mark.gpu


def run_and_check(fa, oracle, q, k, v, dtype, tq, tk, tv, causal, wl, wr, slopes=None, what="", out=None):
    """q,k,v: contiguous numpy bits [B,H,S,D] / [B,Hk,S,D]; tq,tk,tv: torch views of the same values."""
    import torch
    B, H, S, D = q.shape
    rep = H // k.shape[1]
    kf, vf = (np.repeat(x, rep, axis=1) if rep > 1 else x for x in (k, v))
    o_ref, lse_ref = oracle.full(q, kf, vf, dtype, None, causal, wl, wr, slopes)
    ts = None if slopes is None else torch.from_numpy(slopes).cuda()
    o, lse = fa.flash_attention_forward(tq, tk, tv, causal=causal, window_left=wl, window_right=wr, alibi_slopes=ts, out=out)
    torch.cuda.synchronize()
    assert o.shape == (B, H, S, D) and lse.shape == (B, H, S)
    err = errors(oracle.to_f32(from_torch(o.contiguous()), dtype), oracle.to_f32(o_ref, dtype), lse.cpu().numpy(), lse_ref)
    print(what, q.shape, k.shape, dtype, causal, wl, wr, err)
    assert_within(err, dtype, what)
    return o, lse


RAGGED = [
    # S, D, dtype, causal, wl, wr
    (1, 64, 0, False, -1, -1), (1, 128, 0, True, -1, -1), (17, 64, 0, True, -1, -1), (63, 128, 0, False, -1, -1),
    (64, 64, 0, False, -1, -1), (65, 128, 1, True, -1, -1), (100, 64, 0, False, -1, -1), (127, 128, 0, True, -1, -1),
    (129, 64, 1, False, -1, -1), (192, 128, 0, True, -1, -1), (200, 128, 0, False, 50, 20), (333, 64, 0, True, 100, -1),
    (777, 128, 0, False, -1, -1), (1000, 128, 1, True, -1, -1), (1000, 64, 0, False, 128, 128), (2049, 128, 0, True, -1, -1),
    (1300, 128, 0, False, -1, 0),
]


@pytest.mark.parametrize("S,D,dtype,causal,wl,wr", RAGGED)
def test_any_sequence_length(fa, oracle, S, D, dtype, causal, wl, wr):
    """Rows past the end are never stored, keys past the end never seen: the output tensor is allocated with a
    NaN guard band behind it that must stay NaN."""
    import torch
    shape = (2, 3, S, D)
    q, k, v = make_inputs(fa, shape, dtype, seed=500 + S)
    tq, tk, tv = (to_torch(x, dtype) for x in (q, k, v))
    guard = torch.full((2 * 3 * S * D + 4096,), float("nan"), dtype=tq.dtype, device="cuda")
    out = guard[:2 * 3 * S * D].view(shape)
    run_and_check(fa, oracle, q, k, v, dtype, tq, tk, tv, causal, wl, wr, what=f"S={S}", out=out)
    assert bool(torch.isnan(guard[2 * 3 * S * D:]).all())


@pytest.mark.parametrize("S,D,dtype,causal", [(512, 128, 0, True), (640, 64, 1, False), (300, 128, 0, True), (1024, 64, 0, True)])
def test_bshd_layout(fa, oracle, S, D, dtype, causal):
    """Tensors stored [B,S,H,D] (the head stride is D, the row stride H*D), passed as transposed views;
    the output is written with the same strides."""
    shape = (2, 4, S, D)
    q, k, v = make_inputs(fa, shape, dtype, seed=600 + S)
    tq, tk, tv = (to_torch(np.ascontiguousarray(x.transpose(0, 2, 1, 3)), dtype).transpose(1, 2) for x in (q, k, v))
    assert not tq.is_contiguous() and tq.stride() == (S * 4 * D, D, 4 * D, 1)
    o, _ = run_and_check(fa, oracle, q, k, v, dtype, tq, tk, tv, causal, -1, -1, what="BSHD")
    assert o.stride() == tq.stride()


@pytest.mark.parametrize("H,Hk,S,D,dtype,causal,wl", [(8, 2, 512, 128, 0, True, -1), (8, 1, 384, 64, 0, False, -1),
                                                     (6, 3, 640, 128, 1, True, 100), (4, 4, 200, 64, 0, True, -1)])
def test_grouped_query_heads(fa, oracle, H, Hk, S, D, dtype, causal, wl):
    import torch
    q, _, _ = make_inputs(fa, (2, H, S, D), dtype, seed=700 + H)
    _, k, v = make_inputs(fa, (2, Hk, S, D), dtype, seed=701 + H)
    tq, tk, tv = (to_torch(x, dtype) for x in (q, k, v))
    o, lse = run_and_check(fa, oracle, q, k, v, dtype, tq, tk, tv, causal, wl, -1, what=f"GQA {H}/{Hk}")
    # the same values with K/V expanded to one head per query head: bit-identical result
    rep = H // Hk
    o2, lse2 = fa.flash_attention_forward(tq, tk.repeat_interleave(rep, dim=1), tv.repeat_interleave(rep, dim=1),
                                          causal=causal, window_left=wl)
    torch.cuda.synchronize()
    assert torch.equal(o.view(torch.int16), o2.view(torch.int16)) and torch.equal(lse, lse2)
    # ... and through broadcast views (head stride 0 inside a group is not expressible; batch stride 0 is)
    if Hk == 1:
        o3, _ = fa.flash_attention_forward(tq, tk[:1].expand(2, 1, S, D), tv[:1].expand(2, 1, S, D), causal=causal, window_left=wl)
        o4, _ = fa.flash_attention_forward(tq, tk[:1].repeat(2, 1, 1, 1), tv[:1].repeat(2, 1, 1, 1), causal=causal, window_left=wl)
        torch.cuda.synchronize()
        assert torch.equal(o3.view(torch.int16), o4.view(torch.int16))


@pytest.mark.parametrize("H,Hk,S,D,dtype,bshd,wl", [(8, 2, 512, 128, 0, False, -1), (16, 8, 768, 64, 1, True, 200),
                                                       (4, 1, 256, 128, 0, True, -1), (12, 4, 1280, 128, 0, False, 300)])
def test_grouped_heads_with_alibi_in_the_regular_shape(fa, oracle, H, Hk, S, D, dtype, bshd, wl):
    """Grouped K/V heads at a length that is a multiple of 128 with S_kv = S take the kernels of the regular
    problem (strided flavour: the K/V head of a work item comes from its list position).  Slopes differ per query
    head, so a wrong head index shows; the run with K/V expanded to one head per query head must give the same
    bits, and so must every schedule."""
    import torch
    B = 2
    q, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed=900 + H)
    _, k, v = make_inputs(fa, (B, Hk, S, D), dtype, seed=901 + H)
    slopes = (np.power(2.0, -8.0 / H * (np.arange(H) + 1)) * np.where(np.arange(H) % 3 == 0, -1.0, 1.0)).astype(np.float32)
    if bshd:
        tq, tk, tv = (to_torch(np.ascontiguousarray(x.transpose(0, 2, 1, 3)), dtype).transpose(1, 2) for x in (q, k, v))
    else:
        tq, tk, tv = (to_torch(x, dtype) for x in (q, k, v))
    o, lse = run_and_check(fa, oracle, q, k, v, dtype, tq, tk, tv, True, wl, -1, slopes, what=f"GQA {H}/{Hk} ALiBi")
    rep = H // Hk
    ts = torch.from_numpy(slopes).cuda()
    o2, lse2 = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype).repeat_interleave(rep, dim=1),
                                          to_torch(v, dtype).repeat_interleave(rep, dim=1), causal=True, window_left=wl, alibi_slopes=ts)
    torch.cuda.synchronize()
    assert torch.equal(o.contiguous().view(torch.int16), o2.view(torch.int16)) and torch.equal(lse, lse2)
    for sched in (1, 2, 3):
        o3, lse3 = fa.flash_attention_forward(tq, tk, tv, causal=True, window_left=wl, alibi_slopes=ts, sched=sched)
        torch.cuda.synchronize()
        assert torch.equal(o.view(torch.int16), o3.view(torch.int16)) and torch.equal(lse, lse3), sched


def test_padded_rows_and_everything_at_once(fa, oracle):
    """Row stride larger than the head dimension (a slice of a wider tensor), [B,S,H,D] storage, grouped K/V
    heads, a ragged length, causal + left window and ALiBi in one launch."""
    import torch
    B, H, Hk, S, D, dtype = 2, 8, 2, 457, 128, 0
    q, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed=801)
    _, k, v = make_inputs(fa, (B, Hk, S, D), dtype, seed=802)
    slopes = np.power(2.0, -8.0 / H * (np.arange(H) + 1)).astype(np.float32)

    def widen(bits, heads):       # [B,S,heads,D+64] storage, the tensor is the [..., :D] slice seen as [B,heads,S,D]
        wide = torch.full((B, S, heads, D + 64), float("nan"), dtype=torch.float16, device="cuda")
        wide[..., :D] = to_torch(bits, dtype).transpose(1, 2)
        return wide[..., :D].transpose(1, 2)
    tq, tk, tv = widen(q, H), widen(k, Hk), widen(v, Hk)
    assert tq.stride() == (S * H * (D + 64), D + 64, H * (D + 64), 1)
    run_and_check(fa, oracle, q, k, v, dtype, tq, tk, tv, True, 200, -1, slopes, what="padded BSHD GQA ragged ALiBi")


def test_headline_shape_in_bshd_layout(fa, oracle):
    """The headline problem (fp16 B2 H32 S8192 D128 causal) stored [B,S,H,D]: sampled rows against the oracle."""
    import torch
    shape = (2, 32, 8192, 128)
    B, H, S, D = shape
    q, k, v = make_inputs(fa, shape, 0, seed=29)
    tq, tk, tv = (to_torch(x, 0).transpose(1, 2).contiguous().transpose(1, 2) for x in (q, k, v))
    o, lse = fa.flash_attention_forward(tq, tk, tv, causal=True)
    torch.cuda.synchronize()
    rows = sample_rows(shape, 2048, 29)
    o_ref, lse_ref = oracle.rows(q, k, v, rows, 0, None, True, -1, -1)
    err = errors(oracle.to_f32(from_torch(o.contiguous()), 0).reshape(-1, D)[rows], oracle.to_f32(o_ref, 0),
                 lse.cpu().numpy().reshape(-1)[rows], lse_ref)
    print("c3 BSHD", err)
    assert_within(err, 0, "c3 in BSHD layout")
    # The contiguous layout runs with three LDS stages, this one with two: the same products and exponentials,
    # but the row sums are added up in another order in the iterations that fill and drain the pipeline, so the
    # results agree to the last bits rather than bit for bit.
    o2, lse2 = fa.flash_attention_forward(to_torch(q, 0), to_torch(k, 0), to_torch(v, 0), causal=True)
    torch.cuda.synchronize()
    assert float((o.contiguous().float() - o2.float()).abs().max()) <= 2.0 ** -9          # one fp16 ulp at |O| < 4
    assert float((lse - lse2).abs().max()) <= 1e-5


@pytest.mark.parametrize("shape,Hk,S_real", [((2, 16, 1024, 128), 4, 1024), ((4, 32, 512, 64), 32, 500), ((1, 64, 2048, 128), 8, 2048)])
def test_general_layouts_under_every_schedule(fa, oracle, shape, Hk, S_real):
    """[B,S,H,D] storage with grouped K/V heads (and a ragged length) through the three ways of walking the work
    list, with both workgroup shapes occurring among the cases: sampled rows against the oracle, and the same
    bits from every schedule."""
    import torch
    B, H, _, D = shape
    S = S_real
    q, _, _ = make_inputs(fa, (B, H, S, D), 0, seed=61)
    _, k, v = make_inputs(fa, (B, Hk, S, D), 0, seed=62)
    tq, tk, tv = (to_torch(x, 0).transpose(1, 2).contiguous().transpose(1, 2) for x in (q, k, v))
    rows = sample_rows((B, H, S, D), 512, 61)
    rep = H // Hk
    o_ref, lse_ref = oracle.rows(q, np.repeat(k, rep, axis=1), np.repeat(v, rep, axis=1), rows, 0, None, True, -1, -1)
    outs = []
    for sched in (fa.FA_SCHED_DISPATCH, fa.FA_SCHED_PERSISTENT, fa.FA_SCHED_QUEUE):
        o, lse = fa.flash_attention_forward(tq, tk, tv, causal=True, sched=sched)
        torch.cuda.synchronize()
        err = errors(oracle.to_f32(from_torch(o.contiguous()), 0).reshape(-1, D)[rows], oracle.to_f32(o_ref, 0),
                     lse.cpu().numpy().reshape(-1)[rows], lse_ref)
        print(shape, Hk, S, "sched", sched, err)
        assert_within(err, 0, f"general layout, schedule {sched}")
        outs.append((o, lse))
    for o, lse in outs[1:]:
        assert torch.equal(o.view(torch.int16), outs[0][0].view(torch.int16)) and torch.equal(lse, outs[0][1])


@pytest.mark.parametrize("shape,dtype,causal,wl,sched", [((2, 8, 1024, 128), 0, True, -1, 0), ((8, 40, 384, 64), 1, True, 100, 2),
                                                         ((4, 16, 2176, 128), 0, False, -1, 3), ((1, 4, 256, 64), 0, False, -1, 1)])
def test_regular_problem_in_strided_layouts_matches_the_contiguous_run_bit_for_bit(fa, shape, dtype, causal, wl, sched):
    """Lengths a multiple of 128, one K/V head per query head: a strided layout ([B,S,H,D] views, rows padded to a
    larger stride, an output with its own layout) runs the contiguous kernels' instruction stream with strides from
    the arguments, so the bits must be those of the contiguous run (several passes over the resident grid included:
    what a workgroup requests ahead for its next item is addressed through the same strides)."""
    import torch
    B, H, S, D = shape
    q, k, v = make_inputs(fa, shape, dtype, seed=91)
    tq, tk, tv = (to_torch(x, dtype) for x in (q, k, v))
    o_ref, lse_ref = fa.flash_attention_forward(tq, tk, tv, causal=causal, window_left=wl, sched=sched)
    # [B,S,H,D] storage
    sq, sk, sv = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (tq, tk, tv))
    out = torch.full((B, S, H, D), float("nan"), dtype=tq.dtype, device="cuda").transpose(1, 2)
    o1, lse1 = fa.flash_attention_forward(sq, sk, sv, causal=causal, window_left=wl, sched=sched, out=out)
    # rows padded to D + 64 elements, K and V sharing one buffer
    pad = torch.zeros((B, H, S, 2 * D + 64), dtype=tq.dtype, device="cuda")
    pad[..., :D] = tk
    pad[..., D + 64:] = tv
    o2, lse2 = fa.flash_attention_forward(tq, pad[..., :D], pad[..., D + 64:], causal=causal, window_left=wl, sched=sched)
    torch.cuda.synchronize()
    for o, lse in ((o1, lse1), (o2, lse2)):
        assert torch.equal(o.contiguous().view(torch.int16), o_ref.view(torch.int16)) and torch.equal(lse, lse_ref)
