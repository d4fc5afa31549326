"""Twice forty seeded random configurations (lengths, heads, head groups, head dim, dtype, masks, ALiBi, dropout, storage
order, padded rows) through fa_fwd and fa_bwd, compared with an explicit fp32 attention and its autograd gradients in torch on the
GPU.  The oracle-based tests pin the arithmetic on chosen cases; this sweep is there for the index arithmetic of
combinations nobody chose."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def reference(q, k, v, do, causal, wl, wr, slopes, keep=None):
    import torch
    B, H, S, D = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    qf, kf, vf = (t.detach().float().requires_grad_(True) for t in (q, k, v))
    kr, vr = (t.repeat_interleave(H // Hk, dim=1) for t in (kf, vf))
    pos = torch.arange(S, device=q.device)[:, None] + (Sk - S)
    j = torch.arange(Sk, device=q.device)[None, :]
    vis = torch.ones((S, Sk), dtype=torch.bool, device=q.device)
    if causal:
        vis &= j <= pos
    if wl >= 0:
        vis &= pos - j <= wl
    if wr >= 0 and not causal:
        vis &= j - pos <= wr
    s = torch.einsum("bhid,bhjd->bhij", qf, kr) * float(np.float32(1.0 / np.sqrt(D)))
    if slopes is not None:
        s = s - slopes[None, :, None, None] * (pos - j).abs()[None, None].float()
    s = s.masked_fill(~vis, float("-inf"))
    p = torch.nan_to_num(torch.softmax(s, dim=-1), nan=0.0)
    if keep is not None:            # [B,H,S,Sk] factors: 0 or 1/(1-p)
        p = p * keep
    o = torch.einsum("bhij,bhjd->bhid", p, vr)
    (o * do.float()).sum().backward()
    lse = torch.logsumexp(s, dim=-1)
    return o.detach(), lse.detach(), qf.grad, kf.grad, vf.grad, vis


@pytest.mark.parametrize("regular", [False, True], ids=["any_shape", "regular_lengths"])
def test_random_configurations(fa, regular):
    """regular: lengths that are multiples of 128 with as many keys, no ALiBi, no dropout -- the problems that the
    strided kernels take when the storage is not the reference's or K/V heads are grouped; padded rows now and then."""
    import torch
    rng = np.random.default_rng(20240607 + int(regular))
    for case in range(40):
        D = int(rng.choice([64, 128]))
        dtype = torch.bfloat16 if rng.random() < 0.3 else torch.float16
        Hk = int(rng.choice([1, 2, 3]))
        H = Hk * int(rng.choice([1, 1, 2, 4]))
        B = int(rng.integers(1, 3))
        S = 128 * int(rng.integers(1, 9)) if regular else int(rng.integers(1, 700))
        Sk = S if (regular or rng.random() < 0.5) else int(rng.integers(max(1, S - 100), S + 400))
        causal = bool(rng.random() < 0.6)
        wl = int(rng.integers(0, 300)) if rng.random() < 0.4 else -1
        wr = int(rng.integers(0, 300)) if (not causal and rng.random() < 0.4) else -1
        alibi = bool(rng.random() < 0.3) and not regular
        bshd = bool(rng.random() < 0.5)
        pad = 8 * int(rng.integers(1, 4)) if (regular and rng.random() < 0.3) else 0      # unused elements behind every row
        # dropout where the published decision function can be replayed by the numpy implementation as it stands
        # (query positions from 0 up: not more queries than keys)
        drop_p = float(rng.choice([0.1, 0.3, 0.5])) if (Sk >= S and rng.random() < 0.3 and not regular) else 0.0
        seed = int(rng.integers(1, 2 ** 40))
        g = torch.Generator(device="cuda").manual_seed(1000 + case)

        def make(h, s):
            t = torch.randn((B, s, h, D + pad) if bshd else (B, h, s, D + pad), device="cuda", generator=g).to(dtype)[..., :D]
            return t.transpose(1, 2) if bshd else t
        q, do, k, v = make(H, S), make(H, S), make(Hk, Sk), make(Hk, Sk)
        slopes = (torch.rand(H, device="cuda", generator=g) * 0.2 - 0.05).float().contiguous() if alibi else None
        what = dict(case=case, B=B, H=H, Hk=Hk, S=S, Sk=Sk, D=D, dtype=str(dtype), causal=causal, wl=wl, wr=wr, alibi=alibi, bshd=bshd,
                    pad=pad, dropout=drop_p)
        print(what, flush=True)
        kw = dict(causal=causal, window_left=wl, window_right=wr, alibi_slopes=slopes, dropout_prob=drop_p, seed=seed)
        keep, grow = None, 1.0
        if drop_p > 0:
            from parity_util import numpy_keep_mask
            thr = fa.lib().fa_dropout_threshold(drop_p)
            grow = 256.0 / (256 - thr)
            m = np.stack([numpy_keep_mask(seed, bh, Sk, thr)[Sk - S:] for bh in range(B * H)]).reshape(B, H, S, Sk)
            keep = torch.from_numpy(m.astype(np.float32) * grow).cuda()
        # exact products in every row (what the autograd wrapper uses): the comparison is with exact fp32
        # attention, not with the reference verifier's rounded products
        o, lse = fa.flash_attention_forward(q, k, v, exact_first_rows=True, **kw)
        dq, dk, dv = fa.flash_attention_backward(q, k, v, o, lse, do, **kw)
        torch.cuda.synchronize()
        o_ref, lse_ref, dq_ref, dk_ref, dv_ref, vis = reference(q, k, v, do, causal, wl, wr, slopes, keep)
        half = dtype == torch.float16
        assert bool(torch.isfinite(o.float()).all()), what
        # the tolerance, or one and a half ulps of the storage type where a row of few keys makes the output so
        # large that they exceed it: p and the result are each rounded once to the storage type, which puts the
        # result up to one step beside the rounded reference, itself up to half a step from the exact one
        # (an indexing mistake shows up as an error of order one)
        one_ulp = torch.exp2(torch.floor(torch.log2(o_ref.abs().clamp_min(1e-4))) - (10 if half else 7))
        bound = torch.maximum(1.5 * one_ulp, torch.full_like(one_ulp, 2e-3 if half else 1.6e-2)) * grow
        assert bool(((o.float() - o_ref).abs() <= bound).all()), (what, float((o.float() - o_ref).abs().max()))
        seen = torch.isfinite(lse_ref)
        assert bool((lse[~seen] == float("-inf")).all()), what
        if bool(seen.any()):
            assert float((lse[seen] - lse_ref[seen]).abs().max()) <= (2e-3 if half else 8e-3), what
        o_rounding = 0.0
        if drop_p > 0:
            delta_sd = float(((do.float() * o_ref) ** 2).sum(-1).max().sqrt()) * (2.0 ** -11 if half else 2.0 ** -8) / 3 ** 0.5
            o_rounding = 4 * delta_sd * grow * float(max(q.float().abs().max(), k.float().abs().max())) / D ** 0.5
        # Rows that see fewer than eight keys have large P, outputs of magnitude 3 and a delta = dO.O taken from the
        # stored, rounded O; they, and the keys such rows touch, get relaxed bounds.  Everything else -- in a problem
        # of some length nearly all of it -- is held to the forward's bars, so that an indexing mistake of the
        # backward kernels cannot hide under the relaxed ones.
        few = vis.sum(1) < 8                                   # [S] queries
        touched = (vis & few[:, None]).any(0)                  # [Sk] keys that such a query sees
        for name, got, want, loose in (("dQ", dq, dq_ref, few), ("dK", dk, dk_ref, touched), ("dV", dv, dv_ref, touched)):
            d = got.float() - want
            scale = max(1.0, float(want.abs().max()))
            assert bool(torch.isfinite(got.float()).all()), (name, what)
            tight = ~loose
            if bool(tight.any()):
                dt, wt = d[:, :, tight], want[:, :, tight]
                assert float(dt.abs().max()) <= (2e-3 if half else 1.6e-2) * scale * grow + o_rounding, \
                    (name, "max, rows of eight keys and more", float(dt.abs().max()), what)
                if int(tight.sum()) >= 16:
                    floor_t = (1e-5 + o_rounding) * wt.numel() ** 0.5
                    assert float(dt.norm()) <= (1e-3 if half else 8e-3) * grow * float(wt.norm()) + floor_t, \
                        (name, "norm, rows of eight keys and more", float(dt.norm()), float(wt.norm()), what)
            # (bf16: twice the forward's tolerance, here and for the norm below.  A row that sees two or three keys has
            # large P and an output of magnitude 3; delta = dO.O is taken from the stored, rounded O, and one such row
            # in twenty thousand configurations reached 2.2e-2 of the largest gradient; a problem of two queries,
            # which has no other rows, 1.1e-2 of the norm -- 1.3e-3 in fp16, where large problems stay near 3e-4)
            # (with dropout, plus what the rounding of the stored output does to delta = dO.O: a query with a single
            # key has gradient zero, its output row V / (1 - p) is rounded on the way to memory, and dQ and dK of that
            # row come out as that rounding error of delta times K and Q: four standard deviations of it are allowed)
            assert float(d.abs().max()) <= (2e-3 if half else 3.2e-2) * scale * grow + o_rounding, \
                (name, "max", float(d.abs().max()), what)
            # (plus a floor per element: where a query sees one key dS = P (dP - delta) is zero in exact arithmetic.
            # The kernels' dP and delta are then the same sum taken in two orders, and dQ and dK come out as a few
            # 1e-6; with dropout the one output row is V / (1 - p) rounded to the storage type, delta is taken
            # from that rounded row, and they come out as the rounding error of dO.O times K, as above)
            # (problems of fewer than sixteen queries are left to the element-wise bound: all their rows see a few
            # keys, P near one half rounded to the storage type moves such a row by 1e-3 of its size and more)
            floor = (1e-5 + o_rounding) * want.numel() ** 0.5
            assert S < 16 or float(d.norm()) <= (2e-3 if half else 1.6e-2) * grow * float(want.norm()) + floor, (name, "norm", float(d.norm()), what)
