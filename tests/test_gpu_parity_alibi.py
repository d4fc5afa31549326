"""GPU parity of the ALiBi bias (reference src/mask.h:21-26, verifier src/main.cu:200-207): the HIP forward
pass through the C ABI against the CPU oracle on the same seeded inputs, and against closed forms."""
import numpy as np
import pytest

from parity_util import assert_within, errors, from_torch, make_inputs, sample_rows, to_torch

pytestmark = pytest.mark.gpu


def reference_slopes(H):
    """The slopes the reference's main() builds (src/main.cu:38-42): negative, -2^(-8/H * (h+1))."""
    return (-np.power(2.0, -8.0 / H * (np.arange(H) + 1))).astype(np.float32)


def press_slopes(H):
    """The usual ALiBi slopes, 2^(-8/H * (h+1)): the bias pushes distant keys down."""
    return (-reference_slopes(H)).astype(np.float32)


SMALL = [
    # shape (B,H,S,D), dtype, causal, wl, wr, slopes
    ((1, 4, 256, 64), 0, False, -1, -1, "press"),
    ((1, 4, 256, 64), 0, True, -1, -1, "press"),
    ((2, 2, 512, 128), 0, True, -1, -1, "press"),
    ((1, 8, 384, 128), 0, False, -1, -1, "press"),
    ((1, 8, 640, 64), 1, True, -1, -1, "press"),
    ((1, 2, 1024, 128), 1, True, 200, -1, "press"),
    ((1, 2, 1024, 128), 0, False, 128, 128, "press"),
    ((1, 8, 512, 64), 0, True, -1, -1, "reference"),       # the reference's own (negative) slopes
    ((1, 8, 512, 128), 0, False, 128, 128, "reference"),
    ((1, 8, 512, 128), 1, True, 128, -1, "reference"),
    ((1, 3, 512, 128), 0, True, -1, -1, "mixed"),           # a zero slope and both signs in one launch
]


def slopes_for(kind, H):
    if kind == "press":
        return press_slopes(H)
    if kind == "reference":
        return reference_slopes(H)
    return np.array([0.0, 0.03125, -0.0078125], dtype=np.float32)[:H]


@pytest.mark.parametrize("shape,dtype,causal,wl,wr,kind", SMALL)
def test_small_full_tensor_alibi(fa, oracle, shape, dtype, causal, wl, wr, kind):
    import torch
    slopes = slopes_for(kind, shape[1])
    q, k, v = make_inputs(fa, shape, dtype, seed=4321 + shape[2] + dtype)
    o_ref, lse_ref = oracle.full(q, k, v, dtype, None, causal, wl, wr, slopes)
    o, lse = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype), causal=causal,
                                        window_left=wl, window_right=wr, alibi_slopes=torch.from_numpy(slopes).cuda())
    err = errors(oracle.to_f32(from_torch(o), dtype), oracle.to_f32(o_ref, dtype), lse.cpu().numpy(), lse_ref)
    print(shape, dtype, causal, wl, wr, kind, err)
    assert_within(err, dtype, f"alibi {kind} {shape} dtype={dtype} causal={causal} w=({wl},{wr})")


@pytest.mark.parametrize("sched", [1, 3])
@pytest.mark.parametrize("name,shape,dtype,causal,wl,seed", [
    ("c3", (2, 32, 8192, 128), 0, True, -1, 29),
    ("c4", (1, 32, 16384, 128), 1, True, 1024, 30),
    ("c2nc", (4, 16, 2048, 64), 0, False, -1, 28),
])
def test_benchmark_shapes_alibi(fa, oracle, name, shape, dtype, causal, wl, seed, sched):
    """The benchmark shapes with the usual per-head slopes, over a seeded row subset that holds the edge rows."""
    import torch
    B, H, S, D = shape
    slopes = press_slopes(H)
    q, k, v = make_inputs(fa, shape, dtype, seed)
    o, lse = fa.flash_attention_forward(to_torch(q, dtype), to_torch(k, dtype), to_torch(v, dtype), causal=causal,
                                        window_left=wl, sched=sched, alibi_slopes=torch.from_numpy(slopes).cuda())
    torch.cuda.synchronize()
    rows = sample_rows(shape, 2048, seed, (wl, wl + 1) if wl >= 0 else ())
    o_ref, lse_ref = oracle.rows(q, k, v, rows, dtype, None, causal, wl, -1, slopes)
    err = errors(oracle.to_f32(from_torch(o), dtype).reshape(-1, D)[rows], oracle.to_f32(o_ref, dtype),
                 lse.cpu().numpy().reshape(-1)[rows], lse_ref)
    print(name, "alibi sched", sched, "rows", len(rows), err)
    assert bool(torch.isfinite(o.float()).all()) and bool(torch.isfinite(lse).all())
    assert_within(err, dtype, f"alibi {name} sched={sched}")


def test_alibi_closed_form_on_gpu(fa):
    """Q = 0 leaves only the bias.  With V[j, t] = [j mod D == t] the output is O[i, t] = sum over visible keys
    j = t (mod D) of exp(-slope_h |i-j|) / Z_i, which numpy evaluates in fp64 without any oracle code; the
    logsumexp is log Z_i.  Size independent: run at S = 4096, all rows checked."""
    import torch
    B, H, S, D = 1, 4, 4096, 64
    slopes = np.array([0.25, 0.015625, -0.001953125, 0.0], dtype=np.float32)
    q = torch.zeros((B, H, S, D), dtype=torch.float16, device="cuda")
    k = torch.randn((B, H, S, D), dtype=torch.float16, device="cuda")
    v = torch.zeros((S, D), dtype=torch.float16)
    v[torch.arange(S), torch.arange(S) % D] = 1.0
    v = v.cuda().expand(B, H, S, D).contiguous()
    i, j = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
    onehot = np.zeros((S, D))
    onehot[np.arange(S), np.arange(S) % D] = 1.0
    for causal in (False, True):
        o, lse = fa.flash_attention_forward(q, k, v, causal=causal, alibi_slopes=torch.from_numpy(slopes).cuda())
        torch.cuda.synchronize()
        o, lse = o.float().cpu().numpy(), lse.cpu().numpy()
        for h in range(H):
            s = -np.float64(slopes[h]) * np.abs(i - j)
            if causal:
                s = np.where(j <= i, s, -np.inf)
            mx = s.max(axis=1, keepdims=True)
            w = np.exp(s - mx)
            Z = w.sum(axis=1, keepdims=True)
            want = (w / Z) @ onehot
            assert np.max(np.abs(o[0, h] - want)) <= 1e-3, (causal, h)          # fp16 p and fp16 output rounding
            assert np.max(np.abs(lse[0, h] - (mx[:, 0] + np.log(Z[:, 0])))) <= 1e-3, (causal, h)


def test_alibi_zero_slopes_equal_no_alibi(fa):
    """All-zero slopes go through the biased kernel and must reproduce the unbiased result (the exponent is
    computed as s*c - m*c in one rounding there and in two here, hence a tolerance of one output ulp)."""
    import torch
    shape = (2, 4, 1024, 128)
    q, k, v = make_inputs(fa, shape, 0, seed=91)
    tq, tk, tv = (to_torch(x, 0) for x in (q, k, v))
    o0, l0 = fa.flash_attention_forward(tq, tk, tv, causal=True)
    o1, l1 = fa.flash_attention_forward(tq, tk, tv, causal=True, alibi_slopes=torch.zeros(4, device="cuda"))
    torch.cuda.synchronize()
    assert float((o0.float() - o1.float()).abs().max()) <= 1e-3
    assert float((l0 - l1).abs().max()) <= 1e-5


def test_reference_entry_point_alibi(fa, oracle):
    """run_flash_attention with Has_alibi = 1 and the slopes the reference's main() builds (main.cu:36-45)."""
    import torch
    shape = (2, 8, 2048, 64)
    B, H, S, D = shape
    slopes = reference_slopes(H)
    q, k, v = make_inputs(fa, shape, 0, seed=26)
    tq, tk, tv = (to_torch(x, 0) for x in (q, k, v))
    ts = torch.from_numpy(slopes).cuda()
    for causal, local, w in ((1, 0, 0), (0, 1, 128)):
        o = torch.full_like(tq, float("nan"))
        lse = torch.empty((B, H, S), dtype=torch.float32, device="cuda")
        st = fa.run_flash_attention(B, H, S, D, tq, tk, tv, o, lse, None, False, bool(causal), bool(local), True, w, ts)
        assert st == fa.FA_OK
        rows = sample_rows(shape, 2048, 126 + causal)
        o_ref, lse_ref = oracle.rows(q, k, v, rows, 0, None, bool(causal), w if local else -1, w if local else -1, slopes)
        err = errors(oracle.to_f32(from_torch(o), 0).reshape(-1, D)[rows], oracle.to_f32(o_ref, 0),
                     lse.cpu().numpy().reshape(-1)[rows], lse_ref)
        print("run_flash_attention alibi", causal, local, w, err)
        assert_within(err, 0, f"run_flash_attention alibi causal={causal} local={local}")
    # Has_alibi without slopes is an error, not a silent unbiased run
    assert fa.run_flash_attention(B, H, S, D, tq, tk, tv, o, lse, None, False, True, False, True, 0, None) == fa.FA_ERR_NULL_POINTER
