"""Pins the fp64 gradient oracle (oracle/fa_oracle.c, fa_oracle_bwd_f64) against finite differences of the
oracle's own fp64 forward pass and against torch autograd in fp64.  The reference has no backward pass."""
import numpy as np
import pytest

import oracle_binding as ob

F16, BF16 = ob.F16, ob.BF16


def rand_bits(rng, shape, dtype, sigma=1.0):
    return ob.from_f32((rng.standard_normal(shape) * sigma).astype(np.float32), dtype)


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("causal,wl,wr,alibi", [(False, -1, -1, False), (True, -1, -1, False), (True, 20, -1, False),
                                                (False, 9, 13, False), (True, -1, -1, True)])
def test_against_torch_autograd_f64(dtype, causal, wl, wr, alibi):
    import torch
    rng = np.random.default_rng(31)
    shape = (2, 3, 96, 32)
    B, H, S, D = shape
    q, k, v, do = (rand_bits(rng, shape, dtype) for _ in range(4))
    slopes = np.array([0.25, -0.03125, 0.0], dtype=np.float32) if alibi else None
    dq, dk, dv = ob.bwd_f64(q, k, v, do, dtype, None, causal, wl, wr, slopes)
    tq, tk, tv, tdo = (torch.from_numpy(ob.to_f32(x, dtype).astype(np.float64)) for x in (q, k, v, do))
    tq.requires_grad_(True); tk.requires_grad_(True); tv.requires_grad_(True)
    i, j = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
    vis = np.ones((S, S), dtype=bool)
    if causal:
        vis &= j <= i
    if wl >= 0:
        vis &= i - j <= wl
    if wr >= 0:
        vis &= j - i <= wr
    bias = np.zeros((1, H, S, S))
    if alibi:
        bias = -slopes.astype(np.float64)[None, :, None, None] * np.abs(i - j)[None, None]
    bias = np.where(vis[None, None], bias, -np.inf)
    s = torch.einsum("bhid,bhjd->bhij", tq, tk) * float(np.float32(1 / np.sqrt(D))) + torch.from_numpy(bias)
    o = torch.einsum("bhij,bhjd->bhid", torch.softmax(s, dim=-1), tv)
    (o * tdo).sum().backward()
    assert np.allclose(dq, tq.grad.numpy(), atol=1e-11)
    assert np.allclose(dk, tk.grad.numpy(), atol=1e-11)
    assert np.allclose(dv, tv.grad.numpy(), atol=1e-11)


def test_against_finite_differences_of_the_forward_oracle():
    """d/dx of sum(dO * O(x)) by central differences on the fp64 forward oracle, for a few elements of Q, K, V.
    The forward oracle takes storage-type inputs, so the perturbation is one that fp16 represents exactly."""
    rng = np.random.default_rng(32)
    shape = (1, 2, 40, 16)
    B, H, S, D = shape
    q, k, v, do = (rand_bits(rng, shape, F16, 0.5) for _ in range(4))
    dq, dk, dv = ob.bwd_f64(q, k, v, do, F16, None, True, 12, -1)
    dof = ob.to_f32(do, F16).astype(np.float64)
    idx = np.arange(B * H * S)

    def loss(qq, kk, vv):
        o, _ = ob.rows_f64(qq, kk, vv, idx, F16, None, True, 12, -1)
        return float((o.reshape(shape) * dof).sum())
    eps = 2.0 ** -6
    for which, grad in ((0, dq), (1, dk), (2, dv)):
        for pos in ((0, 1, 5, 3), (0, 0, 39, 15), (0, 1, 20, 0)):
            arrs = [q, k, v]
            base = ob.to_f32(arrs[which], F16)
            x0 = np.float32(np.round(base[pos] * 64) / 64)        # a multiple of 2^-6: x0 +- eps are exact in fp16
            hi, lo, mid = base.copy(), base.copy(), base.copy()
            hi[pos], lo[pos], mid[pos] = x0 + eps, x0 - eps, x0
            plus, minus = list(arrs), list(arrs)
            plus[which], minus[which] = ob.from_f32(hi, F16), ob.from_f32(lo, F16)
            fd = (loss(*plus) - loss(*minus)) / (2 * eps)
            at_mid = list(arrs)
            at_mid[which] = ob.from_f32(mid, F16)
            g = ob.bwd_f64(*at_mid, do, F16, None, True, 12, -1)[which][pos]
            assert abs(fd - g) <= 2e-3 * max(1.0, abs(g)), (which, pos, fd, g)


def test_structure_of_the_gradients():
    """dV_j = sum_i P_ij dO_i: with Q = 0 and no mask P is uniform, so every dV row is the mean of dO;
    dQ and dK vanish when V rows are all equal (O does not depend on the softmax then)."""
    rng = np.random.default_rng(33)
    shape = (1, 1, 48, 16)
    q0 = np.zeros(shape, dtype=np.uint16)
    k, v, do = (rand_bits(rng, shape, F16) for _ in range(3))
    _, _, dv = ob.bwd_f64(q0, k, v, do, F16)
    assert np.allclose(dv[0, 0], np.broadcast_to(ob.to_f32(do, F16)[0, 0].astype(np.float64).mean(axis=0), (48, 16)), atol=1e-12)
    q = rand_bits(rng, shape, F16)
    vconst = np.broadcast_to(v[:, :, :1, :], shape).copy()
    dq, dk, _ = ob.bwd_f64(q, k, vconst, do, F16, None, True)
    assert np.max(np.abs(dq)) <= 1e-12 and np.max(np.abs(dk)) <= 1e-12


@pytest.mark.parametrize("dtype,causal,p", [(F16, False, 0.25), (F16, True, 0.5), (BF16, True, 0.1)])
def test_dropout_gradients_against_torch_autograd_f64(dtype, causal, p):
    """With dropout the output is sum_j m_ij p_ij v_j, m_ij = keep_ij / (1 - p).  The keep decisions come from
    the numpy implementation of their published definition (parity_util.numpy_keep_mask), not from oracle code;
    torch differentiates softmax -> mask -> matmul in fp64."""
    import torch
    from parity_util import numpy_keep_mask
    rng = np.random.default_rng(33)
    shape = (1, 3, 80, 32)
    B, H, S, D = shape
    thr, seed = int(round(p * 256)), 0x1234ABCD5678
    q, k, v, do = (rand_bits(rng, shape, dtype) for _ in range(4))
    dq, dk, dv = ob.bwd_f64(q, k, v, do, dtype, None, causal, -1, -1, None, dropout=(thr, seed))
    tq, tk, tv, tdo = (torch.from_numpy(ob.to_f32(x, dtype).astype(np.float64)) for x in (q, k, v, do))
    tq.requires_grad_(True); tk.requires_grad_(True); tv.requires_grad_(True)
    i, j = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
    bias = np.where((j <= i) if causal else np.ones((S, S), dtype=bool), 0.0, -np.inf)
    keep = np.stack([numpy_keep_mask(seed, bh, S, thr) for bh in range(B * H)]).reshape(B, H, S, S)
    m = torch.from_numpy(keep.astype(np.float64) * (256.0 / (256.0 - thr)))
    s = torch.einsum("bhid,bhjd->bhij", tq, tk) * float(np.float32(1 / np.sqrt(D))) + torch.from_numpy(bias)
    o = torch.einsum("bhij,bhjd->bhid", torch.softmax(s, dim=-1) * m, tv)
    (o * tdo).sum().backward()
    assert 0.02 < 1.0 - keep.mean() < 0.98
    assert np.allclose(dq, tq.grad.numpy(), atol=1e-11)
    assert np.allclose(dk, tk.grad.numpy(), atol=1e-11)
    assert np.allclose(dv, tv.grad.numpy(), atol=1e-11)
