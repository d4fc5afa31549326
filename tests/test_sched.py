"""Host mirror of the tile scheduler (csrc/fa_sched.h through the C ABI): key-tile ranges against the
reference's Schedule<0>::next formulas (flash_forward.h:52-61), tile classification against the per-element
mask predicate by brute force, longest-first order, pair counts."""
import ctypes
import itertools

import numpy as np
import pytest


def visible(i, j, causal, wl, wr):
    if causal and j > i:
        return False
    if wl >= 0 and i - j > wl:
        return False
    if wr >= 0 and j - i > wr:
        return False
    return True


MASKS = [(0, -1, -1), (1, -1, -1), (0, 128, 128), (1, 128, -1), (1, 1024, -1), (0, 100, 37), (0, -1, 0), (1, 0, -1), (0, 300, -1)]


def tile_range(L, S, bk, causal, wl, wr, q0, rows):
    lo, hi = ctypes.c_int(), ctypes.c_int()
    L.fa_sched_tile_range(S, bk, causal, wl, wr, q0, rows, ctypes.byref(lo), ctypes.byref(hi))
    return lo.value, hi.value


@pytest.mark.parametrize("causal,wl,wr", MASKS)
def test_classification_matches_element_predicate(fa, causal, wl, wr):
    L = fa.lib()
    for S, rows, bk in itertools.product((128, 384, 1024), (32, 64, 128, 256), (32, 64, 128)):
        i = np.arange(S)[:, None]
        j = np.arange(S)[None, :]
        vis = np.ones((S, S), dtype=bool)
        if causal:
            vis &= j <= i
        if wl >= 0:
            vis &= i - j <= wl
        if wr >= 0:
            vis &= j - i <= wr
        for q0 in range(0, S, rows):
            r = min(rows, S - q0)
            lo, hi = tile_range(L, S, bk, causal, wl, wr, q0, r)
            for t in range(S // bk):
                block = vis[q0:q0 + r, t * bk:(t + 1) * bk]
                want = fa.FA_TILE_FULL if block.all() else (fa.FA_TILE_PARTIAL if block.any() else fa.FA_TILE_SKIP)
                assert L.fa_sched_classify(bk, causal, wl, wr, q0, r, t) == want
                if block.any():
                    assert lo <= t <= hi          # every tile with a visible pair is visited
            # the visited range is tight at both ends
            assert vis[q0:q0 + r, lo * bk:(lo + 1) * bk].any() and vis[q0:q0 + r, hi * bk:(hi + 1) * bk].any()


def test_tile_range_equals_reference_formulas(fa):
    """Br = Bc = 128, the reference's tile shape: n_block_min/max of flash_forward.h:52-61."""
    L = fa.lib()
    Br = Bc = 128
    for S in (128, 1024, 4096):
        for causal, local, w in ((0, 0, 0), (1, 0, 0), (0, 1, 128), (1, 1, 128), (0, 1, 300), (1, 1, 1024)):
            for bx in range(S // Br):
                n_min = max(0, (bx * Br - w) // Bc) if local else 0
                n_max = (S + Bc - 1) // Bc
                if local:
                    n_max = min(n_max, ((bx + 1) * Br + w + Bc - 1) // Bc)
                if causal:
                    n_max = min(n_max, ((bx + 1) * Br + Bc - 1) // Bc)
                wl = w if local else -1
                wr = w if local else -1
                assert tile_range(L, S, Bc, causal, wl, wr, bx * Br, Br) == (n_min, n_max - 1)


@pytest.mark.parametrize("shape", [(1, 4, 256, 64), (4, 16, 2048, 64), (2, 32, 8192, 128), (1, 3, 384, 128)])
@pytest.mark.parametrize("causal,wl,wr", [(0, -1, -1), (1, -1, -1), (1, 1024, -1)])
def test_every_item_once_and_longest_first(fa, shape, causal, wl, wr):
    L = fa.lib()
    B, N, S, d = shape
    n = L.fa_sched_num_items(B, N, S, d, causal, wl, wr)
    br, bk = L.fa_sched_block_rows(B, N, S, d, causal, wl, wr), L.fa_sched_block_keys(d)
    assert br in (128, 256)
    assert n == B * N * ((S + br - 1) // br)
    seen = set()
    costs = []
    bh, q0 = ctypes.c_int(), ctypes.c_int()
    for item in range(n):
        assert L.fa_sched_item(B, N, S, d, causal, wl, wr, item, ctypes.byref(bh), ctypes.byref(q0)) == 0
        assert 0 <= bh.value < B * N and q0.value % br == 0 and 0 <= q0.value < S
        seen.add((bh.value, q0.value))
        lo, hi = tile_range(L, S, bk, causal, wl, wr, q0.value, min(br, S - q0.value))
        costs.append(hi - lo + 1)
        if B * N % 8 == 0:
            assert bh.value % 8 == item % 8      # a head stays on one XCD under round-robin dispatch
    assert len(seen) == n
    # heads come in groups of eight (one per XCD); inside a group the cost never increases along the list
    # (longest first), except that a trailing partial query block may be cheaper than what follows it
    per_group = 8 * ((S + br - 1) // br)
    if S % br == 0:
        for g0 in range(0, n, per_group):
            grp = costs[g0:g0 + per_group]
            assert all(a >= b for a, b in zip(grp, grp[1:]))
    assert L.fa_sched_item(B, N, S, d, causal, wl, wr, n, ctypes.byref(bh), ctypes.byref(q0)) != 0


def test_pair_counts_and_flops(fa):
    L = fa.lib()
    for S, causal, wl, wr in ((256, 0, -1, -1), (2048, 1, -1, -1), (8192, 1, -1, -1), (16384, 1, 1024, -1), (512, 0, 100, 37)):
        want = sum(min(S - 1, i + (0 if causal else (wr if wr >= 0 else S))) - max(0, i - (wl if wl >= 0 else S)) + 1 for i in range(S))
        assert L.fa_count_pairs(S, causal, wl, wr) == want
    # the five benchmark configurations
    assert L.fa_algorithmic_flops(1, 4, 256, 64, 0, -1, -1) == 4.0 * 4 * 64 * 65536
    assert L.fa_count_pairs(2048, 1, -1, -1) == 2098176
    assert L.fa_count_pairs(8192, 1, -1, -1) == 33558528
    assert L.fa_count_pairs(16384, 1, 1024, -1) == 16268800
    assert L.fa_count_pairs(32768, 1, -1, -1) == 536887296
    assert abs(L.fa_algorithmic_flops(2, 32, 8192, 128, 1, -1, -1) - 1.0996e12) < 1e8


@pytest.mark.parametrize("N,Nk", [(8, 8), (8, 2), (8, 1), (32, 8), (12, 4), (6, 3), (5, 0)])
def test_grouped_heads_list_walks_the_kv_heads_fastest(fa, N, Nk):
    """Every (batch entry, query head) once; query head h reads K/V head h / (N / Nk) (include/fa_fwd.h,
    n_kv_heads); consecutive list positions inside a group of Nk belong to consecutive K/V heads."""
    L = fa.lib()
    hk = Nk if Nk > 0 else N
    group = N // hk
    seen = set()
    b, q, k = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    for bh in range(3 * N):
        assert L.fa_sched_heads(N, Nk, bh, ctypes.byref(b), ctypes.byref(q), ctypes.byref(k)) == 0
        assert b.value == bh // N and 0 <= q.value < N and k.value == q.value // group
        assert k.value == (bh % N) % hk
        seen.add((b.value, q.value))
    assert len(seen) == 3 * N
    assert L.fa_sched_heads(8, 3, 0, ctypes.byref(b), ctypes.byref(q), ctypes.byref(k)) != 0      # 3 does not divide 8
    assert L.fa_sched_heads(8, 2, -1, ctypes.byref(b), ctypes.byref(q), ctypes.byref(k)) != 0
