"""C-ABI boundary without a GPU: the library loads, exports every symbol include/*.h declares, and
rejects bad arguments with status codes (the reference exits/aborts/throws: utils.h:16-23,
flash_forward.h:384-387,587-589)."""
import ctypes
import os

import numpy as np
import re

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = "".join(open(os.path.join(REPO, "include", h)).read() for h in ("fa_fwd.h", "fa_bwd.h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"^\s*(?:const\s+)?(?:int|void|unsigned long long|long long|double|char)\s*\*?\s*(\w+)\s*\(", text, flags=re.M)
    return sorted(set(names))


def test_header_and_library_agree(fa):
    names = declared_functions()
    assert sorted(fa.EXPORTED_SYMBOLS) == names
    L = fa.lib()
    for n in names:
        assert getattr(L, n) is not None


def test_struct_layout_matches_header(fa):
    text = open(os.path.join(REPO, "include", "fa_fwd.h")).read()
    body = re.search(r"typedef struct fa_fwd_params \{(.*?)\} fa_fwd_params;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = [re.search(r"(\w+)\s*(\[\d+\])?\s*;", line).group(1) for line in body.splitlines() if ";" in line]
    assert fields == [f[0] for f in fa.FaFwdParams._fields_]
    # size and the offset of the last field as the C compiler lays the struct out
    import subprocess
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "layout.c")
        with open(src, "w") as f:
            f.write('#include <stdio.h>\n#include <stddef.h>\n#include "fa_fwd.h"\n'
                    'int main(void){printf("%zu %zu %zu\\n", sizeof(fa_fwd_params), offsetof(fa_fwd_params, o_strides),'
                    ' offsetof(fa_fwd_params, dtype));return 0;}\n')
        exe = os.path.join(tmp, "layout")
        subprocess.run(["gcc", "-I", os.path.join(REPO, "include"), src, "-o", exe], check=True)
        size, off_last, off_dtype = (int(x) for x in subprocess.run([exe], check=True, stdout=subprocess.PIPE, text=True).stdout.split())
    assert size == ctypes.sizeof(fa.FaFwdParams)
    assert off_last == fa.FaFwdParams.o_strides.offset and off_dtype == fa.FaFwdParams.dtype.offset
    # the first twenty are mykernelParamType's, in its order (include/utils.h:143-165)
    assert fields[:20] == ["Q", "K", "V", "O", "L", "M", "B", "N", "S", "d", "Tr", "Tc", "softmax_scale", "dropout_prob",
                           "seed", "states", "window_size_left", "window_size_right", "alibi_slopes_ptr", "split_num"]


def test_backward_struct_layout_and_status_codes(fa):
    text = open(os.path.join(REPO, "include", "fa_bwd.h")).read()
    body = re.search(r"typedef struct fa_bwd_params \{(.*?)\} fa_bwd_params;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = []
    for line in body.splitlines():
        if ";" in line:
            decl = re.sub(r"\[\d+\]", "", line.split(";")[0])
            fields += [re.findall(r"(\w+)\s*$", part)[0] for part in decl.split(",")]
    assert fields == [f[0] for f in fa.FaBwdParams._fields_]
    import subprocess
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "layout.c")
        with open(src, "w") as f:
            f.write('#include <stdio.h>\n#include <stddef.h>\n#include "fa_bwd.h"\n'
                    'int main(void){printf("%zu %zu %zu\\n", sizeof(fa_bwd_params), offsetof(fa_bwd_params, softmax_scale),'
                    ' offsetof(fa_bwd_params, seed));return 0;}\n')
        exe = os.path.join(tmp, "layout")
        subprocess.run(["gcc", "-I", os.path.join(REPO, "include"), src, "-o", exe], check=True)
        size, off_scale, off_ws = (int(x) for x in subprocess.run([exe], check=True, stdout=subprocess.PIPE, text=True).stdout.split())
    assert size == ctypes.sizeof(fa.FaBwdParams)
    assert off_scale == fa.FaBwdParams.softmax_scale.offset and off_ws == fa.FaBwdParams.seed.offset

    L = fa.lib()
    ok = dict(B=2, N=4, S=1024, d=128, q_ptr=0x1000, k_ptr=0x2000, v_ptr=0x3000, o_ptr=0x4000, do_ptr=0x5000,
              lse_ptr=0x6000, dq_ptr=0x7000, dk_ptr=0x8000, dv_ptr=0x9000, workspace_ptr=0xA000, workspace_bytes=2 * 2 * 4 * 1024 * 4)

    def status(**kw):
        a = dict(ok)
        a.update(kw)
        return L.fa_bwd_validate(ctypes.byref(fa.make_bwd_params(**a)))
    assert status() == fa.FA_OK
    assert L.fa_bwd_workspace_bytes(ctypes.byref(fa.make_bwd_params(**ok))) == 2 * 2 * 4 * 1024 * 4
    assert L.fa_bwd_validate(None) == fa.FA_ERR_NULL_POINTER
    for missing in ("q_ptr", "k_ptr", "v_ptr", "o_ptr", "do_ptr", "lse_ptr", "dq_ptr", "dk_ptr", "dv_ptr"):
        assert status(**{missing: 0}) == fa.FA_ERR_NULL_POINTER
    assert status(B=0) == fa.FA_ERR_BAD_SHAPE and status(S=-128) == fa.FA_ERR_BAD_SHAPE
    assert status(d=96) == fa.FA_ERR_HEAD_DIM
    assert status(S=1000) == fa.FA_OK and status(S_kv=-1) == fa.FA_ERR_BAD_SHAPE
    assert status(n_kv_heads=3) == fa.FA_ERR_LAYOUT and status(n_kv_heads=2) == fa.FA_OK
    assert status(dropout_prob=1.0) == fa.FA_ERR_UNSUPPORTED and status(dropout_prob=0.3) == fa.FA_OK
    assert status(strides=dict(dk=(8, 8, 100))) == fa.FA_ERR_LAYOUT and status(strides=dict(q=(4 * 1024 * 256, 256, 4 * 256))) == fa.FA_OK
    assert status(dtype=7) == fa.FA_ERR_DTYPE
    assert status(softmax_scale=0.0) == fa.FA_ERR_SCALE and status(softmax_scale=float("nan")) == fa.FA_ERR_SCALE
    assert status(dq_ptr=0x7008) == fa.FA_ERR_LAYOUT
    assert status(workspace_ptr=0) == fa.FA_ERR_WORKSPACE and status(workspace_bytes=2 * 2 * 4 * 1024 * 4 - 1) == fa.FA_ERR_WORKSPACE
    # launching needs a device; without one the call fails with a status, it does not crash
    assert L.fa_bwd(ctypes.byref(fa.make_bwd_params(**dict(ok, d=80))), None) == fa.FA_ERR_HEAD_DIM
    assert L.fa_bwd_algorithmic_flops(2, 4, 1024, 128, 0, -1, -1) == 2.5 * L.fa_algorithmic_flops(2, 4, 1024, 128, 0, -1, -1)


def test_validate_status_codes(fa):
    L = fa.lib()
    ok = dict(B=2, N=8, S=2048, d=64, q_ptr=0x1000, k_ptr=0x2000, v_ptr=0x3000, o_ptr=0x4000)

    def status(**kw):
        a = dict(ok)
        a.update(kw)
        return L.fa_fwd_validate(ctypes.byref(fa.make_params(**a)))

    def status_raw(raw, **kw):
        a = dict(ok)
        a.update(kw)
        p = fa.make_params(**a)
        for k, v in raw.items():
            setattr(p, k, v)
        return L.fa_fwd_validate(ctypes.byref(p))

    assert status() == fa.FA_OK
    assert L.fa_fwd_validate(None) == fa.FA_ERR_NULL_POINTER
    for missing in ("q_ptr", "k_ptr", "v_ptr", "o_ptr"):
        assert status(**{missing: 0}) == fa.FA_ERR_NULL_POINTER
    assert status(B=0) == fa.FA_ERR_BAD_SHAPE
    assert status(N=-1) == fa.FA_ERR_BAD_SHAPE
    assert status(S=0) == fa.FA_ERR_BAD_SHAPE
    for d in (0, 32, 96, 256):
        assert status(d=d, softmax_scale=0.1) == fa.FA_ERR_HEAD_DIM            # the reference throws, flash_forward.h:587-589
    for S in (1, 64, 100, 2048 + 64):
        assert status(S=S) == fa.FA_OK                      # any length (the reference silently assumes S % 128 == 0)
    assert status(dtype=2) == fa.FA_ERR_DTYPE
    assert status(softmax_scale=0.0) == fa.FA_ERR_SCALE
    assert status(softmax_scale=float("nan")) == fa.FA_ERR_SCALE
    assert status(softmax_scale=float("inf")) == fa.FA_ERR_SCALE
    assert status_raw(dict(dropout_prob=0.1)) == fa.FA_OK                    # dropout is accepted ...
    assert status_raw(dict(states=0x10)) == fa.FA_OK                         # ... the curand states are ignored
    for bad_p in (1.0, 1.5, -0.1, float("nan")):
        assert status_raw(dict(dropout_prob=bad_p)) == fa.FA_ERR_UNSUPPORTED
    assert status_raw(dict(alibi_slopes_ptr=0x10)) == fa.FA_OK               # ALiBi slopes are accepted
    assert status(B=70000, N=70000, S=128) == fa.FA_ERR_TOO_LARGE
    # layouts: K/V heads must divide the query heads, strides are multiples of 8 elements with a row stride of
    # at least the head dimension, pointers are 16-byte aligned
    assert status(n_kv_heads=2) == fa.FA_OK and status(n_kv_heads=8) == fa.FA_OK
    assert status(n_kv_heads=3) == fa.FA_ERR_LAYOUT and status(n_kv_heads=-1) == fa.FA_ERR_LAYOUT
    bshd = (2048 * 8 * 64, 64, 8 * 64)
    assert status(q_strides=bshd, k_strides=bshd, v_strides=bshd, o_strides=bshd) == fa.FA_OK
    assert status(q_strides=(2048 * 8 * 64, 64, 8 * 64 + 4)) == fa.FA_ERR_LAYOUT
    assert status(k_strides=(2048 * 8 * 64, 64, 32)) == fa.FA_ERR_LAYOUT
    assert status(v_strides=(-8, 64, 512)) == fa.FA_ERR_LAYOUT
    assert status(o_strides=(0, 0, 1 << 25)) == fa.FA_ERR_TOO_LARGE
    assert status(q_ptr=0x1008) == fa.FA_ERR_LAYOUT
    # an output with a zero batch or head stride would have several writers per element; inputs may broadcast
    assert status(o_strides=(0, 2048 * 64, 64)) == fa.FA_ERR_LAYOUT
    assert status(o_strides=(8 * 2048 * 64, 0, 64)) == fa.FA_ERR_LAYOUT
    assert status(k_strides=(0, 2048 * 64, 64)) == fa.FA_OK
    assert status(B=1, o_strides=(0, 2048 * 64, 64)) == fa.FA_OK
    # tile and mask arithmetic is 32-bit: S + S_kv must stay below 2^30
    assert status(B=1, N=1, S=0x20000000) == fa.FA_ERR_TOO_LARGE
    assert status(B=1, N=1, S=128, S_kv=0x3fffff80) == fa.FA_ERR_TOO_LARGE
    assert status(B=1, N=1, S=128, S_kv=0x3fffff00) == fa.FA_OK
    # fa_fwd itself refuses the same blocks before touching any device
    p = fa.make_params(**dict(ok, d=96))
    assert L.fa_fwd(ctypes.byref(p), None) == fa.FA_ERR_HEAD_DIM


def test_static_scratch_entry_point_checks_before_touching_a_device(fa):
    L = fa.lib()
    limit = L.fa_fwd_static_scratch_bytes()
    assert limit == 32 << 20
    ok = dict(B=2, N=8, S=4, d=64, q_ptr=0x1000, k_ptr=0x2000, v_ptr=0x3000, o_ptr=0x4000, S_kv=4096)
    # the same argument checks as fa_fwd, workspace fields ignored
    assert L.fa_fwd_split_static(ctypes.byref(fa.make_params(**dict(ok, d=96))), None) == fa.FA_ERR_HEAD_DIM
    assert L.fa_fwd_split_static(None, None) == fa.FA_ERR_NULL_POINTER
    # partial results beyond the static array are refused with a status of their own
    big = fa.make_params(**dict(ok, B=8, N=32, S=128, S_kv=8192, d=128, split_num=16))
    assert L.fa_fwd_workspace_bytes(ctypes.byref(big)) > limit
    assert L.fa_fwd_split_static(ctypes.byref(big), None) == fa.FA_ERR_SCRATCH_LIMIT
    assert b"static scratch" in L.fa_strerror(fa.FA_ERR_SCRATCH_LIMIT)


def test_python_stride_marshalling():
    """What the binding hands the ABI for tensors whose strides the ABI cannot take as they are."""
    import torch
    fa = __import__("conftest").load_package()
    dense = torch.zeros(2, 4, 16, 64, dtype=torch.float16)
    assert fa.abi_strides(dense) == (dense, None) or fa.abi_strides(dense)[1] is None
    bshd = torch.zeros(2, 16, 4, 64, dtype=torch.float16).transpose(1, 2)
    t, st = fa.abi_strides(bshd)
    assert t is bshd and st == (16 * 4 * 64, 64, 4 * 64)
    # an expanded gradient (zero strides, as produced by o.sum().backward()) must not reach the ABI as
    # (0, 0, 0), which means "dense": it is copied
    expanded = torch.ones(64, dtype=torch.float16).expand(2, 4, 16, 64)
    assert expanded.stride() == (0, 0, 0, 1)
    t, st = fa.abi_strides(expanded)
    assert st is None and t.is_contiguous() and t.shape == expanded.shape
    part = torch.zeros(2, 1, 16, 64, dtype=torch.float16).expand(2, 4, 16, 64)       # one zero stride
    t, st = fa.abi_strides(part)
    assert st is None and t.is_contiguous()
    # strides that are no multiple of 8 elements, or a head dimension that is not contiguous: copied
    odd = torch.zeros(2, 4, 16, 68, dtype=torch.float16)[..., :64]
    t, st = fa.abi_strides(odd)
    assert st is None and t.is_contiguous()
    strided_d = torch.zeros(2, 4, 16, 128, dtype=torch.float16)[..., ::2]
    t, st = fa.abi_strides(strided_d)
    assert st is None and t.is_contiguous()
    # a row stride larger than d that is a multiple of 8 passes through
    wide = torch.zeros(2, 4, 16, 96, dtype=torch.float16)[..., :64]
    t, st = fa.abi_strides(wide)
    assert t is wide and st == (4 * 16 * 96, 16 * 96, 96)
    # strides of size-one dimensions carry no information and never make the triple all zero or odd
    one = torch.zeros(1, 4, 16, 96, dtype=torch.float16)[..., :64].as_strided((1, 4, 16, 64), (3, 16 * 96, 96, 1))
    t, st = fa.abi_strides(one)
    assert t is one and st[1:] == (16 * 96, 96) and st[0] % 8 == 0 and st[0] > 0


def test_reference_entry_point_rejects_unsupported_flags(fa):
    L = fa.lib()
    args = [2, 8, 2048, 64, 0x1000, 0x2000, 0x3000, 0x4000, None, None]
    assert L.run_flash_attention(*args, 1, 0, 0, 0, 0, None, 1.0, None) == fa.FA_ERR_UNSUPPORTED   # dropout with p = 1
    assert L.run_flash_attention(*args, 0, 0, 0, 1, 0, None, 0.0, None) == fa.FA_ERR_NULL_POINTER  # ALiBi without slopes
    bad = list(args)
    bad[3] = 48
    assert L.run_flash_attention(*bad, 0, 0, 0, 0, 0, None, 0.0, None) == fa.FA_ERR_HEAD_DIM
    bad = list(args)
    bad[4] = None
    assert L.run_flash_attention(*bad, 0, 1, 0, 0, 0, None, 0.0, None) == fa.FA_ERR_NULL_POINTER


def test_strerror_covers_every_status(fa):
    L = fa.lib()
    seen = set()
    for st in range(0, -12, -1):
        msg = L.fa_strerror(st).decode()
        assert msg and msg != "unknown status"
        seen.add(msg)
    assert len(seen) == 12
    assert L.fa_strerror(-99).decode() == "unknown status"


def test_missing_library_fails_loudly(fa, monkeypatch):
    monkeypatch.setattr(fa, "_lib", None)
    monkeypatch.setattr(fa, "LIB_PATH", "/nonexistent/libfa_fwd_gfx950.so")
    with pytest.raises(RuntimeError, match="is missing"):
        fa.lib()


def test_python_wrapper_refuses_cpu_tensors(fa):
    import torch
    q = torch.zeros(1, 1, 128, 64, dtype=torch.float16)
    with pytest.raises(ValueError):
        fa.flash_attention_forward(q, q, q)


def test_dropout_host_mirror(fa):
    """fa_dropout_threshold rounds p to 1/256; fa_dropout_keep follows the published definition (numpy Philox)."""
    from parity_util import numpy_keep_mask
    L = fa.lib()
    assert [L.fa_dropout_threshold(p) for p in (0.0, -1.0, 0.001, 0.1, 0.5, 0.999, 1.0)] == [0, 0, 0, 26, 128, 255, 255]
    for seed, bh, thr in ((48, 3, 26), (0xFEDCBA9876543210, 70, 200)):
        want = numpy_keep_mask(seed, bh, 80, thr)
        got = np.array([[L.fa_dropout_keep(seed, bh, i, j, thr) for j in range(80)] for i in range(80)], dtype=bool)
        assert np.array_equal(got, want)


def test_backward_key_block_schedule_against_brute_force(fa):
    """The key-owning backward kernel walks the query tiles that see its keys; its range and tile classes come
    from the forward's arithmetic with the mask's two sides exchanged and shifted by S_kv - S.  Checked here
    against the mask predicate itself, pair by pair, for lengths that differ either way."""
    L = fa.lib()
    rng = np.random.default_rng(5)
    cases = [(256, 0, 1, -1, -1), (300, 0, 1, 37, -1), (200, 456, 1, -1, -1), (320, 70, 1, 20, -1), (129, 513, 0, 10, 10),
             (192, 64, 1, -1, -1), (257, 100, 0, -1, -1), (64, 640, 0, 100, 3), (500, 500, 0, -1, 33), (70, 300, 1, 0, -1)]
    for S, S_kv, causal, wl, wr in cases:
        Sk = S_kv or S
        pos = np.arange(S)[:, None] + (Sk - S)
        j = np.arange(Sk)[None, :]
        vis = np.ones((S, Sk), dtype=bool)
        if causal:
            vis &= j <= pos
        if wl >= 0:
            vis &= pos - j <= wl
        if wr >= 0 and not causal:
            vis &= j - pos <= wr
        n_tiles = (S + 63) // 64
        for rows in (32, 256):
            for k_begin in range(0, Sk, rows):
                n = min(rows, Sk - k_begin)
                block = vis[:, k_begin:k_begin + n]
                lo, hi = ctypes.c_int(), ctypes.c_int()
                L.fa_bwd_sched_query_tile_range(S, S_kv, causal, wl, wr, k_begin, n, ctypes.byref(lo), ctypes.byref(hi))
                seen = [t for t in range(n_tiles) if block[64 * t:64 * t + 64].any()]
                if not seen:
                    assert lo.value > hi.value, (S, S_kv, causal, wl, wr, k_begin)
                    continue
                # the band is contiguous: the range is exactly the tiles with a visible pair
                assert (lo.value, hi.value) == (seen[0], seen[-1]), (S, S_kv, causal, wl, wr, k_begin, rows)
                for t in range(lo.value, hi.value + 1):
                    if 64 * t + 64 > S:
                        continue                      # the ragged last tile is always treated as mixed by the kernel
                    sub = block[64 * t:64 * t + 64]
                    cls = L.fa_bwd_sched_classify(S, S_kv, causal, wl, wr, k_begin, n, t)
                    assert cls == (2 if sub.all() else 0 if not sub.any() else 1), (S, S_kv, causal, wl, wr, k_begin, rows, t)


def test_backward_lds_layout_arithmetic_on_the_host():
    """The header the backward kernels take their LDS addresses from compiles as C: what the direct loads write
    is what both read patterns find, every address stays inside the tile, and neither pattern has a bank
    conflict (tests/c/check_bwd_layout.c)."""
    import subprocess
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        exe = os.path.join(tmp, "check_bwd_layout")
        subprocess.run(["gcc", "-O1", "-Wall", "-Wextra", "-I", os.path.join(REPO, "flash-attn-rtx5060_amd", "csrc"),
                        os.path.join(REPO, "tests", "c", "check_bwd_layout.c"), "-o", exe], check=True)
        out = subprocess.run([exe], stdout=subprocess.PIPE, text=True)
    assert out.returncode == 0, out.stdout


def test_key_split_suggestion_fills_the_device_once(fa):
    """fa_fwd_suggest_splits: work items (K/V-head groups packed into one item when few queries sit behind long
    keys) times splits should cover the 512 resident 4-wave workgroups of a 256-CU device once, with at least
    four 64-key tiles per split; problems that fill the device by themselves are not split."""
    L = fa.lib()

    def suggest(B, N, Nk, S, S_kv):
        p = fa.make_params(B, N, S, 128, 0x1000, 0x2000, 0x3000, 0x4000, causal=True, n_kv_heads=0 if Nk == N else Nk, S_kv=S_kv)
        return L.fa_fwd_suggest_splits(ctypes.byref(p))
    assert suggest(16, 32, 8, 1, 8192) == 4          # 128 packed items
    assert suggest(4, 32, 32, 1, 32768) == 4         # 128 items
    assert suggest(8, 32, 8, 4, 8192) == 8           # 64 packed items
    assert suggest(1, 32, 8, 1, 65536) == 64         # 8 packed items
    assert suggest(1, 8, 8, 1, 1024) == 4            # 8 items, capped by four tiles per split (16 tiles)
    assert suggest(64, 32, 8, 1, 2048) == 1          # 512 packed items fill the device
    assert suggest(2, 32, 32, 8192, 0) == 1          # a prefill-sized problem
