"""ctypes binding of the CPU oracle (oracle/libfa_oracle.so).  Test-side only."""
import ctypes
import os

import numpy as np

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F16, BF16 = 0, 1


class Cfg(ctypes.Structure):
    _fields_ = [("B", ctypes.c_int), ("H", ctypes.c_int), ("S", ctypes.c_int), ("D", ctypes.c_int),
                ("dtype", ctypes.c_int), ("scale", ctypes.c_float), ("causal", ctypes.c_int),
                ("window_left", ctypes.c_int), ("window_right", ctypes.c_int), ("alibi_slopes", ctypes.c_void_p),
                ("dropout_threshold", ctypes.c_int), ("dropout_seed", ctypes.c_uint64)]


_libs = {}


def lib(scalar=False):
    name = "libfa_oracle_scalar.so" if scalar else "libfa_oracle.so"
    if name not in _libs:
        path = os.path.join(REPO, "oracle", name)
        if not os.path.exists(path):
            raise RuntimeError(f"{path} missing: run `make -C oracle`")
        L = ctypes.CDLL(path)
        L.fa_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.fa_oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.fa_oracle_f16_to_f32.restype = ctypes.c_float
        L.fa_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.fa_oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.fa_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.fa_oracle_bf16_to_f32.restype = ctypes.c_float
        L.fa_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        vp = ctypes.c_void_p
        L.fa_oracle_rows.argtypes = [ctypes.POINTER(Cfg), vp, vp, vp, vp, ctypes.c_int64, vp, vp, ctypes.c_int]
        L.fa_oracle_full.argtypes = [ctypes.POINTER(Cfg), vp, vp, vp, vp, vp, ctypes.c_int]
        L.fa_oracle_rows_f64.argtypes = [ctypes.POINTER(Cfg), vp, vp, vp, vp, ctypes.c_int64, vp, vp, ctypes.c_int]
        L.fa_oracle_literal.argtypes = [ctypes.POINTER(Cfg), vp, vp, vp, vp]
        L.fa_oracle_bwd_f64.argtypes = [ctypes.POINTER(Cfg), vp, vp, vp, vp, vp, vp, vp, ctypes.c_int]
        L.fa_oracle_dropout_keep.argtypes = [ctypes.c_uint64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.fa_oracle_philox4x32_10.restype = None
        L.fa_oracle_philox4x32_10.argtypes = [ctypes.POINTER(ctypes.c_uint32)] * 3
        _libs[name] = L
    return _libs[name]


def _cfg(shape, dtype, scale, causal, wl, wr, slopes, dropout=(0, 0)):
    B, H, S, D = shape
    c = Cfg(B, H, S, D, dtype, scale, int(bool(causal)), wl, wr, None, int(dropout[0]), int(dropout[1]))
    if slopes is not None:
        c.alibi_slopes = slopes.ctypes.data
    return c


def _check(arrs):
    for a in arrs:
        assert a.dtype == np.uint16 and a.flags["C_CONTIGUOUS"]


def default_threads():
    return max(1, min(16, os.cpu_count() or 1))


def rows(q, k, v, row_idx, dtype=F16, scale=None, causal=False, wl=-1, wr=-1, slopes=None, threads=None, scalar=False,
         dropout=(0, 0)):
    """Faithful oracle on selected flat rows -> (O [n, D] uint16 bits, lse [n] float32).
    dropout = (threshold 0..255, seed)."""
    _check((q, k, v))
    B, H, S, D = q.shape
    scale = np.float32(1.0 / np.sqrt(D)) if scale is None else np.float32(scale)
    idx = np.ascontiguousarray(row_idx, dtype=np.int64)
    o = np.empty((len(idx), D), dtype=np.uint16)
    lse = np.empty((len(idx),), dtype=np.float32)
    c = _cfg(q.shape, dtype, scale, causal, wl, wr, slopes, dropout)
    rc = lib(scalar).fa_oracle_rows(ctypes.byref(c), q.ctypes.data, k.ctypes.data, v.ctypes.data, idx.ctypes.data,
                                    len(idx), o.ctypes.data, lse.ctypes.data, threads or default_threads())
    assert rc == 0
    return o, lse


def full(q, k, v, dtype=F16, scale=None, causal=False, wl=-1, wr=-1, slopes=None, threads=None, scalar=False, dropout=(0, 0)):
    B, H, S, D = q.shape
    o, lse = rows(q, k, v, np.arange(B * H * S, dtype=np.int64), dtype, scale, causal, wl, wr, slopes, threads, scalar, dropout)
    return o.reshape(B, H, S, D), lse.reshape(B, H, S)


def rows_f64(q, k, v, row_idx, dtype=F16, scale=None, causal=False, wl=-1, wr=-1, slopes=None, threads=None, dropout=(0, 0)):
    _check((q, k, v))
    B, H, S, D = q.shape
    scale = np.float32(1.0 / np.sqrt(D)) if scale is None else np.float32(scale)
    idx = np.ascontiguousarray(row_idx, dtype=np.int64)
    o = np.empty((len(idx), D), dtype=np.float64)
    lse = np.empty((len(idx),), dtype=np.float64)
    c = _cfg(q.shape, dtype, scale, causal, wl, wr, slopes, dropout)
    rc = lib().fa_oracle_rows_f64(ctypes.byref(c), q.ctypes.data, k.ctypes.data, v.ctypes.data, idx.ctypes.data,
                                  len(idx), o.ctypes.data, lse.ctypes.data, threads or default_threads())
    assert rc == 0
    return o, lse


def literal(q, k, v, dtype=F16, scale=None, causal=False, wl=-1, wr=-1, slopes=None, scalar=False, dropout=(0, 0)):
    _check((q, k, v))
    B, H, S, D = q.shape
    scale = np.float32(1.0 / np.sqrt(D)) if scale is None else np.float32(scale)
    o = np.empty((B, H, S, D), dtype=np.uint16)
    c = _cfg(q.shape, dtype, scale, causal, wl, wr, slopes, dropout)
    rc = lib(scalar).fa_oracle_literal(ctypes.byref(c), q.ctypes.data, k.ctypes.data, v.ctypes.data, o.ctypes.data)
    assert rc == 0
    return o


def bwd_f64(q, k, v, do, dtype=F16, scale=None, causal=False, wl=-1, wr=-1, slopes=None, threads=None, dropout=(0, 0)):
    """fp64 gradients (dQ, dK, dV), each [B,H,S,D] float64, of sum(dO * O)."""
    _check((q, k, v, do))
    B, H, S, D = q.shape
    scale = np.float32(1.0 / np.sqrt(D)) if scale is None else np.float32(scale)
    dq, dk, dv = (np.empty((B, H, S, D), dtype=np.float64) for _ in range(3))
    c = _cfg(q.shape, dtype, scale, causal, wl, wr, slopes, dropout)
    rc = lib().fa_oracle_bwd_f64(ctypes.byref(c), q.ctypes.data, k.ctypes.data, v.ctypes.data, do.ctypes.data,
                                 dq.ctypes.data, dk.ctypes.data, dv.ctypes.data, threads or default_threads())
    assert rc == 0
    return dq, dk, dv


def to_f32(bits, dtype):
    """uint16 storage bits -> float32 numpy."""
    bits = np.asarray(bits, dtype=np.uint16)
    if dtype == F16:
        return bits.view(np.float16).astype(np.float32)
    return (bits.astype(np.uint32) << 16).view(np.float32)


def from_f32(x, dtype):
    """float32 numpy -> uint16 storage bits, round-to-nearest-even (numpy for fp16, bit trick for bf16)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if dtype == F16:
        return x.astype(np.float16).view(np.uint16)
    u = x.view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)
