"""Python binding of libfa_fwd_gfx950.so (ctypes over the C ABI in include/fa_fwd.h).

Mirrors the reference operator ``run_flash_attention``
(reference src/flash_forward.h:593-612) for callers that hold their tensors in
PyTorch: same argument meaning, tensors are contiguous [B, N, S, d] fp16/bf16 on
the GPU.  PyTorch is used only for device memory and the current stream; all
arithmetic happens in the HIP library.  There is no fallback: if the shared
library has not been built, importing a symbol from it raises.

The directory name contains a hyphen, so the package is loaded by path::

    import importlib.util, sys
    spec = importlib.util.spec_from_file_location(
        "flash_attn_rtx5060_amd", "<repo>/flash-attn-rtx5060_amd/__init__.py")
    mod = importlib.util.module_from_spec(spec); sys.modules[spec.name] = mod
    spec.loader.exec_module(mod)
"""
import ctypes
import math
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfa_fwd_gfx950.so")
HOST_LIB_PATH = os.path.join(_HERE, "lib", "libfa_host.so")
HARNESS_PATH = os.path.join(_HERE, "bin", "fa_harness")

FA_OK = 0
FA_ERR_NULL_POINTER = -1
FA_ERR_BAD_SHAPE = -2
FA_ERR_HEAD_DIM = -3
FA_ERR_SEQLEN_MULTIPLE = -4
FA_ERR_UNSUPPORTED = -5
FA_ERR_DTYPE = -6
FA_ERR_SCALE = -7
FA_ERR_DEVICE = -8
FA_ERR_NO_DEVICE = -9
FA_ERR_TOO_LARGE = -10
FA_ERR_LAYOUT = -11
FA_ERR_WORKSPACE = -12
FA_ERR_SCRATCH_LIMIT = -13
FA_DTYPE_F16 = 0
FA_DTYPE_BF16 = 1
FA_SCHED_AUTO, FA_SCHED_DISPATCH, FA_SCHED_PERSISTENT, FA_SCHED_QUEUE = 0, 1, 2, 3
FA_TILE_SKIP, FA_TILE_PARTIAL, FA_TILE_FULL = 0, 1, 2

#: every symbol include/fa_fwd.h declares
EXPORTED_SYMBOLS = (
    "fa_fwd_validate", "fa_fwd", "fa_init", "fa_fwd_split_static", "fa_fwd_static_scratch_bytes",
    "fa_reset_work_queues", "fa_release_work_queue", "run_flash_attention", "fa_strerror", "fa_last_device_error",
    "fa_sched_block_rows", "fa_sched_block_keys", "fa_sched_num_items", "fa_sched_item",
    "fa_sched_heads", "fa_sched_tile_range", "fa_sched_classify", "fa_count_pairs", "fa_algorithmic_flops",
    "fa_dropout_threshold", "fa_dropout_keep", "fa_fwd_workspace_bytes", "fa_fwd_suggest_splits",
    "fa_bwd_validate", "fa_bwd", "fa_bwd_workspace_bytes", "fa_bwd_fast_workspace_bytes", "fa_bwd_min_fast_workspace_bytes",
    "fa_bwd_algorithmic_flops",
    "fa_bwd_sched_query_tile_range", "fa_bwd_sched_classify",
    "fa_dev_count", "fa_dev_name", "fa_dev_malloc", "fa_dev_free", "fa_dev_h2d", "fa_dev_d2h",
    "fa_dev_memset", "fa_dev_sync", "fa_event_create", "fa_event_record", "fa_event_sync",
    "fa_event_elapsed_ms", "fa_event_destroy",
)


class FaFwdParams(ctypes.Structure):
    """struct fa_fwd_params of include/fa_fwd.h (field-for-field)."""
    _fields_ = [
        ("Q", ctypes.c_void_p), ("K", ctypes.c_void_p), ("V", ctypes.c_void_p), ("O", ctypes.c_void_p),
        ("L", ctypes.c_void_p), ("M", ctypes.c_void_p),
        ("B", ctypes.c_int), ("N", ctypes.c_int), ("S", ctypes.c_int), ("d", ctypes.c_int),
        ("Tr", ctypes.c_int), ("Tc", ctypes.c_int),
        ("softmax_scale", ctypes.c_float), ("dropout_prob", ctypes.c_float),
        ("seed", ctypes.c_ulonglong), ("states", ctypes.c_void_p),
        ("window_size_left", ctypes.c_int), ("window_size_right", ctypes.c_int),
        ("alibi_slopes_ptr", ctypes.c_void_p), ("split_num", ctypes.c_int),
        ("dtype", ctypes.c_int), ("is_causal", ctypes.c_int), ("sched", ctypes.c_int),
        ("n_kv_heads", ctypes.c_int),
        ("q_strides", ctypes.c_longlong * 3), ("k_strides", ctypes.c_longlong * 3),
        ("v_strides", ctypes.c_longlong * 3), ("o_strides", ctypes.c_longlong * 3),
        ("S_kv", ctypes.c_int), ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_ulonglong),
        ("exact_first_rows", ctypes.c_int),
    ]


class FaBwdParams(ctypes.Structure):
    """struct fa_bwd_params of include/fa_bwd.h (field-for-field)."""
    _fields_ = [
        ("Q", ctypes.c_void_p), ("K", ctypes.c_void_p), ("V", ctypes.c_void_p), ("O", ctypes.c_void_p),
        ("dO", ctypes.c_void_p), ("L", ctypes.c_void_p),
        ("dQ", ctypes.c_void_p), ("dK", ctypes.c_void_p), ("dV", ctypes.c_void_p),
        ("B", ctypes.c_int), ("N", ctypes.c_int), ("S", ctypes.c_int), ("d", ctypes.c_int),
        ("softmax_scale", ctypes.c_float),
        ("window_size_left", ctypes.c_int), ("window_size_right", ctypes.c_int),
        ("dtype", ctypes.c_int), ("is_causal", ctypes.c_int),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_ulonglong),
        ("n_kv_heads", ctypes.c_int), ("S_kv", ctypes.c_int), ("alibi_slopes_ptr", ctypes.c_void_p),
        ("q_strides", ctypes.c_longlong * 3), ("k_strides", ctypes.c_longlong * 3),
        ("v_strides", ctypes.c_longlong * 3), ("o_strides", ctypes.c_longlong * 3),
        ("do_strides", ctypes.c_longlong * 3), ("dq_strides", ctypes.c_longlong * 3),
        ("dk_strides", ctypes.c_longlong * 3), ("dv_strides", ctypes.c_longlong * 3),
        ("dropout_prob", ctypes.c_float), ("seed", ctypes.c_ulonglong),
    ]


class FaError(RuntimeError):
    def __init__(self, status, detail=""):
        self.status = status
        msg = lib().fa_strerror(status).decode()
        super().__init__(f"fa_fwd status {status}: {msg}{(' (' + detail + ')') if detail else ''}")


_lib = None
_host = None


def lib():
    """The C-ABI library; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run `make -C {_HERE}` (hipcc, gfx950) first")
        # PyTorch ships its own copy of the HIP runtime.  A process that uses both must load PyTorch's first, so
        # that this library binds to the same runtime instance; loaded the other way round, the second runtime
        # to initialise reports "no ROCm-capable device".
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = ctypes.CDLL(LIB_PATH)
        L.fa_strerror.restype = ctypes.c_char_p
        L.fa_strerror.argtypes = [ctypes.c_int]
        L.fa_last_device_error.restype = ctypes.c_char_p
        L.fa_fwd_validate.argtypes = [ctypes.POINTER(FaFwdParams)]
        L.fa_fwd.argtypes = [ctypes.POINTER(FaFwdParams), ctypes.c_void_p]
        L.fa_fwd_split_static.argtypes = [ctypes.POINTER(FaFwdParams), ctypes.c_void_p]
        L.fa_fwd_static_scratch_bytes.restype = ctypes.c_ulonglong
        L.fa_release_work_queue.argtypes = [ctypes.c_void_p]
        L.fa_fwd_workspace_bytes.restype = ctypes.c_ulonglong
        L.fa_fwd_workspace_bytes.argtypes = [ctypes.POINTER(FaFwdParams)]
        L.fa_fwd_suggest_splits.argtypes = [ctypes.POINTER(FaFwdParams)]
        L.run_flash_attention.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p] * 6 + [ctypes.c_int] * 5 + [
            ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p]
        L.fa_sched_block_rows.argtypes = [ctypes.c_int] * 7
        L.fa_sched_block_keys.argtypes = [ctypes.c_int]
        L.fa_sched_num_items.restype = ctypes.c_longlong
        L.fa_sched_num_items.argtypes = [ctypes.c_int] * 7
        L.fa_sched_item.argtypes = [ctypes.c_int] * 7 + [ctypes.c_longlong, ctypes.POINTER(ctypes.c_int),
                                                         ctypes.POINTER(ctypes.c_int)]
        L.fa_sched_heads.argtypes = [ctypes.c_int] * 3 + [ctypes.POINTER(ctypes.c_int)] * 3
        L.fa_sched_tile_range.restype = None
        L.fa_sched_tile_range.argtypes = [ctypes.c_int] * 7 + [ctypes.POINTER(ctypes.c_int)] * 2
        L.fa_sched_classify.argtypes = [ctypes.c_int] * 7
        L.fa_count_pairs.restype = ctypes.c_longlong
        L.fa_count_pairs.argtypes = [ctypes.c_int] * 4
        L.fa_algorithmic_flops.restype = ctypes.c_double
        L.fa_algorithmic_flops.argtypes = [ctypes.c_int] * 7
        L.fa_dropout_threshold.argtypes = [ctypes.c_float]
        L.fa_bwd_validate.argtypes = [ctypes.POINTER(FaBwdParams)]
        L.fa_bwd.argtypes = [ctypes.POINTER(FaBwdParams), ctypes.c_void_p]
        L.fa_bwd_workspace_bytes.restype = ctypes.c_ulonglong
        L.fa_bwd_workspace_bytes.argtypes = [ctypes.POINTER(FaBwdParams)]
        L.fa_bwd_fast_workspace_bytes.restype = ctypes.c_ulonglong
        L.fa_bwd_fast_workspace_bytes.argtypes = [ctypes.POINTER(FaBwdParams)]
        L.fa_bwd_min_fast_workspace_bytes.restype = ctypes.c_ulonglong
        L.fa_bwd_min_fast_workspace_bytes.argtypes = [ctypes.POINTER(FaBwdParams)]
        L.fa_bwd_algorithmic_flops.restype = ctypes.c_double
        L.fa_bwd_algorithmic_flops.argtypes = [ctypes.c_int] * 7
        L.fa_bwd_sched_query_tile_range.restype = None
        L.fa_bwd_sched_query_tile_range.argtypes = [ctypes.c_int] * 7 + [ctypes.POINTER(ctypes.c_int)] * 2
        L.fa_bwd_sched_classify.argtypes = [ctypes.c_int] * 8
        L.fa_dropout_keep.argtypes = [ctypes.c_ulonglong, ctypes.c_longlong, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        _lib = L
    return _lib


def host_lib():
    """Host-side helper library (seeded input generator, host/fa_inputs.h)."""
    global _host
    if _host is None:
        if not os.path.exists(HOST_LIB_PATH):
            raise RuntimeError(f"{HOST_LIB_PATH} is missing: run `make -C {_HERE}` first")
        H = ctypes.CDLL(HOST_LIB_PATH)
        H.fa_fill_normal.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int, ctypes.c_int, ctypes.c_uint64,
                                     ctypes.c_uint32, ctypes.c_float, ctypes.c_double, ctypes.c_float, ctypes.c_int]
        H.fa_input_normal.restype = ctypes.c_float
        H.fa_input_normal.argtypes = [ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint64]
        H.fa_input_row_selected.argtypes = [ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_double]
        H.fa_philox4x32_10.restype = None
        H.fa_philox4x32_10.argtypes = [ctypes.POINTER(ctypes.c_uint32)] * 3
        for name, rt, at in (("fa_f32_to_f16_bits", ctypes.c_uint16, ctypes.c_float),
                             ("fa_f32_to_bf16_bits", ctypes.c_uint16, ctypes.c_float),
                             ("fa_f16_bits_to_f32", ctypes.c_float, ctypes.c_uint16),
                             ("fa_bf16_bits_to_f32", ctypes.c_float, ctypes.c_uint16)):
            getattr(H, name).restype = rt
            getattr(H, name).argtypes = [at]
        _host = H
    return _host


def make_params(B, N, S, d, q_ptr=0, k_ptr=0, v_ptr=0, o_ptr=0, lse_ptr=0, softmax_scale=None, causal=False,
                window_left=-1, window_right=-1, dtype=FA_DTYPE_F16, sched=FA_SCHED_AUTO, alibi_ptr=0,
                n_kv_heads=0, q_strides=None, k_strides=None, v_strides=None, o_strides=None, dropout_prob=0.0, seed=0,
                S_kv=0, split_num=0, workspace_ptr=0, workspace_bytes=0, exact_first_rows=False):
    """A filled fa_fwd_params.  Strides are (batch, head, row) in elements, None = contiguous [B,N,S,d]."""
    p = FaFwdParams()
    p.exact_first_rows = int(bool(exact_first_rows))
    p.alibi_slopes_ptr = alibi_ptr or None
    p.n_kv_heads = n_kv_heads
    p.dropout_prob, p.seed = dropout_prob, seed
    p.S_kv, p.split_num, p.workspace, p.workspace_bytes = S_kv, split_num, workspace_ptr or None, workspace_bytes
    for name, st in (("q_strides", q_strides), ("k_strides", k_strides), ("v_strides", v_strides), ("o_strides", o_strides)):
        if st is not None:
            setattr(p, name, (ctypes.c_longlong * 3)(*st))
    p.Q, p.K, p.V, p.O, p.L = q_ptr or None, k_ptr or None, v_ptr or None, o_ptr or None, lse_ptr or None
    p.B, p.N, p.S, p.d = B, N, S, d
    p.softmax_scale = (1.0 / math.sqrt(d)) if softmax_scale is None else softmax_scale
    p.window_size_left, p.window_size_right = window_left, window_right
    p.dtype, p.is_causal, p.sched = dtype, int(bool(causal)), sched
    return p


def abi_strides(t):
    """What the C ABI gets for a 4-d tensor [.., .., rows, d]: ``(tensor, strides)`` with strides None for a
    dense tensor and the (batch, head, row) element strides otherwise.  The ABI reads an all-zero triple as
    "dense", wants every stride to be a non-negative multiple of 8 elements, the row stride at least d and the
    last dimension contiguous; a tensor that does not fit that (an expanded gradient with zero strides, an
    odd slice) is replaced by a dense copy.  Strides of dimensions of size one carry no information and are
    set to the dense value."""
    if t.is_contiguous():
        return t, None
    st = list(t.stride())
    shape = list(t.shape)
    ok = st[3] == 1
    dense = shape[3]
    norm = [0, 0, 0]
    for k in (2, 1, 0):
        if shape[k] == 1:
            norm[k] = max(dense, 8)
        else:
            norm[k] = st[k]
            if st[k] <= 0 or st[k] % 8 != 0:
                ok = False
        dense *= shape[k]
    if shape[2] > 1 and st[2] < shape[3]:
        ok = False
    if not ok:
        return t.contiguous(), None
    return t, tuple(norm)


def flash_attention_forward(q, k, v, softmax_scale=None, causal=False, window_left=-1, window_right=-1,
                            return_lse=True, out=None, lse=None, sched=FA_SCHED_AUTO, alibi_slopes=None,
                            dropout_prob=0.0, seed=0, splits=1, exact_first_rows=False, static_scratch=False):
    """O, LSE = attention(q, k, v) on the GPU through fa_fwd().  q is [B, N, S, d], k and v are
    [B, Nk, S, d] with Nk dividing N (Nk < N: grouped-query attention); any strides with a contiguous last
    dimension are passed through (a [B, S, N, d] tensor is given as ``t.transpose(1, 2)``), any S >= 1.
    k and v may be longer or shorter than q ([B, Nk, S_kv, d]): query i then sits at key position
    i + S_kv - S.  ``splits``: an int > 1, or "auto", splits the keys of every query block over several
    workgroups and merges the partial results (few queries, long keys).
    ``alibi_slopes``: fp32 GPU tensor [N]; slope[h]*|i-j| is subtracted from every scaled score (mask.h:21-26).
    ``exact_first_rows``: see fa_fwd_params.exact_first_rows.  ``static_scratch``: go through
    fa_fwd_split_static (the key splits' partial results in the library's own static device array)."""
    import torch
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise ValueError("q, k, v must live on the GPU")
    if q.dtype not in (torch.float16, torch.bfloat16) or k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError("q, k, v must share dtype float16 or bfloat16")
    if q.dim() != 4 or k.shape != v.shape or k.dim() != 4 or (q.shape[0], q.shape[3]) != (
            k.shape[0], k.shape[3]) or k.shape[1] == 0 or q.shape[1] % k.shape[1] != 0 or k.shape[2] == 0:
        raise ValueError("q must be [B, N, S, d], k and v [B, Nk, S_kv, d] with Nk dividing N")
    (q, q_st), (k, k_st), (v, v_st) = abi_strides(q), abi_strides(k), abi_strides(v)
    B, N, S, d = q.shape
    Nk, S_kv = k.shape[1], k.shape[2]
    if alibi_slopes is not None and not (alibi_slopes.is_cuda and alibi_slopes.dtype == torch.float32
                                         and alibi_slopes.is_contiguous() and tuple(alibi_slopes.shape) == (N,)):
        raise ValueError("alibi_slopes must be a contiguous float32 GPU tensor of shape [N]")
    if out is None:
        out = torch.empty_like(q)          # keeps q's strides
    if out.shape != q.shape or out.dtype != q.dtype:
        raise ValueError("out must have q's shape and dtype")
    out_abi, o_st = abi_strides(out)
    if out_abi is not out:
        raise ValueError("out needs a contiguous head dimension and positive strides that are multiples of 8")
    if return_lse and lse is None:
        lse = torch.empty((B, N, S), dtype=torch.float32, device=q.device)
    p = make_params(B, N, S, d, q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                    lse.data_ptr() if return_lse else 0, softmax_scale, causal, window_left, window_right,
                    FA_DTYPE_BF16 if q.dtype == torch.bfloat16 else FA_DTYPE_F16, sched,
                    0 if alibi_slopes is None else alibi_slopes.data_ptr(), 0 if Nk == N else Nk,
                    q_st, k_st, v_st, o_st,
                    dropout_prob=dropout_prob, seed=seed, S_kv=0 if S_kv == S else S_kv, exact_first_rows=exact_first_rows)
    if splits == "auto":
        splits = lib().fa_fwd_suggest_splits(ctypes.byref(p))
    workspace = None
    if splits and splits > 1:
        p.split_num = int(splits)
        need = lib().fa_fwd_workspace_bytes(ctypes.byref(p))
        if need and not static_scratch:
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)   # stream-ordered: freed after the launch
            p.workspace, p.workspace_bytes = workspace.data_ptr(), need
    stream = torch.cuda.current_stream(q.device).cuda_stream
    entry = lib().fa_fwd_split_static if static_scratch else lib().fa_fwd
    st = entry(ctypes.byref(p), ctypes.c_void_p(stream))
    if st != FA_OK:
        raise FaError(st, lib().fa_last_device_error().decode() if st == FA_ERR_DEVICE else "")
    return (out, lse) if return_lse else out


def make_bwd_params(B, N, S, d, q_ptr=0, k_ptr=0, v_ptr=0, o_ptr=0, do_ptr=0, lse_ptr=0, dq_ptr=0, dk_ptr=0, dv_ptr=0,
                    softmax_scale=None, causal=False, window_left=-1, window_right=-1, dtype=FA_DTYPE_F16,
                    workspace_ptr=0, workspace_bytes=0, n_kv_heads=0, S_kv=0, alibi_ptr=0, strides=None, dropout_prob=0.0,
                    seed=0):
    """strides: dict name -> (batch, head, row) element strides for any of q, k, v, o, do, dq, dk, dv."""
    p = FaBwdParams()
    p.Q, p.K, p.V, p.O, p.dO, p.L = q_ptr, k_ptr, v_ptr, o_ptr, do_ptr, lse_ptr
    p.dQ, p.dK, p.dV = dq_ptr, dk_ptr, dv_ptr
    p.B, p.N, p.S, p.d = B, N, S, d
    p.softmax_scale = softmax_scale if softmax_scale is not None else (1.0 / math.sqrt(d) if d > 0 else 0.0)
    p.window_size_left, p.window_size_right = window_left, window_right
    p.dtype, p.is_causal = dtype, int(causal)
    p.workspace, p.workspace_bytes = workspace_ptr, workspace_bytes
    p.n_kv_heads, p.S_kv, p.alibi_slopes_ptr = n_kv_heads, S_kv, alibi_ptr
    p.dropout_prob, p.seed = dropout_prob, seed
    for name, st in (strides or {}).items():
        if st is not None:
            getattr(p, name + "_strides")[:] = list(st)
    return p


def flash_attention_backward(q, k, v, o, lse, do, softmax_scale=None, causal=False, window_left=-1, window_right=-1,
                             alibi_slopes=None, dropout_prob=0.0, seed=0, five_products="auto", poison_workspace=False,
                             workspace_limit=None):
    """dq, dk, dv = gradients of attention(q, k, v) given the gradient ``do`` of its output, on the GPU through
    fa_bwd().  o and lse are what flash_attention_forward returned for the same q, k, v, mask, slopes, dropout
    probability and seed.
    ``five_products``: True asks for the workspace that selects the five-product form (fa_bwd_fast_workspace_bytes:
    B*N*S*S elements more), False for the small one; "auto" takes, when the problem qualifies, the dS blocks of about
    2 GiB worth of heads (the form then runs over the heads in chunks, which measures no slower), at least
    fa_bwd_min_fast_workspace_bytes and at most ``workspace_limit`` bytes when that is given; when the device has no
    room for it, the least, and when not for that either, the small one.  ``poison_workspace`` (for tests) fills the workspace with
    NaN bit patterns first: the kernels must not read anything in it that they have not written.
    Shapes and strides as in flash_attention_forward (q, o, do [B, N, S, d]; k, v [B, Nk, S_kv, d]; lse
    [B, N, S] float32 contiguous); dq, dk, dv come back with the strides of q, k, v."""
    import torch
    if not all(t.is_cuda and t.dtype == q.dtype and t.dim() == 4 for t in (q, k, v, o, do)):
        raise ValueError("q, k, v, o, do must be 4-d GPU tensors of one dtype")
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("tensors must be float16 or bfloat16")
    if o.shape != q.shape or do.shape != q.shape or k.shape != v.shape or (q.shape[0], q.shape[3]) != (
            k.shape[0], k.shape[3]) or k.shape[1] == 0 or q.shape[1] % k.shape[1] != 0 or k.shape[2] == 0:
        raise ValueError("q, o, do must be [B, N, S, d], k and v [B, Nk, S_kv, d] with Nk dividing N")
    B, N, S, d = q.shape
    Nk, S_kv = k.shape[1], k.shape[2]
    if not (lse.is_cuda and lse.dtype == torch.float32 and lse.is_contiguous() and tuple(lse.shape) == (B, N, S)):
        raise ValueError("lse must be a contiguous float32 GPU tensor [B, N, S]")
    if alibi_slopes is not None and not (alibi_slopes.is_cuda and alibi_slopes.dtype == torch.float32
                                         and alibi_slopes.is_contiguous() and tuple(alibi_slopes.shape) == (N,)):
        raise ValueError("alibi_slopes must be a contiguous float32 GPU tensor of shape [N]")
    # inputs the ABI cannot address (zero strides of an expanded gradient, strides that are no multiple of 8)
    # are replaced by dense copies; the gradients keep the strides of q, k, v where the ABI can write those
    tensors, strides = {}, {}
    for n, t in dict(q=q, k=k, v=v, o=o, do=do).items():
        tensors[n], strides[n] = abi_strides(t)
    q, k, v, o, do = (tensors[n] for n in ("q", "k", "v", "o", "do"))
    for n, like in (("dq", q), ("dk", k), ("dv", v)):
        g = torch.empty_like(like)                    # keeps a dense or permuted layout
        g_abi, g_st = abi_strides(g)
        if g_abi is not g:
            g, g_st = torch.empty(like.shape, dtype=like.dtype, device=like.device), None
        tensors[n], strides[n] = g, g_st
    dq, dk, dv = tensors["dq"], tensors["dk"], tensors["dv"]
    p = make_bwd_params(B, N, S, d, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), do.data_ptr(),
                        lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), softmax_scale, causal,
                        window_left, window_right, FA_DTYPE_BF16 if q.dtype == torch.bfloat16 else FA_DTYPE_F16,
                        n_kv_heads=0 if Nk == N else Nk, S_kv=0 if S_kv == S else S_kv,
                        alibi_ptr=0 if alibi_slopes is None else alibi_slopes.data_ptr(), strides=strides,
                        dropout_prob=dropout_prob, seed=seed)
    small = lib().fa_bwd_workspace_bytes(ctypes.byref(p))
    fast = lib().fa_bwd_fast_workspace_bytes(ctypes.byref(p)) if five_products else 0
    sizes = [small]                       # tried from the back; the small workspace is what is left when nothing else fits
    if fast and five_products is True and workspace_limit is None:
        sizes.append(fast)
    elif fast:
        # "auto": whole chunks of eight K/V heads' dS blocks, about 2 GiB of them (chunks measure no slower than the
        # full size: B2 N32 S8192 D128 3.27 ms with 2.2 or 4.4 GB against 3.34 with 8.6), never fewer heads than the
        # library accepts and never more bytes than the limit; sizes that depend on the problem alone, so that
        # torch's allocator hands the same block back call after call (and no query of the device's free memory:
        # torch's memory statistics cost a millisecond per call, ten times a short problem's backward pass)
        least = lib().fa_bwd_min_fast_workspace_bytes(ctypes.byref(p))
        off = (small + 255) // 256 * 256
        kv_total = q.shape[0] * k.shape[1]
        per_head = (fast - off) // kv_total
        heads = max((least - off) // per_head, (2 << 30) // per_head // 8 * 8)
        limit = workspace_limit if workspace_limit is not None else fast
        if off + heads * per_head > limit:
            heads = (limit - off) // per_head // 8 * 8 if limit > off else 0
        want = fast if heads >= kv_total else off + heads * per_head
        if least <= limit and want > least:
            sizes.append(least)
        if heads > 0 and least <= want <= limit:
            sizes.append(want)
    workspace = None
    while workspace is None:              # stream-ordered: freed after the launch
        need = sizes.pop()
        try:
            workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
        except torch.cuda.OutOfMemoryError:
            if not sizes:
                raise
    if poison_workspace:
        workspace.fill_(0xff)
    p.workspace, p.workspace_bytes = workspace.data_ptr(), need
    st = lib().fa_bwd(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream(q.device).cuda_stream))
    if st != FA_OK:
        raise FaError(st, lib().fa_last_device_error().decode() if st == FA_ERR_DEVICE else "")
    return dq, dk, dv


_autograd_function = None


def flash_attention(q, k, v, softmax_scale=None, causal=False, window_left=-1, window_right=-1, alibi_slopes=None,
                    dropout_prob=0.0, seed=0):
    """Differentiable attention for PyTorch callers: fa_fwd in the forward pass, fa_bwd in the backward pass
    (which replays the dropout decisions from ``seed``; nothing but O and the logsumexp is saved).  Shapes and
    layouts as in flash_attention_forward.  Plumbing only: both passes are the library's kernels."""
    global _autograd_function
    import torch
    if _autograd_function is None:
        class _FlashAttention(torch.autograd.Function):
            @staticmethod
            def forward(ctx, q, k, v, opts):
                # exact products in every row: the logsumexp must be the one fa_bwd recomputes P from
                o, lse = flash_attention_forward(q, k, v, exact_first_rows=True, **opts)
                ctx.save_for_backward(q, k, v, o, lse)
                ctx.opts = opts
                return o

            @staticmethod
            def backward(ctx, do):
                q, k, v, o, lse = ctx.saved_tensors
                dq, dk, dv = flash_attention_backward(q, k, v, o, lse, do, **ctx.opts)
                return dq, dk, dv, None
        _autograd_function = _FlashAttention
    opts = dict(softmax_scale=softmax_scale, causal=causal, window_left=window_left, window_right=window_right,
                alibi_slopes=alibi_slopes, dropout_prob=dropout_prob, seed=seed)
    return _autograd_function.apply(q, k, v, opts)


def run_flash_attention(B, N, S, d, Q, K, V, O, L=None, M=None, Is_dropout=False, Is_causal=False, Is_local=False,
                        Has_alibi=False, window_size=0, alibi_slopes=None, dropout_prob=0.0, states=None):
    """The reference's entry point with its argument order (flash_forward.h:593-612); Q..L are torch
    tensors (or None) whose device pointers are passed through; returns the status code."""
    def ptr(t):
        return None if t is None else ctypes.c_void_p(t.data_ptr())
    return lib().run_flash_attention(B, N, S, d, ptr(Q), ptr(K), ptr(V), ptr(O), ptr(L), ptr(M), int(Is_dropout),
                                     int(Is_causal), int(Is_local), int(Has_alibi), int(window_size),
                                     ptr(alibi_slopes), float(dropout_prob), ptr(states))


def fill_normal(rows, d, dtype, seed, tensor, sigma=1.0, fraction=0.0, row_mult=1.0, nthreads=8):
    """numpy uint16 array [rows, d] of storage bits from the harness's seeded generator."""
    import numpy as np
    out = np.empty((rows, d), dtype=np.uint16)
    rc = host_lib().fa_fill_normal(out.ctypes.data, rows, d, dtype, seed, tensor, sigma, fraction, row_mult, nthreads)
    if rc != 0:
        raise ValueError("fa_fill_normal rejected its arguments")
    return out
