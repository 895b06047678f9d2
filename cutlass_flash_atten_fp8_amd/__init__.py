"""FP8 flash-attention forward for AMD MI355X (gfx950).

Host-side mirror of the reference's operator interface (weishengying/cutlass_flash_atten_fp8):

    from attention_cutlass_fp8 import flash_attention_v2_cutlass       # reference test.py:3
    o = flash_attention_v2_cutlass(q, k, v, is_causal, softmax_scale)[0]

`attention_cutlass_fp8` is the compiled PyTorch binding (csrc/attention_api.cpp); importing this package
registers it under that top-level name.  `flash_attention_v2_cutlass` below is the same operator driven
from Python through the C ABI of libfa8.so (include/fa8_api.h) with ctypes; both end in the same HIP
kernels.  There is no CPU or PyTorch fallback: if libfa8.so is missing, importing the operator raises.
"""
import ctypes
import importlib.util
import os
import sys
import sysconfig

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIBFA8_PATH = os.path.join(_PKG_DIR, "libfa8.so")
_EXT_NAME = "attention_cutlass_fp8"
EXT_PATH = os.path.join(_PKG_DIR, _EXT_NAME + sysconfig.get_config_var("EXT_SUFFIX"))

# codes of include/fa8_api.h
FA8_DTYPE_E4M3, FA8_DTYPE_E5M2 = 0, 1
FA8_OUT_FP16, FA8_OUT_E4M3, FA8_OUT_E5M2 = 0, 1, 2
FA8_V_ROWS, FA8_V_TRANSPOSED = 0, 1
FA8_CAUSAL_TOP_LEFT, FA8_CAUSAL_BOTTOM_RIGHT = 0, 1
FA8_SCHEDULE_AUTO, FA8_SCHEDULE_ROLLING, FA8_SCHEDULE_PIPELINED, FA8_SCHEDULE_DENSE = 0, 1, 2, 3
(FA8_QUERY_VERSION, FA8_QUERY_KV_BLOCK, FA8_QUERY_Q_BLOCK, FA8_QUERY_KV_ASCENDING, FA8_QUERY_THREADS,
 FA8_QUERY_PARAMS_SIZE) = range(6)
FA8_EXPORTS = ("fa8_fwd_validate", "fa8_fwd", "fa8_fwd_schedule", "fa8_query", "fa8_error_string")


class Fa8FwdParams(ctypes.Structure):
    """struct Fa8FwdParams of include/fa8_api.h."""
    _fields_ = [
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("o", ctypes.c_void_p),
        ("batch", ctypes.c_int32), ("heads", ctypes.c_int32), ("seqlen_q", ctypes.c_int32),
        ("seqlen_k", ctypes.c_int32), ("head_dim", ctypes.c_int32), ("is_causal", ctypes.c_int32),
        ("in_dtype", ctypes.c_int32), ("out_dtype", ctypes.c_int32), ("v_layout", ctypes.c_int32),
        ("softmax_scale", ctypes.c_float),
        ("q_batch_stride", ctypes.c_int64), ("q_head_stride", ctypes.c_int64), ("q_row_stride", ctypes.c_int64),
        ("k_batch_stride", ctypes.c_int64), ("k_head_stride", ctypes.c_int64), ("k_row_stride", ctypes.c_int64),
        ("v_batch_stride", ctypes.c_int64), ("v_head_stride", ctypes.c_int64), ("v_row_stride", ctypes.c_int64),
        ("o_batch_stride", ctypes.c_int64), ("o_head_stride", ctypes.c_int64), ("o_row_stride", ctypes.c_int64),
        ("lse", ctypes.c_void_p), ("lse_batch_stride", ctypes.c_int64), ("lse_head_stride", ctypes.c_int64),
        ("heads_k", ctypes.c_int32), ("causal_align", ctypes.c_int32),
        ("schedule", ctypes.c_int32), ("reserved0", ctypes.c_int32),
    ]


_lib = None


def lib():
    """The loaded libfa8.so with typed entry points.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIBFA8_PATH):
            raise ImportError(
                f"{LIBFA8_PATH} is missing: build it with `python -m cutlass_flash_atten_fp8_amd.build` "
                "(there is no CPU or PyTorch fallback for the attention kernels)")
        L = ctypes.CDLL(LIBFA8_PATH)
        L.fa8_fwd_validate.restype = ctypes.c_int
        L.fa8_fwd_validate.argtypes = [ctypes.POINTER(Fa8FwdParams)]
        L.fa8_fwd.restype = ctypes.c_int
        L.fa8_fwd.argtypes = [ctypes.POINTER(Fa8FwdParams), ctypes.c_void_p]
        L.fa8_fwd_schedule.restype = ctypes.c_int
        L.fa8_fwd_schedule.argtypes = [ctypes.POINTER(Fa8FwdParams)]
        L.fa8_query.restype = ctypes.c_int
        L.fa8_query.argtypes = [ctypes.c_int]
        L.fa8_error_string.restype = ctypes.c_char_p
        L.fa8_error_string.argtypes = [ctypes.c_int]
        _lib = L
    return _lib


def error_string(code):
    return lib().fa8_error_string(int(code)).decode()


def query(what):
    return int(lib().fa8_query(int(what)))


def load_extension():
    """Import the compiled binding and register it as the top-level module `attention_cutlass_fp8`."""
    if _EXT_NAME in sys.modules:
        return sys.modules[_EXT_NAME]
    if not os.path.exists(EXT_PATH):
        raise ImportError(f"{EXT_PATH} is missing: build it with `python -m cutlass_flash_atten_fp8_amd.build`")
    import torch  # noqa: F401  (the binding links against libtorch)
    spec = importlib.util.spec_from_file_location(_EXT_NAME, EXT_PATH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    sys.modules[_EXT_NAME] = mod
    return mod


def make_params(q, k, v, o, is_causal, softmax_scale, v_transposed=False, lse=None, causal_bottom_right=False,
                schedule=0):
    """Fill Fa8FwdParams from torch tensors (any device: only shapes, strides and pointers are read).
    k and v may have fewer heads than q (grouped-query attention); lse, if given, is a float32 [B,H,Nq] output."""
    import torch
    in_codes = {torch.float8_e4m3fn: FA8_DTYPE_E4M3, torch.float8_e5m2: FA8_DTYPE_E5M2}
    out_codes = {torch.float16: FA8_OUT_FP16, torch.float8_e4m3fn: FA8_OUT_E4M3, torch.float8_e5m2: FA8_OUT_E5M2}
    if q.dtype not in in_codes:
        raise RuntimeError(f"q must be torch.float8_e4m3fn or torch.float8_e5m2 (OCP fp8), got {q.dtype}")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError("q, k and v must have the same dtype")
    if o.dtype not in out_codes:
        raise RuntimeError("out_dtype must be torch.float16 or the fp8 type of the inputs")
    for name, t in (("q", q), ("k", k), ("v", v), ("o", o)):
        if t.dim() != 4:
            raise RuntimeError(f"{name} must be 4-dimensional [batch, heads, seqlen, head_dim], got {t.dim()} dims")
        if t.stride(3) != 1:
            raise RuntimeError(f"the last dimension of {name} must be contiguous")
    p = Fa8FwdParams()
    p.q, p.k, p.v, p.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
    p.batch, p.heads, p.seqlen_q, p.head_dim = q.shape
    p.seqlen_k = k.shape[2]
    p.is_causal = int(bool(is_causal))
    p.in_dtype = in_codes[q.dtype]
    p.out_dtype = out_codes[o.dtype]
    p.v_layout = FA8_V_TRANSPOSED if v_transposed else FA8_V_ROWS
    p.softmax_scale = float(softmax_scale)
    for name, t in (("q", q), ("k", k), ("v", v), ("o", o)):
        setattr(p, name + "_batch_stride", t.stride(0))
        setattr(p, name + "_head_stride", t.stride(1))
        setattr(p, name + "_row_stride", t.stride(2))
    p.heads_k = k.shape[1]
    p.causal_align = FA8_CAUSAL_BOTTOM_RIGHT if causal_bottom_right else FA8_CAUSAL_TOP_LEFT
    p.schedule = int(schedule)
    if lse is not None:
        if lse.dtype != torch.float32 or lse.dim() != 3 or lse.stride(2) != 1:
            raise RuntimeError("lse must be a float32 [batch, heads, seqlen_q] tensor with contiguous rows")
        p.lse, p.lse_batch_stride, p.lse_head_stride = lse.data_ptr(), lse.stride(0), lse.stride(1)
    return p


def flash_attention_v2_cutlass(q, k, v, is_causal, softmax_scale, *, v_transposed=False, out_dtype=None, return_lse=False,
                               causal_bottom_right=False, schedule=0):
    """The reference operator (reference csrc/flash_attention.cu:639-668) through the C ABI.

    q, k: fp8 [B,H,N,d] on the GPU; v: [B,H,N,d] (or [B,H,d,N] with v_transposed=True, as the reference
    requires of its caller, test.py:71).  Returns [O], O fp16 [B,H,N,d] (out_dtype=q.dtype gives the
    reference's fp8 O, stored in the input element type).  Runs on torch's current stream without synchronising.  Raises
    RuntimeError on bad arguments, like the reference's TORCH_CHECKs (include/attention_api.cuh:12-18).
    Beyond the reference: k/v may have fewer heads than q (grouped-query attention), return_lse=True returns
    [O, lse] with lse the float32 [B,H,Nq] log-sum-exp of the scaled logits, causal_bottom_right=True aligns the
    causal diagonal with the last key when seqlen_q != seqlen_k; schedule (FA8_SCHEDULE_*) is a performance hint that
    never changes the result.
    """
    import torch
    for name, t in (("q", q), ("k", k), ("v", v)):
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be a GPU tensor")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
        if t.dim() != 4:
            raise RuntimeError(f"{name} must be 4-dimensional [batch, heads, seqlen, head_dim], got {t.dim()} dims")
    B, H, Nq, D = q.shape
    Nk, Hk = k.shape[2], k.shape[1]
    if k.shape[0] != B or k.shape[3] != D:
        raise RuntimeError(f"k must be [{B}, heads_k, seqlen_k, {D}], got {tuple(k.shape)}")
    if Hk < 1 or H % Hk != 0:
        raise RuntimeError(f"the number of q heads ({H}) must be a multiple of the number of k/v heads ({Hk})")
    want_v = (B, Hk, D, Nk) if v_transposed else (B, Hk, Nk, D)
    if tuple(v.shape) != want_v:
        raise RuntimeError(f"v must be {list(want_v)}, got {tuple(v.shape)}")
    if k.device != q.device or v.device != q.device:
        raise RuntimeError("q, k and v must be on the same device")
    o = torch.empty((B, H, Nq, D), dtype=out_dtype or torch.float16, device=q.device)
    lse = torch.empty((B, H, Nq), dtype=torch.float32, device=q.device) if return_lse else None
    p = make_params(q, k, v, o, is_causal, softmax_scale, v_transposed, lse, causal_bottom_right, schedule)
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        rc = lib().fa8_fwd(ctypes.byref(p), ctypes.c_void_p(stream))
    if rc != 0:
        raise RuntimeError(f"flash_attention_v2_cutlass: {error_string(rc)} (code {rc})")
    return [o, lse] if return_lse else [o]


# Make `from attention_cutlass_fp8 import flash_attention_v2_cutlass` work once this package is imported
# (only when the binding has been built; the ctypes operator above does not need it).
if os.path.exists(EXT_PATH) and os.path.exists(LIBFA8_PATH):
    try:
        load_extension()
    except Exception as _e:  # pragma: no cover - reported on first explicit load_extension()
        _EXT_IMPORT_ERROR = _e
