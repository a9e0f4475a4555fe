"""ctypes binding of libtpa_gfx950.so (declared in include/tpa_abi.h).

PyTorch is used only as the owner of device memory and streams; every kernel is reached
through the C ABI.  There is no CPU fallback: a missing library raises.
"""

from __future__ import annotations

import ctypes
import os
import threading

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("TPA_GFX950_LIB") or os.path.join(os.path.dirname(_PKG_DIR), "lib", "libtpa_gfx950.so")

TPA_DTYPE_F32 = 0
TPA_DTYPE_BF16 = 1

KERNEL_AUTO = 0
KERNEL_GENERIC = 1
KERNEL_MFMA = 2

ABI_VERSION = 9


class TpaFactor(ctypes.Structure):
    _fields_ = [
        ("ptr", ctypes.c_void_p),
        ("stride_b", ctypes.c_int64),
        ("stride_l", ctypes.c_int64),
        ("stride_r", ctypes.c_int64),
    ]


class TpaFwdArgs(ctypes.Structure):
    _fields_ = [
        ("qa", TpaFactor),
        ("qb", TpaFactor),
        ("ka", TpaFactor),
        ("kb", TpaFactor),
        ("va", TpaFactor),
        ("vb", TpaFactor),
        ("q_segment_ids", ctypes.c_void_p),
        ("kv_segment_ids", ctypes.c_void_p),
        ("o", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("B", ctypes.c_int32),
        ("lq", ctypes.c_int32),
        ("lk", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("dk", ctypes.c_int32),
        ("dv", ctypes.c_int32),
        ("rq", ctypes.c_int32),
        ("rk", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("sm_scale", ctypes.c_float),
        ("causal", ctypes.c_int32),
        ("kernel", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
        ("num_splits", ctypes.c_int32),
        ("kv_lengths", ctypes.c_void_p),
        ("page_table", ctypes.c_void_p),
        ("page_size", ctypes.c_int32),
        ("pages_per_seq", ctypes.c_int32),
        ("causal_offset", ctypes.c_int32),
        ("nomat", ctypes.c_int32),
    ]


class MhaFwdArgs(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("bias", ctypes.c_void_p),
        ("o", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("B", ctypes.c_int32),
        ("lq", ctypes.c_int32),
        ("lk", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("dk", ctypes.c_int32),
        ("dv", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("sm_scale", ctypes.c_float),
        ("causal", ctypes.c_int32),
        ("kernel", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
        ("num_splits", ctypes.c_int32),
    ]


class TpaGrad(ctypes.Structure):
    _fields_ = TpaFactor._fields_


class TpaBwdArgs(ctypes.Structure):
    _fields_ = [
        ("qa", TpaFactor),
        ("qb", TpaFactor),
        ("ka", TpaFactor),
        ("kb", TpaFactor),
        ("va", TpaFactor),
        ("vb", TpaFactor),
        ("q_segment_ids", ctypes.c_void_p),
        ("kv_segment_ids", ctypes.c_void_p),
        ("o", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("d_o", ctypes.c_void_p),
        ("dqa", TpaGrad),
        ("dqb", TpaGrad),
        ("dka", TpaGrad),
        ("dkb", TpaGrad),
        ("dva", TpaGrad),
        ("dvb", TpaGrad),
        ("B", ctypes.c_int32),
        ("lq", ctypes.c_int32),
        ("lk", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("dk", ctypes.c_int32),
        ("dv", ctypes.c_int32),
        ("rq", ctypes.c_int32),
        ("rk", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("sm_scale", ctypes.c_float),
        ("causal", ctypes.c_int32),
        ("kernel", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
        ("causal_offset", ctypes.c_int32),
    ]


class MhaBwdArgs(ctypes.Structure):
    _fields_ = [
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("bias", ctypes.c_void_p),
        ("o", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("d_o", ctypes.c_void_p),
        ("dq", ctypes.c_void_p),
        ("dk_out", ctypes.c_void_p),
        ("dv_out", ctypes.c_void_p),
        ("B", ctypes.c_int32),
        ("lq", ctypes.c_int32),
        ("lk", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("dk", ctypes.c_int32),
        ("dv", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("sm_scale", ctypes.c_float),
        ("causal", ctypes.c_int32),
        ("kernel", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
    ]


class TpaAppendArgs(ctypes.Structure):
    _fields_ = [
        ("x", ctypes.c_void_p),
        ("w", ctypes.c_void_p),
        ("rope_cos", ctypes.c_void_p),
        ("rope_sin", ctypes.c_void_p),
        ("positions", ctypes.c_void_p),
        ("kv_lengths", ctypes.c_void_p),
        ("new_kv_lengths", ctypes.c_void_p),
        ("qa", TpaFactor),
        ("qb", TpaFactor),
        ("ka", TpaFactor),
        ("kb", TpaFactor),
        ("va", TpaFactor),
        ("vb", TpaFactor),
        ("page_table", ctypes.c_void_p),
        ("page_size", ctypes.c_int32),
        ("pages_per_seq", ctypes.c_int32),
        ("B", ctypes.c_int32),
        ("n", ctypes.c_int32),
        ("d_model", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("rq", ctypes.c_int32),
        ("rk", ctypes.c_int32),
        ("cache_len", ctypes.c_int32),
        ("rope_len", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("kernel", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
    ]


class TpaError(RuntimeError):
    """A non-zero return code of the C ABI."""

    def __init__(self, func: str, code: int, text: str):
        super().__init__(f"{func} failed with code {code}: {text}")
        self.code = code


_lib = None
_lib_lock = threading.Lock()


def load_library(path: str | None = None) -> ctypes.CDLL:
    """Load libtpa_gfx950.so once and declare its prototypes.  Raises if it is not built."""
    global _lib
    with _lib_lock:
        if _lib is not None and path is None:
            return _lib
        p = path or LIB_PATH
        if not os.path.exists(p):
            raise RuntimeError(
                f"{p} is not built: run `make -C {os.path.join(os.path.dirname(_PKG_DIR), 'csrc')}` "
                "(there is no fallback implementation)"
            )
        lib = ctypes.CDLL(p)
        lib.tpa_abi_version.restype = ctypes.c_int
        lib.tpa_abi_version.argtypes = []
        lib.tpa_strerror.restype = ctypes.c_char_p
        lib.tpa_strerror.argtypes = [ctypes.c_int]
        for name in ("tpa_fwd", "tpa_decode", "tpa_decode_noalloc"):
            fn = getattr(lib, name)
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.POINTER(TpaFwdArgs), ctypes.c_void_p]
        lib.mha_fwd.restype = ctypes.c_int
        lib.mha_fwd.argtypes = [ctypes.POINTER(MhaFwdArgs), ctypes.c_void_p]
        lib.tpa_cache_append.restype = ctypes.c_int
        lib.tpa_cache_append.argtypes = [ctypes.POINTER(TpaAppendArgs), ctypes.c_void_p]
        lib.tpa_cache_append_workspace_bytes.restype = ctypes.c_size_t
        lib.tpa_cache_append_workspace_bytes.argtypes = [ctypes.c_int32] * 8
        lib.tpa_decode_workspace_bytes.restype = ctypes.c_size_t
        lib.tpa_decode_workspace_bytes.argtypes = [ctypes.c_int32] * 6
        lib.tpa_decode_default_splits.restype = ctypes.c_int32
        lib.tpa_decode_default_splits.argtypes = [ctypes.c_int32] * 4
        lib.mha_fwd_workspace_bytes.restype = ctypes.c_size_t
        lib.mha_fwd_workspace_bytes.argtypes = [ctypes.c_int32] * 6
        lib.tpa_fwd_workspace_bytes.restype = ctypes.c_size_t
        lib.tpa_fwd_workspace_bytes.argtypes = [ctypes.c_int32] * 8
        lib.tpa_fwd_nomat_workspace_bytes.restype = ctypes.c_size_t
        lib.tpa_fwd_nomat_workspace_bytes.argtypes = [ctypes.c_int32] * 8
        lib.tpa_bwd.restype = ctypes.c_int
        lib.tpa_bwd.argtypes = [ctypes.POINTER(TpaBwdArgs), ctypes.c_void_p]
        lib.mha_bwd.restype = ctypes.c_int
        lib.mha_bwd.argtypes = [ctypes.POINTER(MhaBwdArgs), ctypes.c_void_p]
        lib.tpa_bwd_workspace_bytes.restype = ctypes.c_size_t
        lib.tpa_bwd_workspace_bytes.argtypes = [ctypes.c_int32] * 6
        lib.mha_bwd_workspace_bytes.restype = ctypes.c_size_t
        lib.mha_bwd_workspace_bytes.argtypes = [ctypes.c_int32] * 7
        if lib.tpa_abi_version() != ABI_VERSION:
            raise RuntimeError(f"{p}: ABI version {lib.tpa_abi_version()} != {ABI_VERSION}")
        if path is None:
            _lib = lib
        return lib


def check(func: str, code: int) -> None:
    if code != 0:
        raise TpaError(func, code, load_library().tpa_strerror(code).decode())


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return TPA_DTYPE_F32
    if dtype == torch.bfloat16:
        return TPA_DTYPE_BF16
    raise TypeError(f"unsupported dtype {dtype}: the kernels take float32 or bfloat16")


def factor(t: torch.Tensor) -> TpaFactor:
    """A [b, l, r, x] tensor (or a view of one) whose last dimension is contiguous."""
    if t.dim() != 4:
        raise ValueError(f"factor arrays are 4-D [b, l, r, x], got shape {tuple(t.shape)}")
    if t.shape[-1] > 1 and t.stride(-1) != 1:
        raise ValueError("the last dimension of a factor array must be contiguous")
    return TpaFactor(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def grad(t: torch.Tensor) -> TpaGrad:
    """A float32 [b, l, r, x] tensor (or a view of one) that a gradient is written into."""
    if t.dtype != torch.float32:
        raise TypeError("gradient arrays are float32")
    f = factor(t)
    return TpaGrad(f.ptr, f.stride_b, f.stride_l, f.stride_r)


def current_stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream
