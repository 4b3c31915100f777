"""ctypes binding of liblvx.so (the gfx950 kernels behind a C ABI, include/lvx.h).

There is no fallback: if the library is missing or a call is rejected the host
code raises.  PyTorch is used only to own device memory and the stream.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("LVX_LIB") or os.path.join(_HERE, "liblvx.so")

LVX_BF16 = 1
LVX_F16 = 2


class LvxError(RuntimeError):
    pass


class AttnShape(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("Hq", C.c_int32), ("Hkv", C.c_int32), ("D", C.c_int32),
        ("Lq", C.c_int32), ("Lkv", C.c_int32), ("dtype", C.c_int32), ("scale", C.c_float),
        ("kv_len", C.c_void_p), ("kv_start", C.c_void_p), ("kv_end", C.c_void_p),
        ("bias", C.c_void_p), ("bias_stride_b", C.c_int64), ("bias_stride_h", C.c_int64), ("bias_stride_r", C.c_int64),
    ]


class Tensor4(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("stride_b", C.c_int64), ("stride_h", C.c_int64), ("stride_s", C.c_int64)]


# every symbol include/lvx.h declares: name -> (restype, argtypes)
_P = C.c_void_p
_SHAPE = C.POINTER(AttnShape)
_T = C.POINTER(Tensor4)
SYMBOLS = {
    "lvx_version": (C.c_int, []),
    "lvx_strerror": (C.c_char_p, [C.c_int]),
    "lvx_fwd_workspace_bytes": (C.c_size_t, [_SHAPE, C.c_int32, C.c_int32]),
    "lvx_fwd": (C.c_int, [_SHAPE, _T, _T, _T, _T, _P, C.c_int32, C.c_int32, C.c_int32, _P, C.c_size_t, _P]),
    "lvx_fwd_acc": (C.c_int, [_SHAPE, _T, _T, _T, _T, _P, _T, _P, C.c_int32, C.c_int32, C.c_int32, _P, C.c_size_t, _P]),
    "lvx_fwd_noalloc": (C.c_int, [_SHAPE, _T, _T, _T, _T, _P, C.c_int32, C.c_int32, C.c_int32, _P]),
    "lvx_noalloc_scratch_bytes": (C.c_size_t, []),
    "lvx_merge": (C.c_int, [_SHAPE, _T, _P, _T, _P, C.c_int32, C.c_int32, _P]),
    "lvx_bias_hull": (C.c_int, [_SHAPE, _P, _P, _P]),
    "lvx_bias_is_interval": (C.c_int, [_SHAPE, _P, _P, _P, _P]),
    "lvx_bwd_preprocess": (C.c_int, [_SHAPE, _T, _T, _P, C.c_int32, C.c_int32, _P]),
    "lvx_bwd": (C.c_int, [_SHAPE, _T, _T, _T, _T, _P, _P, _T, _T, _T, C.c_int32, C.c_int32, C.c_int32,
                          _P, C.c_size_t, _P]),
    "lvx_bwd_workspace_bytes": (C.c_size_t, [_SHAPE, C.c_int32]),
    "lvx_cast_f32": (C.c_int, [_P, _T, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, _P]),
    "lvx_kv_proj": (C.c_int, [_P, C.c_int64, _P, _P, C.c_int64, C.c_int32, _P, _P, C.c_int64,
                              C.c_int32, C.c_int32, C.c_int32, C.c_int32, _P]),
    "lvx_kv_proj_norm": (C.c_int, [_P, C.c_int64, _P, _P, C.c_int64, C.c_int32, _P, _P, C.c_int64,
                                   C.c_int32, C.c_int32, C.c_int32, _P, C.c_float, _P, _P, C.c_int32, _P]),
    "lvx_k_norm_bwd": (C.c_int, [_P, C.c_int64, _P, C.c_int64, _P, _P, _P, C.c_int64, _P,
                                 C.c_int32, C.c_int32, C.c_int32, _P]),
    "lvx_dx_vis": (C.c_int, [_P, _P, C.c_int64, _P, _P, C.c_int64, C.c_int32, _P, C.c_int64,
                             C.c_int32, C.c_int32, C.c_int32, C.c_int32, _P]),
    "lvx_dw_kv": (C.c_int, [_P, C.c_int64, _P, _P, C.c_int64, _P, _P, C.c_int64, C.c_int32,
                            C.c_int32, C.c_int32, C.c_int32, C.c_int32, _P]),
}

_lib: Optional[C.CDLL] = None


def load() -> C.CDLL:
    """dlopen liblvx.so and type every entry point.  Raises if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LvxError(
            f"{LIB_PATH} is missing: the HIP kernels are not built. "
            "Run `python lv-xattn_amd/build.py` (needs hipcc); there is no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().lvx_strerror(rc).decode()
        raise LvxError(f"{what} failed: {msg} (code {rc})")


def stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def t4(t: torch.Tensor) -> Tensor4:
    """[B, H, S, D] tensor (any strides, unit last stride) -> lvx_tensor."""
    if t.dim() != 4 or t.stride(3) != 1:
        raise LvxError(f"expected a 4-d tensor with unit last stride, got shape {tuple(t.shape)} "
                       f"strides {t.stride()}")
    return Tensor4(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()
