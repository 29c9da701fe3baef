"""ctypes binding of libbgtq.so (the C ABI declared in include/bgtq.h).

Thin by design: torch tensors go in as raw device pointers plus element
strides, the current HIP stream is passed along, and a non-zero return code
raises.  There is no fallback: if the library is missing or was built for
another plan layout the import of any device path fails loudly.
"""
import ctypes
import os

import torch

from . import plan as _plan
from .build import LIB_PATH

_lib = None

c_i = ctypes.c_int
c_i64 = ctypes.c_int64
c_p = ctypes.c_void_p
c_f = ctypes.c_float

_SIGNATURES = {
    "bgtq_plan_sizeof": (ctypes.c_size_t, []),
    "bgtq_abi_version": (c_i, []),
    "bgtq_decode_kernel_revision": (c_i, []),
    "bgtq_strerror": (ctypes.c_char_p, [c_i]),
    "bgtq_encode_k": (c_i, [c_p, c_p, c_i64, c_i64, c_i64, c_i, c_i, c_i,
                            c_p, c_i64, c_i64, c_i64, c_i,
                            c_p, c_i64, c_i64, c_i64, c_i,
                            c_p, c_i, c_i, c_i, c_i, c_p]),
    "bgtq_encode_v": (c_i, [c_p, c_p, c_i64, c_i64, c_i64, c_i, c_i, c_i,
                            c_p, c_i64, c_i64, c_i64, c_i,
                            c_p, c_i64, c_i64, c_i64,
                            c_p, c_i, c_i, c_i, c_p]),
    "bgtq_compress_k_codes": (c_i, [c_p, c_p, c_i64, c_p, c_p, c_i, c_i, c_i, c_p]),
    "bgtq_compress_v_codes": (c_i, [c_p, c_p, c_i64, c_p, c_p, c_p]),
    "bgtq_rotate_q": (c_i, [c_p, c_p, c_i64, c_i64, c_p, c_i64, c_i64, c_i, c_i, c_i, c_p]),
    "bgtq_decode_prepare": (c_i, [c_p, c_p, c_i64, c_i64, c_i64, c_p, c_i64, c_i64, c_i64, c_i, c_i, c_i,
                                  c_p, c_i64, c_i64, c_i64, c_i,
                                  c_p, c_i64, c_i64, c_i64, c_i,
                                  c_p, c_i64, c_i64, c_i64, c_i,
                                  c_p, c_i64, c_i64, c_i64,
                                  c_p, c_i, c_i, c_i, c_i, c_i,
                                  c_p, c_i64, c_i64, c_p, c_i64, c_i64, c_i, c_p]),
    "bgtq_set_decode_path": (c_i, [c_i]),
    "bgtq_workspace_bytes": (ctypes.c_size_t, [c_i, c_i, c_i]),
    "bgtq_default_splits": (c_i, [c_i, c_i, c_i]),
    "bgtq_decode_attn": (c_i, [c_p, c_p, c_i64, c_i64,
                               c_p, c_i64, c_i64, c_i64, c_i,
                               c_p, c_i64, c_i64, c_i64,
                               c_p, c_i64, c_i64, c_i64, c_i,
                               c_p, c_i64, c_i64, c_i64,
                               c_p, c_i, c_i, c_i, c_i, c_i,
                               c_p, c_p, c_i, c_i, c_f, c_p]),
    "bgtq_decode_attend_static": (c_i, [c_p, c_p, c_i64, c_i64,
                                        c_p, c_i64, c_i64, c_i64, c_i,
                                        c_p, c_i64, c_i64, c_i64,
                                        c_p, c_i64, c_i64, c_i64, c_i,
                                        c_p, c_i64, c_i64, c_i64,
                                        c_p, c_i, c_i, c_i, c_i, c_i,
                                        c_i, c_i, c_f, c_i, c_p, c_i64, c_i64, c_p, c_p]),
    "bgtq_last_decode_path": (c_i, []),
    "bgtq_window_attn": (c_i, [c_p, c_i64, c_i64, c_p, c_p, c_i64, c_i64, c_i64, c_p, c_i,
                               c_i, c_i, c_i, c_f, c_p, c_p, c_p]),
    "bgtq_window_swap": (c_i, [c_p, c_p, c_i64, c_i64, c_i64, c_p, c_p, c_i64, c_i64, c_p, c_i, c_i, c_i,
                               c_p, c_p, c_p]),
    "bgtq_dequant_kv": (c_i, [c_p,
                              c_p, c_i64, c_i64, c_i64, c_i,
                              c_p, c_i64, c_i64, c_i64,
                              c_p, c_i64, c_i64, c_i64, c_i,
                              c_p, c_i64, c_i64, c_i64,
                              c_i, c_i, c_i, c_i, c_i,
                              c_p, c_i64, c_i64, c_i64,
                              c_p, c_i64, c_i64, c_i64, c_p]),
    "bgtq_prefill_attn": (c_i, [c_p,
                                c_p, c_i64, c_i64, c_i64,
                                c_p, c_i64, c_i64, c_i64, c_i,
                                c_p, c_i64, c_i64, c_i64,
                                c_p, c_i64, c_i64, c_i64, c_i,
                                c_p, c_i64, c_i64, c_i64,
                                c_i, c_i, c_i, c_i, c_i, c_i, c_i,
                                c_i, c_i, ctypes.c_float, c_i,
                                c_p, c_i64, c_i64, c_i64, c_p]),
    "bgtq_lse_reduce": (c_i, [c_p, c_p, c_p, c_i, c_p, c_p, c_i,
                              c_i, c_i, c_i, c_i, c_p, c_i64, c_i64, c_p, c_p]),
}


class BgtqError(RuntimeError):
    pass


def lib():
    """Load (once) and return the ctypes handle; raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise BgtqError(
            f"{LIB_PATH} is missing: build it with `python -m blockgtq_amd.build` "
            "(there is no CPU or eager fallback for the packed-KV path)")
    handle = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(handle, name)
        fn.restype = res
        fn.argtypes = args
    if handle.bgtq_plan_sizeof() != _plan.PLAN_DTYPE.itemsize:
        raise BgtqError(
            f"plan layout mismatch: library {handle.bgtq_plan_sizeof()} bytes, "
            f"host mirror {_plan.PLAN_DTYPE.itemsize} bytes")
    _lib = handle
    return _lib


def exported_symbols():
    """Names every build of the library must export (mirrors include/bgtq.h)."""
    return sorted(_SIGNATURES)


def check(code: int, what: str):
    if code != 0:
        msg = lib().bgtq_strerror(code).decode()
        raise BgtqError(f"{what} failed: {msg} (code {code})")


def ptr(t):
    """Device pointer of a tensor (or None)."""
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def stream_ptr(device=None):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def require_cuda(t: torch.Tensor, name: str):
    if not t.is_cuda:
        raise BgtqError(f"{name} must live on the GPU; the packed-KV path has no CPU fallback")
