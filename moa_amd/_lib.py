"""ctypes binding of libmoa_hip.so (declared in include/moa_hip.h).

There is no fallback: if the library is missing or does not load, every
operator of this package raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
from typing import Optional, Sequence

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmoa_hip.so")

MOA_OK = 0
MOA_ERR_ARG = -1
MOA_ERR_UNSUPPORTED = -2
MOA_ERR_LAUNCH = -3
MOA_ERR_WORKSPACE = -4

MOA_DTYPE_F16 = 0
MOA_DTYPE_BF16 = 1
MOA_DTYPE_F32 = 2

MOA_DECODE_NOALLOC_MAX_BYTES = 32 << 20

ABI_VERSION = 1

# name -> (restype, argtypes); must list every symbol include/moa_hip.h declares
_I64P = POINTER(c_int64)
SIGNATURES = {
    "moa_abi_version": (c_int, []),
    "moa_last_error": (c_char_p, []),
    "moa_prefill_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, _I64P, _I64P, _I64P, _I64P,
                                c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_int,
                                c_void_p]),
    "moa_decode_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int64]),
    "moa_decode_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p,
                               c_void_p, c_int, c_int, c_int, c_int, c_int64, c_float, c_int, c_void_p]),
    "moa_decode_fwd_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                       c_int, c_int, c_int64, c_float, c_int, c_void_p]),
    "moa_cache_append": (c_int, [c_void_p, c_void_p, _I64P, _I64P, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int,
                                 c_int, c_int64, c_int, c_void_p]),
    "moa_cache_prefill_workspace_bytes": (c_size_t, [c_int, c_int]),
    "moa_cache_prefill_insert": (c_int, [c_void_p, c_void_p, _I64P, _I64P, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                         c_void_p, c_size_t, c_int64, c_int, c_int, c_int, c_int, c_int64,
                                         c_int64, c_int, c_void_p]),
    "moa_rope_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, _I64P, _I64P, _I64P, _I64P, c_void_p,
                             c_void_p, _I64P, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "moa_rope_cache_append": (c_int, [c_void_p, c_void_p, c_void_p, _I64P, _I64P, _I64P, c_void_p, c_void_p,
                                      c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int,
                                      c_int, c_int64, c_int, c_void_p]),
}

_lib: Optional[ctypes.CDLL] = None


class MoaKernelError(RuntimeError):
    """The HIP library is missing, or a launch failed."""


def load() -> ctypes.CDLL:
    """Loads the library once; raises MoaKernelError when it cannot."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MoaKernelError(
            f"{LIB_PATH} is not built. Run `python -m moa_amd.build` (needs hipcc). "
            "moa_amd has no CPU or PyTorch fallback for its kernels.")
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as e:  # pragma: no cover - depends on the machine
        raise MoaKernelError(f"cannot load {LIB_PATH}: {e}") from e
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise MoaKernelError(f"{LIB_PATH} does not export {name}; rebuild it") from e
        fn.restype = res
        fn.argtypes = args
    v = lib.moa_abi_version()
    if v != ABI_VERSION:
        raise MoaKernelError(f"{LIB_PATH} has ABI version {v}, this package expects {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


def last_error() -> str:
    return load().moa_last_error().decode("utf-8", "replace")


def check(rc: int, assertion_for_arg: bool = True) -> None:
    """Maps a return code to the exception class the reference raises for the
    same condition: AssertionError for shape/dtype problems
    (MoA/kernels/mixture_of_attention.py:216,227,316), NotImplementedError for
    paths that are not covered (:478-479,486-487)."""
    if rc == MOA_OK:
        return
    msg = last_error()
    if rc == MOA_ERR_ARG and assertion_for_arg:
        raise AssertionError(msg)
    if rc == MOA_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise MoaKernelError(f"libmoa_hip error {rc}: {msg}")


def i64_array(values: Sequence[int]):
    return (c_int64 * len(values))(*[int(v) for v in values])


def dtype_code(torch_dtype) -> int:
    import torch

    if torch_dtype == torch.float16:
        return MOA_DTYPE_F16
    if torch_dtype == torch.bfloat16:
        return MOA_DTYPE_BF16
    if torch_dtype == torch.float32:
        return MOA_DTYPE_F32
    raise AssertionError(f"unsupported dtype {torch_dtype}")


def current_stream_ptr(device) -> int:
    """The raw HIP stream torch is currently using on ``device`` (through torch's internal accessor
    when it exists: the public ``torch.cuda.current_stream`` costs several microseconds per call)."""
    import torch

    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None:
        return raw(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


def ptr(t) -> Optional[int]:
    return None if t is None else t.data_ptr()
