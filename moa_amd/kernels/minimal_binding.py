"""The smallest binding of the C ABI that stands in for the reference's
``from flashinfer import moa_prefill, moa_decode`` (MoA/kernels/mixture_of_attention.py:22-30): ctypes,
pointers and sizes only.  Argument order follows the reference's call sites (:436-444, :466-473).  It is
what a maintainer of the reference would add next to that module; ``moa_amd.kernels.mixture_of_attention``
is the same binding with the checks, error classes and grouped-query handling the package needs.  The
library is looked up next to the package unless ``MOA_HIP_LIB`` names another build of it."""
import os
import ctypes, torch
_lib = ctypes.CDLL(os.environ.get("MOA_HIP_LIB", os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "libmoa_hip.so")))
_lib.moa_last_error.restype = ctypes.c_char_p
_lib.moa_decode_workspace_bytes.restype = ctypes.c_size_t
_lib.moa_decode_workspace_bytes.argtypes = [ctypes.c_int] * 4 + [ctypes.c_int64]
_I64x4 = ctypes.c_int64 * 4
_ws = {}

def _check(rc):
    if rc != 0:
        raise RuntimeError(_lib.moa_last_error().decode())

def moa_prefill(q, k, v, causal=True, num_global_blocks=None, num_band_blocks=None, kv_layout="HND",
                sm_scale=None):
    # q [B,N,H,D]; k, v [B,H,N,D]; block counts int64 [H] on the device; returns [B,N,H,D]
    B, N, H, D = q.shape
    o = torch.empty_like(q)
    bhnd = lambda t: _I64x4(t.stride(0), t.stride(2), t.stride(1), t.stride(3))   # strides in B,H,N,D order
    _check(_lib.moa_prefill_fwd(
        ctypes.c_void_p(q.data_ptr()), ctypes.c_void_p(k.data_ptr()), ctypes.c_void_p(v.data_ptr()),
        ctypes.c_void_p(o.data_ptr()), bhnd(q), _I64x4(*k.stride()), _I64x4(*v.stride()), bhnd(o),
        B, H, k.shape[1], N, D, ctypes.c_void_p(num_global_blocks.data_ptr()),
        ctypes.c_void_p(num_band_blocks.data_ptr()), ctypes.c_float(sm_scale or D ** -0.5),
        0 if q.dtype == torch.float16 else 1, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    return o

def moa_decode(q, k, v, head_start_index, head_valid_length, sm_scale):
    # q [B,1,H,D]; k, v [B,sumC,D]; index tensors int64 [B,H]; returns [B,1,H,D]
    B, _, H, D = q.shape
    sumC = k.shape[1]
    need = _lib.moa_decode_workspace_bytes(B, H, H, D, sumC)
    ws = _ws.get(q.device)
    if ws is None or ws.numel() < need:
        ws = _ws[q.device] = torch.empty(need, dtype=torch.uint8, device=q.device)
    o = torch.empty_like(q)
    _check(_lib.moa_decode_fwd(
        ctypes.c_void_p(q.contiguous().data_ptr()), ctypes.c_void_p(k.data_ptr()), ctypes.c_void_p(v.data_ptr()),
        ctypes.c_void_p(o.data_ptr()), ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(ws.numel()),
        ctypes.c_void_p(head_start_index.data_ptr()), ctypes.c_void_p(head_valid_length.data_ptr()),
        B, H, H, D, ctypes.c_int64(sumC), ctypes.c_float(sm_scale),
        0 if q.dtype == torch.float16 else 1, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    return o

CUDA_KERNEL_AVAILABLE = True
