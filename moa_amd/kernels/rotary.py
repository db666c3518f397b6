"""Rotary position embedding on the GPU, for the step in front of the attention path.

Mirrors ``apply_rotary_pos_emb`` of transformers 4.44.2 (the reference's pinned
dependency, requirements.txt:8) as the reference's caller uses it
(MoA/models/llama/modeling_llama.py:252): same arguments, same result bits.
"""
from typing import Optional, Tuple

import torch
from torch import Tensor

from .. import _lib


def _bhnd_strides(t: Tensor):
    return _lib.i64_array(t.stride())


def _cos_sin_strides(cos: Tensor, sin: Tensor, B: int, N: int, D: int):
    assert cos.shape == sin.shape and cos.dim() == 3, "cos and sin must be [batch, seq_len, head_dim]"
    assert cos.shape[0] in (1, B) and cos.shape[1] == N and cos.shape[2] == D, (
        f"cos/sin shape {tuple(cos.shape)} does not match batch {B}, seq_len {N}, head_dim {D}")
    if cos.stride(-1) != 1:
        cos = cos.contiguous()
    if sin.stride() != cos.stride():
        sin = sin.contiguous()
        cos = cos.contiguous()
    sb = 0 if cos.shape[0] == 1 else cos.stride(0)
    return cos, sin, _lib.i64_array([sb, cos.stride(1), 1])


def apply_rotary_pos_emb(q: Optional[Tensor], k: Optional[Tensor], cos: Tensor, sin: Tensor,
                         position_ids=None, unsqueeze_dim: int = 1) -> Tuple[Optional[Tensor], Optional[Tensor]]:
    """``q_embed = q*cos + rotate_half(q)*sin`` and the same for ``k``.

    q ``[batch, q_heads, seq_len, head_dim]``, k ``[batch, kv_heads, seq_len, head_dim]`` (any strides
    with a contiguous last dim), cos/sin ``[batch or 1, seq_len, head_dim]`` in the same dtype.
    Returns new tensors laid out like their inputs when those are dense (a transposed view of a
    ``[batch, seq_len, heads, head_dim]`` projection gives a result with the same strides, as torch's
    elementwise evaluation of the formula does: both sides of the kernel then stream through memory),
    contiguous otherwise.  Only ``unsqueeze_dim=1`` (heads in dim 1) is covered.
    """
    if unsqueeze_dim != 1:
        raise NotImplementedError("apply_rotary_pos_emb: only unsqueeze_dim=1 ([batch, heads, seq, dim]) is covered")
    ref = q if q is not None else k
    assert ref is not None, "q and k are both None"
    if ref.device.type != "cuda":
        raise _lib.MoaKernelError("apply_rotary_pos_emb: tensors must live on the GPU; moa_amd has no CPU path")
    B, _, N, D = ref.shape
    assert cos.dtype == ref.dtype and sin.dtype == ref.dtype, "cos/sin must have the dtype of q/k"
    cos, sin, css = _cos_sin_strides(cos, sin, B, N, D)
    outs = []
    for t in (q, k):
        if t is None:
            outs.append(None)
            continue
        assert t.dim() == 4 and t.shape[0] == B and t.shape[2] == N and t.shape[3] == D and t.dtype == ref.dtype
        outs.append(torch.empty_like(t))   # keeps the strides of a dense input, contiguous otherwise
    qi = q if q is None or q.stride(-1) == 1 else q.contiguous()
    ki = k if k is None or k.stride(-1) == 1 else k.contiguous()
    lib = _lib.load()
    rc = lib.moa_rope_fwd(
        _lib.ptr(qi), _lib.ptr(ki), _lib.ptr(outs[0]), _lib.ptr(outs[1]),
        None if qi is None else _bhnd_strides(qi), None if ki is None else _bhnd_strides(ki),
        None if qi is None else _bhnd_strides(outs[0]), None if ki is None else _bhnd_strides(outs[1]),
        cos.data_ptr(), sin.data_ptr(), css, B, 0 if qi is None else qi.shape[1], 0 if ki is None else ki.shape[1],
        N, D, _lib.dtype_code(ref.dtype), _lib.current_stream_ptr(ref.device))
    _lib.check(rc)
    return outs[0], outs[1]
