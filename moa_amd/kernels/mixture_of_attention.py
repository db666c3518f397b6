"""Mixture of Sparse Attention -- operator interface.

Same surface as the reference's MoA/kernels/mixture_of_attention.py:
``mixture_of_sparse_attention`` (:358-487) dispatches between sparse prefill
and sparse decode; ``moa_prefill`` / ``moa_decode`` take the place of the two
ops the reference imports from its external CUDA package (:22-30, call sites
:435-444 and :465-473).  Here both run hand-written gfx950 kernels from
libmoa_hip.so; there is no Triton and no CPU path.
"""
from __future__ import annotations

import warnings
from typing import Dict, Optional, Tuple

import torch
import torch.nn.functional as F
from torch import LongTensor, Tensor

from moa_amd import _lib

BLOCK_M = 64
BLOCK_N = 64

_workspaces: Dict[Tuple[int, int, str], Tensor] = {}


def _workspace(device: torch.device, nbytes: int, tag: str, stream: int) -> Tensor:
    """A per-(device, stream) scratch buffer that only ever grows, so steady
    state calls allocate nothing."""
    key = (device.index or 0, stream, tag)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def _require_gpu(t: Tensor, who: str) -> None:
    if not t.is_cuda:
        raise _lib.MoaKernelError(
            f"{who}: tensors must live on the GPU; moa_amd has no CPU path for its kernels")


def _as_i64(t: Tensor, device: torch.device) -> Tensor:
    if t.dtype != torch.int64 or t.device != device or not t.is_contiguous():
        t = t.to(device=device, dtype=torch.int64).contiguous()
    return t


def moa_prefill(
    q: Tensor,
    k: Tensor,
    v: Tensor,
    causal: bool = True,
    num_global_blocks: LongTensor = None,
    num_band_blocks: LongTensor = None,
    kv_layout: str = "HND",
    sm_scale: Optional[float] = None,
) -> Tensor:
    """Block-sparse causal prefill.

    q ``[B, N, Hq, D]`` (any strides with a unit D stride), k, v ``[B, Hkv, N, D]``
    (``kv_layout="HND"``), ``num_global_blocks`` / ``num_band_blocks`` int64
    ``[Hkv]`` block counts.  Returns ``[B, N, Hq, D]`` contiguous.  Argument
    meaning follows the call at MoA/kernels/mixture_of_attention.py:435-444.
    """
    assert causal, "only causal attention is defined for MoA prefill"
    assert kv_layout == "HND", "k and v are expected as [B, H, N, D]"
    _require_gpu(q, "moa_prefill")
    assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4
    B, N, Hq, D = q.shape
    Hkv = k.shape[1]
    assert k.shape[0] == B and v.shape[0] == B and v.shape[1] == Hkv
    assert k.shape[-1] == D and v.shape[-1] == D, "q, k, v must share head_dim"
    assert k.shape[2] == N and v.shape[2] == N, "prefill expects as many keys as queries"
    assert q.dtype in (torch.float16, torch.bfloat16), "moa prefill runs in fp16 or bf16"
    assert k.dtype == q.dtype and v.dtype == q.dtype
    assert Hq % Hkv == 0
    assert num_global_blocks is not None and num_band_blocks is not None
    assert num_global_blocks.numel() == Hkv and num_band_blocks.numel() == Hkv
    if sm_scale is None:
        sm_scale = D ** -0.5
    dev = q.device
    if q.stride(-1) != 1:
        q = q.contiguous()
    if k.stride(-1) != 1:
        k = k.contiguous()
    if v.stride(-1) != 1:
        v = v.contiguous()
    sink = _as_i64(num_global_blocks, dev)
    local = _as_i64(num_band_blocks, dev)
    o = torch.empty((B, N, Hq, D), dtype=q.dtype, device=dev)
    # strides in (B, H, N, D) order
    qs = _lib.i64_array([q.stride(0), q.stride(2), q.stride(1), q.stride(3)])
    ks = _lib.i64_array(k.stride())
    vs = _lib.i64_array(v.stride())
    os_ = _lib.i64_array([o.stride(0), o.stride(2), o.stride(1), o.stride(3)])
    lib = _lib.load()
    rc = lib.moa_prefill_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), qs, ks, vs, os_,
                             B, Hq, Hkv, N, D, sink.data_ptr(), local.data_ptr(), float(sm_scale),
                             _lib.dtype_code(q.dtype), _lib.current_stream_ptr(dev))
    _lib.check(rc)
    return o


def moa_decode(
    q: Tensor,
    k: Tensor,
    v: Tensor,
    head_start_index: LongTensor,
    head_valid_length: LongTensor,
    sm_scale: float,
) -> Tensor:
    """Single-token decode over the packed per-head caches.

    q ``[B, 1, Hq, D]``, k, v ``[B, sumC, D]`` contiguous, ``head_start_index`` /
    ``head_valid_length`` int64 ``[B, Hkv]``.  Returns ``[B, 1, Hq, D]``.
    Argument meaning follows MoA/kernels/mixture_of_attention.py:389-392,465-473.
    """
    _require_gpu(q, "moa_decode")
    assert q.dim() == 4 and q.shape[1] == 1, "decode takes one query token: q is [B, 1, H, D]"
    assert k.dim() == 3 and v.dim() == 3, "k and v are the packed caches [B, sum_h C_h, D]"
    B, _, Hq, D = q.shape
    assert k.shape == v.shape and k.shape[0] == B and k.shape[2] == D
    assert q.dtype in (torch.float16, torch.bfloat16), "moa decode runs in fp16 or bf16"
    assert k.dtype == q.dtype and v.dtype == q.dtype
    assert k.is_contiguous() and v.is_contiguous(), "the packed caches must be contiguous"
    assert head_start_index is not None and head_valid_length is not None
    Hkv = head_start_index.shape[-1]
    assert head_start_index.shape == (B, Hkv) and head_valid_length.shape == (B, Hkv)
    dev = q.device
    sumC = k.shape[1]
    q3 = q.reshape(B, Hq, D)
    if not q3.is_contiguous():
        q3 = q3.contiguous()
    hs = _as_i64(head_start_index, dev)
    hv = _as_i64(head_valid_length, dev)
    o = torch.empty((B, 1, Hq, D), dtype=q.dtype, device=dev)
    lib = _lib.load()
    need = lib.moa_decode_workspace_bytes(B, Hq, Hkv, D, sumC)
    stream = _lib.current_stream_ptr(dev)
    ws = _workspace(dev, need, "decode", stream)
    rc = lib.moa_decode_fwd(q3.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), ws.data_ptr(),
                            ws.numel(), hs.data_ptr(), hv.data_ptr(), B, Hq, Hkv, D, sumC,
                            float(sm_scale), _lib.dtype_code(q.dtype), stream)
    _lib.check(rc)
    return o


def _dense_debug_attention(query, key, value, sm_scale, head_start_index, head_valid_length,
                           attention_dropout, is_prefill):
    """The reference's ``implementation="sdpa"`` debug path
    (mixture_of_attention.py:184-356): dense causal prefill (the MoA sparsity is
    NOT applied) and grouped dense decode over full rings.  PyTorch ops, kept
    for cross-checking only."""
    from moa_amd.attention.cache_utils import StaticCircularCache

    assert query.dtype in (torch.float16, torch.bfloat16)
    if is_prefill:
        assert query.shape[-1] == key.shape[-1] and key.shape[-1] == value.shape[-1]
        return F.scaled_dot_product_attention(query, key, value, dropout_p=attention_dropout,
                                              is_causal=query.shape[-2] > 1, scale=sm_scale).transpose(1, 2)
    head_index = StaticCircularCache.head_start_index_valid_length_to_head_index(
        head_start_index, head_valid_length)
    ks = StaticCircularCache.to_group_contigious(key, head_index)
    vs = StaticCircularCache.to_group_contigious(value, head_index)
    outs, h0 = [], 0
    for kk, vv in zip(ks, vs):
        n = kk.shape[1]
        outs.append(F.scaled_dot_product_attention(query[:, h0:h0 + n], kk, vv,
                                                   dropout_p=attention_dropout, scale=sm_scale))
        h0 += n
    return torch.cat(outs, dim=1).transpose(1, 2)


def mixture_of_sparse_attention(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    sm_scale: float,
    attention_mask: LongTensor = None,
    attention_dropout: float = 0.0,
    head_start_index: LongTensor = None,
    head_valid_length: LongTensor = None,
    sink_size: LongTensor = None,
    local_size: LongTensor = None,
    implementation: str = "moa",
) -> Tensor:
    """Same contract as the reference's wrapper (mixture_of_attention.py:358-400).

    Args:
        query: ``(batch, num_heads, query_length, head_dim)``.
        key, value: prefill ``(batch, num_heads, key_length, head_dim)``; sparse decode
            ``(batch, sum_h cache_size_h, head_dim)`` (heads concatenated).
        sm_scale: softmax scale.
        attention_mask: unused, as in the reference ("TBD").
        attention_dropout: must be 0 for ``implementation="moa"``.
        head_start_index, head_valid_length: ``(batch, num_heads)`` int64, decode only.
        sink_size, local_size: ``(num_heads,)`` int64 TOKEN counts (multiples of 64), prefill only.
        implementation: ``"moa"`` (HIP kernels) or ``"sdpa"`` (dense debug path).

    Returns ``(batch, query_length, num_heads, head_dim)``.
    """
    is_prefill = not (key.shape[-2] > query.shape[-2])

    # the reference reads head_valid_length.mean().item() here (:406-407), a host sync
    # whose value only matters for prefill; it is not needed and not done.
    if (not is_prefill) and head_valid_length is None:
        warnings.warn("Cannot determine the average key value length. Falling back to dense prefill and slow sparse decode.")

    fall_back_to_dense = is_prefill and key.shape[-2] <= BLOCK_N
    if fall_back_to_dense:
        warnings.warn(
            f"Falling back to dense prefill and slow sparse decode due to small key/value length {key.shape[-2]}.")

    if implementation in ("sdpa", "flash_attention2"):  # noqa, only used for debug purpose
        if implementation == "flash_attention2":
            raise NotImplementedError("flash_attention2 is not available in this build")
        return _dense_debug_attention(query, key, value, sm_scale, head_start_index, head_valid_length,
                                      attention_dropout, is_prefill)

    if implementation != "moa":
        raise NotImplementedError

    assert attention_dropout == 0.0, "the MoA kernels do not implement dropout"
    if is_prefill:
        # shape constraints of the reference's prefill paths (:315-316, block_sparse_attention_prefill.py:649-650)
        Lq, Lk, Lv = query.shape[-1], key.shape[-1], value.shape[-1]
        assert Lq == Lk and Lk == Lv
        H = key.shape[1]
        if fall_back_to_dense:
            # one block: dense causal == one sink block (:412-415)
            sink_blocks = torch.ones(H, dtype=torch.int64, device=query.device)
            band_blocks = torch.ones(H, dtype=torch.int64, device=query.device)
        else:
            assert sink_size is not None and local_size is not None
            sink_blocks = sink_size // BLOCK_N
            band_blocks = local_size // BLOCK_N
        # query arrives [B, H, N, D], usually a transposed view of [B, N, H, D]: pass the view
        return moa_prefill(query.transpose(1, 2), key, value, causal=True,
                           num_global_blocks=sink_blocks, num_band_blocks=band_blocks,
                           kv_layout="HND", sm_scale=sm_scale)
    return moa_decode(query.transpose(1, 2), key, value, head_start_index, head_valid_length, sm_scale)
