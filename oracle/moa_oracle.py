"""CPU oracle for the MoA sparse-attention hot path.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the smoke
check and the benchmark's CPU-baseline leg may import it; the product package
never does and fails loudly when its HIP library is missing.

It restates, on the CPU (numpy int64 for index work, numpy fp64 / torch fp32
for arithmetic), what the reference computes on the path

    StaticCircularCache.update  ->  mixture_of_sparse_attention

Each function cites the reference lines it follows (paths are relative to the
reference checkout).  What pins each function (see tests/test_oracle_*.py):

  live_kv_blocks / moa_token_mask   the two are independent formulations (block
      enumeration of the kernel's loop vs. a closed-form token predicate) and
      are checked against each other exhaustively on small (N, ns, nl); the
      special cases nl >= nb or ns >= nb reduce to plain causal attention.
  prefill_masked_dense              library routine (torch SDPA with a boolean
      mask); special case == is_causal SDPA (the case the reference's own test
      pins, tests/attention_kernel_test.py:35-76); V == 1 => O == 1.
  prefill_blockwise                 follows the kernel's block loop and its
      base-2 incremental softmax; checked against prefill_masked_dense and a
      brute-force triple loop.
  prefill_p_rounded                 the same attention with the softmax weights rounded to the
      storage type in front of P.V (where the reference's kernel rounds them); equals
      prefill_masked_dense without rounding, a pure-Python loop that rounds through torch's
      casts on a tiny input, and itself under integer shifts of the reference exponent.
  decode_segments                   closed form; checked against
      decode_grouped_sdpa (the reference's grouped-SDPA decode), ring-order
      invariance and prefill/decode consistency.
  RingModel                         plain list + deque; pins
      StaticCircularCacheOracle (the formula restatement) bit-exactly, and
      both are checked against golden vectors in tests/golden/.
  moa_config_to_cache_config        hand-computed known answers + shipped
      plans.
  rope_reference                    the published formula of transformers'
      apply_rotary_pos_emb (the reference's pinned dependency, not vendored);
      checked bit for bit against the installed transformers' function, a
      hand-computed known answer, identity at position 0, norm preservation
      and the relative-position property in fp64.

Parity unpinned (no reference test, fixture or runnable implementation covers
it): the external ``flashinfer.moa_decode`` CUDA op.  Its semantics are taken
from its call site and argument docs (MoA/kernels/mixture_of_attention.py:389-392,
465-473) and from the reference's grouped-SDPA decode which it replaces.
"""

from __future__ import annotations

import math
from collections import deque
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

BLOCK = 64  # MoA/kernels/mixture_of_attention.py:32-33

# --------------------------------------------------------------------------
# Prefill: which keys a query sees
# --------------------------------------------------------------------------


def live_kv_blocks(m: int, ns: int, nl: int) -> List[int]:
    """KV block ids visited for query block ``m`` of a head with ``ns`` sink
    blocks and ``nl`` local blocks, in visiting order.

    Follows the kernel's loop: MoA/kernels/block_sparse_attention_prefill.py:558-567
    (max_block_idx = m; skip ids with  max_sink_idx < id < min_local_idx).
    """
    max_block_idx = m
    min_local_idx = max(0, max_block_idx + 1 - nl)
    max_sink_idx = min(ns - 1, max_block_idx)
    out = []
    j = 0
    while j <= max_block_idx:
        if j > max_sink_idx and j < min_local_idx:
            pass
        else:
            out.append(j)
        j += 1
    return out


def moa_token_mask(n_ctx: int, ns: int, nl: int, block: int = BLOCK) -> np.ndarray:
    """Dense boolean mask [n_ctx, n_ctx]; True = query i may see key j.

    Closed form of block layout AND causal (MoA/attention/convert.py:159-192 with
    the sink+band layout of block_sparse_attention_prefill.py:558-580):
        j <= i  and  ( floor(j/B) < ns  or  floor(j/B) >= floor(i/B) + 1 - nl ).
    """
    i = np.arange(n_ctx)[:, None]
    j = np.arange(n_ctx)[None, :]
    bi, bj = i // block, j // block
    return (j <= i) & ((bj < ns) | (bj >= bi + 1 - nl))


def moa_token_mask_from_blocks(n_ctx: int, ns: int, nl: int, block: int = BLOCK) -> np.ndarray:
    """Same mask built the way the kernel walks it: per query block enumerate
    live_kv_blocks, then apply the in-block causal test
    (block_sparse_attention_prefill.py:579-580)."""
    nb = (n_ctx + block - 1) // block
    mask = np.zeros((n_ctx, n_ctx), dtype=bool)
    for m in range(nb):
        r0, r1 = m * block, min((m + 1) * block, n_ctx)
        for jb in live_kv_blocks(m, ns, nl):
            c0, c1 = jb * block, min((jb + 1) * block, n_ctx)
            rows = np.arange(r0, r1)[:, None]
            cols = np.arange(c0, c1)[None, :]
            mask[r0:r1, c0:c1] = rows >= cols
    return mask


def count_live_pairs(n_ctx: int, ns: int, nl: int, block: int = BLOCK) -> Tuple[int, int]:
    """(#unmasked (i,j) pairs, #live tiles) for one head -- the algorithmic
    work figure of the prefill kernel.  Exact count from the mask definition."""
    nb = (n_ctx + block - 1) // block
    pairs = 0
    tiles = 0
    for m in range(nb):
        rows = min((m + 1) * block, n_ctx) - m * block
        for jb in live_kv_blocks(m, ns, nl):
            tiles += 1
            cols = min((jb + 1) * block, n_ctx) - jb * block
            if jb == m:
                # causal triangle inside the diagonal block
                pairs += sum(min(r + 1, cols) for r in range(rows))
            else:
                pairs += rows * cols
    return pairs, tiles


# --------------------------------------------------------------------------
# Prefill arithmetic
# --------------------------------------------------------------------------


def prefill_masked_dense(q, k, v, sm_scale: float, sink_blocks, local_blocks,
                         block: int = BLOCK):
    """Dense masked attention in fp32 with torch SDPA on the CPU.

    q, k, v: torch tensors [B, H, N, D] (any float dtype; computed in fp32).
    sink_blocks/local_blocks: per-head block counts [H].
    Returns fp32 [B, H, N, D].  Rows with no visible key return 0, as the
    kernel's accumulator does (block_sparse_attention_prefill.py:529-531).

    Same library call as the reference's dense paths
    (MoA/kernels/mixture_of_attention.py:328-336,
     MoA/kernels/block_sparse_attention_prefill.py:293-301).
    """
    import torch
    import torch.nn.functional as F

    B, H, N, D = q.shape
    qf, kf, vf = q.float().cpu(), k.float().cpu(), v.float().cpu()
    out = torch.empty(B, H, N, D, dtype=torch.float32)
    for h in range(H):
        mask_np = moa_token_mask(N, int(sink_blocks[h]), int(local_blocks[h]), block)
        mask = torch.from_numpy(mask_np)
        dead = ~mask.any(dim=-1)
        if dead.any():
            mask = mask.clone()
            mask[dead, 0] = True  # avoid NaN rows inside SDPA; zeroed below
        o = F.scaled_dot_product_attention(
            qf[:, h:h + 1], kf[:, h:h + 1], vf[:, h:h + 1],
            attn_mask=mask[None, None], scale=sm_scale)
        if dead.any():
            o[:, :, dead, :] = 0.0
        out[:, h] = o[:, 0]
    return out


def prefill_blockwise(q: np.ndarray, k: np.ndarray, v: np.ndarray, sm_scale: float,
                      ns: int, nl: int, block: int = BLOCK) -> np.ndarray:
    """One head, fp64, following the kernel's structure: per query block, loop
    over live KV blocks with the base-2 online softmax and its incremental
    normalisation (block_sparse_attention_prefill.py:537-610), without the
    fp16 roundings.  q, k, v: [N, D].  Small inputs only."""
    N, D = q.shape
    nb = (N + block - 1) // block
    out = np.zeros((N, D), dtype=np.float64)
    qk_scale = sm_scale * 1.4426950408889634
    for m in range(nb):
        r0, r1 = m * block, min((m + 1) * block, N)
        qm = q[r0:r1].astype(np.float64) * qk_scale
        m_i = np.full(r1 - r0, -np.inf)
        l_i = np.zeros(r1 - r0)
        acc = np.zeros((r1 - r0, D))
        offs_m = np.arange(r0, r1)
        for jb in live_kv_blocks(m, ns, nl):
            c0, c1 = jb * block, min((jb + 1) * block, N)
            qk = qm @ k[c0:c1].astype(np.float64).T
            offs_n = np.arange(c0, c1)
            qk = np.where(offs_m[:, None] >= offs_n[None, :], qk, -np.inf)
            m_ij = qk.max(axis=1)
            with np.errstate(invalid="ignore"):
                p = np.where(np.isneginf(m_ij)[:, None], 0.0, np.exp2(qk - m_ij[:, None]))
            l_ij = p.sum(axis=1)
            m_new = np.maximum(m_i, m_ij)
            with np.errstate(invalid="ignore"):
                alpha = np.where(np.isneginf(m_new), 0.0, np.exp2(m_i - m_new))
                beta = np.where(np.isneginf(m_new), 0.0, np.exp2(m_ij - m_new))
            l_i = l_i * alpha
            l_new = l_i + beta * l_ij
            safe = np.where(l_new > 0, l_new, 1.0)
            p = p * (beta / safe)[:, None]
            acc = acc * (l_i / safe)[:, None]
            acc = acc + p @ v[c0:c1].astype(np.float64)
            l_i, m_i = l_new, m_new
        out[r0:r1] = acc
    return out


def prefill_bruteforce(q: np.ndarray, k: np.ndarray, v: np.ndarray, sm_scale: float,
                       ns: int, nl: int, block: int = BLOCK) -> np.ndarray:
    """One head, pure-Python loops, fp64.  Tiny inputs only (N ~ 200, D ~ 16)."""
    N, D = q.shape
    out = np.zeros((N, D))
    for i in range(N):
        ws = []
        js = []
        for j in range(i + 1):
            if (j // block) < ns or (j // block) >= (i // block) + 1 - nl:
                s = 0.0
                for d in range(D):
                    s += float(q[i, d]) * float(k[j, d])
                ws.append(s * sm_scale)
                js.append(j)
        if not js:
            continue
        mx = max(ws)
        es = [math.exp(w - mx) for w in ws]
        z = sum(es)
        for e, j in zip(es, js):
            for d in range(D):
                out[i, d] += e / z * float(v[j, d])
    return out


def round_to_storage(x: np.ndarray, p_dtype: Optional[str]) -> np.ndarray:
    """fp32 values rounded to nearest-even into ``"bf16"`` (8 significant bits) or ``"f16"`` (11 bits,
    subnormals below 2^-14), returned as fp32; ``None`` returns ``x`` unchanged.  bf16 is done on the
    bit pattern (add 0x7fff + lsb, truncate), independent of any library's cast."""
    x = np.asarray(x, dtype=np.float32)
    if p_dtype is None:
        return x
    if p_dtype == "f16":
        return x.astype(np.float16).astype(np.float32)
    assert p_dtype == "bf16", p_dtype
    u = x.view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).reshape(x.shape)


def prefill_p_rounded(q, k, v, sm_scale: float, sink_blocks, local_blocks, p_dtype: Optional[str],
                      block: int = BLOCK, shift: int = 0, rows_per_step: int = 1024) -> np.ndarray:
    """Masked attention whose softmax weights enter the P.V product ROUNDED to the storage type,
    the place where the reference's kernel rounds them (``p.to(tl.float16)`` in front of
    ``tl.dot(p, v)``, MoA/kernels/block_sparse_attention_prefill.py:608-610), everything else exact:

        t_ij = log2(e) * sm_scale * (q_i . k_j)                       fp64
        M_i  = ceil(max_j t_ij) + shift                                an integer
        p_ij = fp32(2^(t_ij - M_i))                                    unnormalised weight
        o_i  = sum_j round(p_ij) v_j / sum_j p_ij                      the sum of weights is NOT rounded (:590)

    Because M_i is an integer, round() is applied to 2^frac * 2^int and the rounding of a binary
    floating-point format does not depend on the power of two: the result is the same for every
    integer ``shift`` (while nothing over- or underflows) and therefore does not depend on the order
    in which an online-softmax kernel meets the keys, as long as that kernel keeps its running
    reference exponent integral.  The reference's own kernel rounds the weight scaled by a
    non-integral running normaliser instead (:593-609); the two differ by independent rounding
    errors of the same size (relative 2^-8 per weight for bf16, 2^-11 for f16).

    q, k, v: torch tensors or arrays [B, H, N, D]; returns fp64 [B, H, N, D].  ``p_dtype=None``
    rounds nothing and equals prefill_masked_dense.  Rows with no visible key return 0.
    """
    def arr(t):
        if hasattr(t, "detach"):
            t = t.detach().float().cpu().numpy()
        return np.asarray(t, dtype=np.float64)

    qa, ka, va = arr(q), arr(k), arr(v)
    B, H, N, D = qa.shape
    out = np.zeros((B, H, N, D), dtype=np.float64)
    c = sm_scale * 1.4426950408889634
    for h in range(H):
        mask = moa_token_mask(N, int(sink_blocks[h]), int(local_blocks[h]), block)
        for b in range(B):
            for r0 in range(0, N, rows_per_step):
                r1 = min(N, r0 + rows_per_step)
                m = mask[r0:r1, :r1]                       # causal: no key beyond the last row of the step
                t = (qa[b, h, r0:r1] @ ka[b, h, :r1].T) * c
                t = np.where(m, t, -np.inf)
                alive = m.any(axis=1)
                M = np.where(alive, np.ceil(np.max(t, axis=1, initial=-np.inf, where=m)), 0.0) + shift
                p = np.exp2(t - M[:, None]).astype(np.float32)
                l = p.astype(np.float64).sum(axis=1)
                pr = round_to_storage(p, p_dtype).astype(np.float64)
                o = pr @ va[b, h, :r1]
                out[b, h, r0:r1] = np.where(alive[:, None], o / np.where(alive, l, 1.0)[:, None], 0.0)
    return out


# --------------------------------------------------------------------------
# Decode arithmetic
# --------------------------------------------------------------------------


def decode_segments(q: np.ndarray, kc: np.ndarray, vc: np.ndarray,
                    head_start: np.ndarray, head_valid: np.ndarray,
                    sm_scale: float, group: int = 1, p_dtype: Optional[str] = None,
                    abs_v: bool = False) -> np.ndarray:
    """Per (b, h): softmax(sm_scale * q . K_seg^T) V_seg over rows
    [start[b,hk], start[b,hk] + valid[b,hk]) of the packed cache; no mask.

    q [B, Hq, D]; kc, vc [B, sumC, D]; head_start/head_valid [B, Hkv] int64;
    query head h reads kv head h // group.  fp64.  Returns [B, Hq, D].
    A head with valid == 0 returns 0.

    ``p_dtype`` ("bf16" / "f16"): the weights enter the product with V rounded to that type, with
    the integral reference exponent of prefill_p_rounded (same formula, same reasons); the
    grouped-query kernel works like that.  ``abs_v``: attend to |V| (the scale of a weight-rounding
    error bound).

    Semantics of the external decode op as used at
    MoA/kernels/mixture_of_attention.py:465-473 (argument docs :389-392), and of
    the grouped-SDPA decode it replaces (:226-310).
    """
    B, Hq, D = q.shape
    out = np.zeros((B, Hq, D), dtype=np.float64)
    for b in range(B):
        for h in range(Hq):
            hk = h // group
            s0 = int(head_start[b, hk])
            n = int(head_valid[b, hk])
            if n == 0:
                continue
            ks = kc[b, s0:s0 + n].astype(np.float64)
            vs = vc[b, s0:s0 + n].astype(np.float64)
            if abs_v:
                vs = np.abs(vs)
            s = ks @ q[b, h].astype(np.float64) * sm_scale
            if p_dtype is None:
                s -= s.max()
                p = np.exp(s)
                out[b, h] = (p / p.sum()) @ vs
            else:
                t = s * 1.4426950408889634
                p = np.exp2(t - np.ceil(t.max())).astype(np.float32)
                out[b, h] = (round_to_storage(p, p_dtype).astype(np.float64) @ vs) / p.astype(np.float64).sum()
    return out


def head_start_valid_to_head_index(head_start: np.ndarray, head_valid: np.ndarray) -> np.ndarray:
    """MoA/attention/cache_utils.py:820-840: [H+1] segment boundaries; requires all
    batch rows equal; the last boundary uses the last head's valid length."""
    assert (head_start == head_start[0]).all()
    assert (head_valid == head_valid[0]).all()
    return np.concatenate([head_start[0], [head_start[0][-1] + head_valid[0][-1]]]).astype(np.int64)


def to_group_contiguous(t: np.ndarray, head_index: np.ndarray) -> List[np.ndarray]:
    """MoA/attention/cache_utils.py:889-951: split a packed [B, sumC, (D)] tensor into
    runs of consecutive heads with equal size, each viewed [B, n, C, (D)]."""
    sizes = head_index[1:] - head_index[:-1]
    groups = []
    i = 0
    H = len(sizes)
    while i < H:
        j = i
        while j + 1 < H and sizes[j + 1] == sizes[i]:
            j += 1
        cnt = j - i + 1
        start = int(head_index[i])
        end = int(head_index[j]) + int(sizes[i])
        sl = t[:, start:end]
        groups.append(sl.reshape((t.shape[0], cnt, int(sizes[i])) + t.shape[2:]).copy())
        i = j + 1
    return groups


def decode_grouped_sdpa(q, kc, vc, head_index, sm_scale: float):
    """The reference's debug decode: group heads of equal ring size and run SDPA
    per group (MoA/kernels/mixture_of_attention.py:226-310).  torch fp32 on CPU.
    q [B,H,1,D]; kc, vc [B,sumC,D]; returns [B,1,H,D]."""
    import torch
    import torch.nn.functional as F

    qf = q.float().cpu()
    kg = to_group_contiguous(kc.float().cpu().numpy(), np.asarray(head_index))
    vg = to_group_contiguous(vc.float().cpu().numpy(), np.asarray(head_index))
    outs = []
    h0 = 0
    for kk, vv in zip(kg, vg):
        n = kk.shape[1]
        o = F.scaled_dot_product_attention(
            qf[:, h0:h0 + n], torch.from_numpy(kk), torch.from_numpy(vv), scale=sm_scale)
        outs.append(o)
        h0 += n
    return torch.cat(outs, dim=1).transpose(1, 2)


# --------------------------------------------------------------------------
# Ring semantics: an independent integer model
# --------------------------------------------------------------------------


class RingModel:
    """One (batch row, head): the first ``s`` tokens are kept forever, the last
    ``c`` of the rest live in a ring.  Pure list + deque; no index formulas
    except the slot a ring token occupies (its age modulo c).

    The physical layout it predicts is the reference's: static tokens at
    start..start+s-1, ring token with ring-ordinal r (0 = first token after the
    static part) at start + s + (r mod c)
    (MoA/attention/cache_utils.py:1046-1054, :1088-1107).
    """

    def __init__(self, start: int, s: int, c: int):
        self.start, self.s, self.c = start, s, c
        self.static: List[int] = []
        self.ring: deque = deque(maxlen=c) if c > 0 else deque(maxlen=0)
        self.n_seen = 0
        self.evicted: List[int] = []

    def push(self, token_id: int) -> None:
        if len(self.static) < self.s:
            self.static.append(token_id)
        else:
            if self.c > 0 and len(self.ring) == self.c:
                self.evicted.append(self.ring[0][1])
            ordinal = self.n_seen - self.s
            if self.c > 0:
                self.ring.append((ordinal, token_id))
            else:
                self.evicted.append(token_id)
        self.n_seen += 1

    def slot_map(self) -> Dict[int, int]:
        """physical slot -> token id"""
        m = {self.start + i: t for i, t in enumerate(self.static)}
        for ordinal, t in self.ring:
            m[self.start + self.s + (ordinal % self.c)] = t
        return m

    @property
    def valid_length(self) -> int:
        return len(self.static) + len(self.ring)

    @property
    def next_slot(self) -> int:
        """Where the next token is written."""
        if self.n_seen < self.s:
            return self.start + self.n_seen
        if self.c == 0:
            return self.start + self.s
        return self.start + self.s + ((self.n_seen - self.s) % self.c)


# --------------------------------------------------------------------------
# StaticCircularCache: restatement of the reference's formulas (int64 numpy)
# --------------------------------------------------------------------------


class StaticCircularCacheOracle:
    """Index bookkeeping and payload movement of the reference cache for ONE
    layer, restated formula by formula.

    ctor      MoA/attention/cache_utils.py:698-818
    decode    :1020-1058
    prefill   :1060-1164 (incl. attention_mask / left padding)

    Payload is any numpy array [B, H, S, D]; the cache is [B, sumC, D].
    """

    def __init__(self, cache_size: Sequence[int], static_size: Sequence[int],
                 batch_size: int, head_dim: int, dtype=np.float32):
        cs = np.asarray(cache_size, dtype=np.int64)
        ss = np.asarray(static_size, dtype=np.int64)
        self.H = len(cs)
        self.B = batch_size
        self.cache_max_length = cs
        self.static_cache_size = ss
        self.circular_cache_size = cs - ss
        starts = np.concatenate([[0], np.cumsum(cs)[:-1]]).astype(np.int64)
        self.head_index = np.concatenate([starts, [starts[-1] + cs[-1]]]).astype(np.int64)
        self.cache_head_start_index = np.broadcast_to(starts, (batch_size, self.H)).copy()
        self.circular_cache_head_index = starts + ss
        self.cache_update_index = np.broadcast_to(starts, (batch_size, self.H)).copy()
        self.layer_cache_size = int(cs.sum())
        self.kv_len = 0
        self.key_cache = np.zeros((batch_size, self.layer_cache_size, head_dim), dtype=dtype)
        self.value_cache = np.zeros((batch_size, self.layer_cache_size, head_dim), dtype=dtype)
        self.mask_cache = np.zeros((batch_size, self.layer_cache_size), dtype=np.int64)
        self.cache_valid_length = np.zeros((batch_size, self.H), dtype=np.int64)

    # -- decode branch -----------------------------------------------------
    def update_decode(self, k_new: np.ndarray, v_new: np.ndarray) -> None:
        """k_new, v_new [B, H, 1, D] (only the last token is used, :1033-1034)."""
        B = self.B
        idx = self.cache_update_index
        bidx = np.arange(B)[:, None]
        self.mask_cache[bidx, idx] = 1
        self.value_cache[bidx, idx] = v_new[:, :, -1, :]
        self.key_cache[bidx, idx] = k_new[:, :, -1, :]
        self.cache_valid_length += (self.cache_valid_length < self.cache_max_length[None, :])
        is_circ = (self.kv_len + 1 > self.static_cache_size)[None, :]
        ch = self.circular_cache_head_index[None, :]
        csz = self.circular_cache_size[None, :]
        with np.errstate(divide="ignore", invalid="ignore"):
            circ = _py_mod(idx + 1 - ch, csz) + ch
        self.cache_update_index = np.where(is_circ, circ, idx + 1)
        self.kv_len += 1

    # -- prefill branch ----------------------------------------------------
    def update_prefill(self, k: np.ndarray, v: np.ndarray,
                       attention_mask: Optional[np.ndarray] = None) -> np.ndarray:
        """k, v [B, H, S, D]; attention_mask [B, >=S] of 0/1 or None.
        Returns the boolean keep map [B, H, S] (which tokens were stored)."""
        B, H, S, _ = k.shape
        if attention_mask is not None:
            am = np.asarray(attention_mask, dtype=np.int64)[:, -S:]
        else:
            am = np.ones((B, S), dtype=np.int64)
        ap = np.cumsum(am, axis=-1) - 1
        ap = np.concatenate([ap, ap[:, -1:] + 1], axis=-1)            # [B, S+1]
        rap = np.flip(np.cumsum(np.flip(am, -1), -1), -1)             # [B, S]
        upd = self.cache_update_index[:, None, :]                      # [B,1,H]
        ch = self.circular_cache_head_index[None, None, :]
        csz = self.circular_cache_size[None, None, :]
        idx_circ = _py_mod(upd + ap[:, :, None] - ch, csz) + ch
        idx_stat = upd + ap[:, :, None]
        slot = np.where(self.kv_len + ap[:, :, None] > self.static_cache_size[None, None, :],
                        idx_circ, idx_stat)                            # [B,S+1,H]
        self.cache_update_index = slot[:, -1, :].copy()
        slot = slot[:, :-1, :].transpose(0, 2, 1)                      # [B,H,S]
        keep = ((rap[:, None, :] <= self.circular_cache_size[None, :, None])
                | (slot < self.circular_cache_head_index[None, :, None])) & (am[:, None, :] == 1)
        self.cache_valid_length = self.cache_valid_length + keep.sum(-1)
        self.kv_len += S
        b_i, h_i, t_i = np.nonzero(keep)
        dst = slot[b_i, h_i, t_i]
        self.mask_cache[b_i, dst] = am[b_i, t_i]
        self.key_cache[b_i, dst] = k[b_i, h_i, t_i]
        self.value_cache[b_i, dst] = v[b_i, h_i, t_i]
        return keep

    def update(self, k, v, attention_mask=None):
        if k.shape[-2] == 1:
            self.update_decode(k, v)
        else:
            self.update_prefill(k, v, attention_mask)


def _py_mod(a: np.ndarray, m: np.ndarray) -> np.ndarray:
    """torch's ``%`` on int64 (sign follows the divisor), which the reference
    relies on at cache_utils.py:1046-1054 and :1088-1096.  Division by a zero
    ring size never occurs in a live branch; it yields 0 here."""
    a = np.asarray(a, dtype=np.int64)
    m = np.broadcast_to(np.asarray(m, dtype=np.int64), a.shape)
    out = np.zeros_like(a)
    nz = m != 0
    out[nz] = np.mod(a[nz], m[nz])
    return out


# --------------------------------------------------------------------------
# Plan -> cache sizes
# --------------------------------------------------------------------------


def moa_config_to_cache_config(moa_config: dict, seq_len: int, max_new_token: int = 1024,
                               sink_size: int = 64, minimum_cache_size: int = 128,
                               split_size: int = 64) -> Dict[str, List[List[int]]]:
    """MoA/attention/cache_utils.py:1183-1239."""
    cache, static = [], []
    for al, bl in zip(moa_config["alphas"], moa_config["betas"]):
        cl, sl = [], []
        for a, b in zip(al, bl):
            c = int(a + (seq_len + max_new_token) * b)
            c = min(c, seq_len + max_new_token)
            c = math.ceil(max(c, minimum_cache_size) / split_size) * split_size
            cl.append(c)
            sl.append(min(c, sink_size))
        cache.append(cl)
        static.append(sl)
    return {"cache_size": cache, "static_size": static}


# --------------------------------------------------------------------------
# Rotary position embedding (the step in front of the path)
# --------------------------------------------------------------------------


def rope_reference(x, cos, sin):
    """``x*cos + rotate_half(x)*sin`` evaluated by torch on the CPU in x's dtype.

    Restates transformers 4.44.2 ``apply_rotary_pos_emb`` / ``rotate_half``
    (models/llama/modeling_llama.py of that package; the reference pins it in
    requirements.txt:8 and calls it at MoA/models/llama/modeling_llama.py:252).
    x ``[B, H, N, D]`` torch tensor, cos/sin ``[B or 1, N, D]``; they are
    unsqueezed at dim 1 like the reference's call (unsqueeze_dim=1).
    """
    import torch

    x = x.cpu()
    cos = cos.cpu().unsqueeze(1)
    sin = sin.cpu().unsqueeze(1)
    half = x.shape[-1] // 2
    rot = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return (x * cos) + (rot * sin)


def rope_cos_sin(positions, head_dim: int, base: float = 10000.0, dtype=None):
    """cos/sin tables ``[B, N, D]`` as LlamaRotaryEmbedding builds them (default rope type):
    inv_freq = base^(-2i/D), freqs = pos * inv_freq in fp32, emb = cat(freqs, freqs), cast to dtype.
    positions: integer tensor ``[B, N]``."""
    import torch

    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    freqs = positions.cpu().float()[:, :, None] * inv_freq[None, None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    cos, sin = emb.cos(), emb.sin()
    if dtype is not None:
        cos, sin = cos.to(dtype), sin.to(dtype)
    return cos, sin

