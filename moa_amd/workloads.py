"""Synthetic workloads of the benchmark configurations: per-head spans from the
elastic rule ``span = alpha + beta * N`` and packed caches filled with noise.

Used by bench.py and the tests; nothing here touches the kernels.
"""
from __future__ import annotations

import math
from typing import List, Tuple

import numpy as np

BLOCK = 64
SINK = 64


def elastic_spans(num_heads: int, n_ctx: int, seed: int, alpha_range=(64.0, 2048.0),
                  beta_range=(0.0, 0.5)) -> List[int]:
    """Per-head window length: alpha ~ U[alpha_range], beta ~ U[beta_range],
    span = min(ceil((alpha + beta * N) / 64) * 64, N)."""
    rng = np.random.default_rng(seed)
    alpha = rng.uniform(alpha_range[0], alpha_range[1], size=num_heads)
    beta = rng.uniform(beta_range[0], beta_range[1], size=num_heads)
    spans = []
    for a, b in zip(alpha, beta):
        s = int(math.ceil((a + b * n_ctx) / BLOCK) * BLOCK)
        spans.append(min(s, (n_ctx // BLOCK) * BLOCK if n_ctx >= BLOCK else BLOCK))
    return spans


def uniform_block_windows(num_heads: int, seed: int, lo_blocks: int = 4, hi_blocks: int = 16) -> List[int]:
    """Windows drawn uniformly from {lo*64, ..., hi*64} (the CPU-reference config)."""
    rng = np.random.default_rng(seed)
    return [int(x) * BLOCK for x in rng.integers(lo_blocks, hi_blocks + 1, size=num_heads)]


def ring_cache_sizes(spans: List[int], sink: int = SINK) -> Tuple[List[int], List[int]]:
    """cache_size = sink + window, static_size = sink for every head."""
    return [sink + s for s in spans], [sink] * len(spans)


def prefill_work(n_ctx: int, sink_blocks: List[int], local_blocks: List[int], batch: int, head_dim: int):
    """(element-exact FLOPs, tile-level FLOPs, live tiles) of one prefill call:
    4 * D flops per unmasked (query, key) pair (two GEMMs, 2 flops per MAC)."""
    nb = (n_ctx + BLOCK - 1) // BLOCK
    pairs = 0
    tiles = 0
    for ns, nl in zip(sink_blocks, local_blocks):
        for m in range(nb):
            rows = min((m + 1) * BLOCK, n_ctx) - m * BLOCK
            hi_sink = min(ns - 1, m)
            lo_local = max(0, m + 1 - nl)
            # live = [0..hi_sink] U [lo_local..m]
            if nl <= 0:
                live = hi_sink + 1
                diag = hi_sink == m
            else:
                live = (hi_sink + 1) + (m - lo_local + 1) - max(0, hi_sink - lo_local + 1)
                diag = True
            if live <= 0:
                continue
            tiles += live
            if diag:
                cols = min((m + 1) * BLOCK, n_ctx) - m * BLOCK
                tri = sum(min(r + 1, cols) for r in range(rows))
                pairs += (live - 1) * rows * BLOCK + tri
            else:
                pairs += live * rows * BLOCK
    flops = 4.0 * head_dim * pairs * batch
    tile_flops = 4.0 * head_dim * BLOCK * BLOCK * tiles * batch
    return flops, tile_flops, tiles * batch


def decode_bytes(valid_rows_total: int, batch: int, heads: int, head_dim: int, elem: int = 2) -> int:
    """K and V rows read once + q and o + the two int64 index arrays."""
    return valid_rows_total * head_dim * 2 * elem + 2 * batch * heads * head_dim * elem + 16 * batch * heads


def rope_append_bytes(batch: int, heads: int, head_dim: int, elem: int = 2) -> int:
    """fused rotary + append step: q, k, v read, q and two cache rows written, cos and sin read,
    plus the append's index traffic."""
    return (6 * batch * heads * head_dim + 2 * batch * head_dim) * elem + 40 * batch * heads


def append_bytes(batch: int, heads: int, head_dim: int, elem: int = 2) -> int:
    """new k, v read + two rows written + update_index r/w, valid_len r/w, mask write."""
    return 4 * batch * heads * head_dim * elem + 40 * batch * heads
