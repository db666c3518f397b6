"""Head permutation of a MoA plan: cluster the heads of a layer that share (alpha, beta) and
re-order the attention projections to match.

Mirrors the three functions of the reference's caller layer that the runtime path depends on
(MoA/attention/permutation_utils.py:5-96 ``permute_attention_projection`` /
``permute_output_projection``, :219-269 ``moa_config_to_permutation``); same names, arguments and
results.  Host-side, one-off per model load: plain index work on the weights.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch
from torch import nn


def moa_config_to_permutation(moa_config) -> Tuple[List[torch.Tensor], List[Dict[int, Tuple[int, int]]]]:
    """Per layer: the stable order of the heads by (alpha, beta) and the runs of equal pairs.

    Returns ``(permutations, clusters)``: ``permutations[l]`` is an int64 tensor whose i-th entry is
    the ORIGINAL index of the head that sits at position i afterwards; ``clusters[l]`` maps a run
    number to the inclusive ``(first, last)`` positions of that run (reference :219-269: sort by
    ``(alpha, beta)`` with the original index as tie-break, then split where the pair changes).
    """
    permutations, clusters = [], []
    for alphas, betas in zip(moa_config["alphas"], moa_config["betas"]):
        pairs = [(float(a), float(b)) for a, b in zip(alphas, betas)]
        order = sorted(range(len(pairs)), key=lambda i: (pairs[i], i))
        permutations.append(torch.tensor(order, dtype=torch.int64))
        runs: Dict[int, Tuple[int, int]] = {}
        first = 0
        for pos in range(1, len(order) + 1):
            if pos == len(order) or pairs[order[pos]] != pairs[order[first]]:
                runs[len(runs)] = (first, pos - 1)
                first = pos
        clusters.append(runs)
    return permutations, clusters


def _expand_groups(permutation: torch.Tensor, num_heads: int, num_key_value_groups: Optional[int]):
    """A permutation of kv heads, expanded to the query heads they own (reference :19-30)."""
    assert permutation.dim() == 1 and permutation.shape[0] == num_heads
    g = 1 if num_key_value_groups is None else int(num_key_value_groups)
    if g == 1:
        return permutation, num_heads
    expanded = (permutation[:, None] * g + torch.arange(g, device=permutation.device, dtype=permutation.dtype)[None, :])
    return expanded.reshape(-1), num_heads * g


def permute_attention_projection(layer: nn.Linear, permutation: Optional[torch.Tensor] = None,
                                 num_heads: Optional[int] = None,
                                 num_key_value_groups: Optional[int] = None) -> None:
    """Re-orders the output rows of a q/k/v projection head by head, in place (reference :5-52):
    afterwards head i of the projection is the old head ``permutation[i]``."""
    if permutation is None:
        return
    permutation, heads = _expand_groups(permutation, num_heads, num_key_value_groups)
    w = layer.weight.data
    head_dim = layer.out_features // heads
    idx = permutation.to(w.device)
    layer.weight.data = w.view(heads, head_dim, layer.in_features).index_select(0, idx).reshape(w.shape).contiguous()
    if layer.bias is not None:
        b = layer.bias.data
        layer.bias.data = b.view(heads, head_dim).index_select(0, idx).reshape(b.shape).contiguous()


def permute_output_projection(layer: nn.Linear, permutation: Optional[torch.Tensor] = None,
                              num_heads: Optional[int] = None,
                              num_key_value_groups: Optional[int] = None) -> None:
    """Re-orders the input columns of o_proj head by head, in place, so that it accepts the
    permuted attention output (reference :55-96)."""
    if permutation is None:
        return
    permutation, heads = _expand_groups(permutation, num_heads, num_key_value_groups)
    w = layer.weight.data
    head_dim = layer.in_features // heads
    idx = permutation.to(w.device)
    layer.weight.data = w.view(layer.out_features, heads, head_dim).index_select(1, idx).reshape(w.shape).contiguous()
