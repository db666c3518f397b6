"""MoA sparse-attention runtime for AMD MI355X.

Mirrors the reference's Python surface for the attention hot path:

    moa_amd.kernels.mixture_of_attention.mixture_of_sparse_attention
    moa_amd.attention.cache_utils.StaticCircularCache
    moa_amd.attention.cache_utils.moa_config_to_cache_config

and runs it on hand-written gfx950 kernels in libmoa_hip.so.
"""
from moa_amd.attention.cache_utils import StaticCircularCache, moa_config_to_cache_config  # noqa: F401
from moa_amd.kernels.mixture_of_attention import (  # noqa: F401
    mixture_of_sparse_attention,
    moa_decode,
    moa_prefill,
)

__all__ = [
    "StaticCircularCache",
    "moa_config_to_cache_config",
    "mixture_of_sparse_attention",
    "moa_prefill",
    "moa_decode",
]
