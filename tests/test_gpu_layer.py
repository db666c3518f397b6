"""GPU tests of the caller layer (moa_amd.models.llama.modeling_llama): the attention layer wired
like the reference's LlamaMixtureAttention.forward, against an oracle composition on the CPU, and
the head-permutation invariance that set_mixture_of_attention(permute_head=True) relies on."""
import copy

import numpy as np
import pytest
import torch

from oracle.moa_oracle import (StaticCircularCacheOracle, decode_segments, prefill_masked_dense, rope_cos_sin,
                               rope_reference)

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-3, 1e-2


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _layer(dev, hidden, Hq, Hkv, D, seed):
    from moa_amd.models.llama.modeling_llama import LlamaMixtureAttention
    torch.manual_seed(seed)
    layer = LlamaMixtureAttention(hidden, Hq, Hkv, D, layer_idx=0, dtype=torch.float16, device=dev).eval()
    for lin in (layer.q_proj, layer.k_proj, layer.v_proj, layer.o_proj):
        lin.weight.data = (torch.randn(lin.weight.shape) * lin.in_features ** -0.5).to(dev, torch.float16)
    return layer


def _reference_step(layer, x, cos, sin, o, is_prefill, ns, nl, G):
    """Oracle composition from the layer's own projections on: rope_reference -> cache oracle ->
    masked dense prefill / ring decode -> o_proj in fp32."""
    B, q_len, _ = x.shape
    Hq, Hkv, D = layer.num_heads, layer.num_key_value_heads, layer.head_dim
    with torch.no_grad():
        q = layer.q_proj(x).view(B, q_len, Hq, D).transpose(1, 2).cpu()
        k = layer.k_proj(x).view(B, q_len, Hkv, D).transpose(1, 2).cpu()
        v = layer.v_proj(x).view(B, q_len, Hkv, D).transpose(1, 2).cpu()
    qr, kr = rope_reference(q, cos, sin), rope_reference(k, cos, sin)
    sm = D ** -0.5
    if is_prefill:
        o.update_prefill(kr.float().numpy(), v.float().numpy())
        kk = kr.float().repeat_interleave(G, dim=1)
        vv = v.float().repeat_interleave(G, dim=1)
        att = prefill_masked_dense(qr.float(), kk, vv, sm, [n for n in ns for _ in range(G)],
                                   [n for n in nl for _ in range(G)])            # [B, Hq, N, D]
        att = att.transpose(1, 2)
    else:
        o.update_decode(kr.float().numpy(), v.float().numpy())
        a = decode_segments(qr[:, :, 0].double().numpy(), o.key_cache, o.value_cache, o.cache_head_start_index,
                            o.cache_valid_length, sm, group=G)
        att = torch.from_numpy(a).float()[:, None]                               # [B, 1, Hq, D]
    att16 = att.to(torch.float16).float()                                        # the kernels emit fp16
    w = layer.o_proj.weight.data.float().cpu()
    return att16.reshape(B, q_len, Hq * D) @ w.t()


@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (8, 2)])
def test_layer_against_oracle_composition(dev, Hq, Hkv):
    from moa_amd import StaticCircularCache
    B, D, hidden, S = 2, 128, 256, 200
    G = Hq // Hkv
    cache_size = [128, 256, 192, 320][:Hkv]
    static = [64] * Hkv
    layer = _layer(dev, hidden, Hq, Hkv, D, seed=Hq)
    cache = StaticCircularCache([cache_size], static_size=[static], batch_size=B, head_dim=D, device=dev,
                                dtype=torch.float16)
    o = StaticCircularCacheOracle(cache_size, static, B, D)
    ns = [s // 64 for s in static]
    nl = [(c - s) // 64 for c, s in zip(cache_size, static)]
    g = torch.Generator().manual_seed(1)
    x = torch.randn(B, S, hidden, generator=g).to(dev, torch.float16)
    cos, sin = rope_cos_sin(torch.arange(S)[None, :], D, dtype=torch.float16)
    with torch.no_grad():
        out = layer(x, (cos.to(dev), sin.to(dev)), cache)
    ref = _reference_step(layer, x, cos, sin, o, True, ns, nl, G)
    err = (out.float().cpu() - ref).abs()
    assert out.shape == (B, S, hidden)
    assert bool((err <= 4 * ATOL + RTOL * ref.abs()).all()), float(err.max())
    for t in range(4):
        x1 = torch.randn(B, 1, hidden, generator=g).to(dev, torch.float16)
        c1, s1 = rope_cos_sin(torch.full((1, 1), S + t), D, dtype=torch.float16)
        with torch.no_grad():
            out = layer(x1, (c1.to(dev), s1.to(dev)), cache)
        ref = _reference_step(layer, x1, c1, s1, o, False, ns, nl, G)
        err = (out.float().cpu() - ref).abs()
        assert bool((err <= 4 * ATOL + RTOL * ref.abs()).all()), (t, float(err.max()))
    assert cache.cache_valid_length[0].cpu().numpy().tolist() == o.cache_valid_length.tolist()


def test_head_permutation_keeps_the_stack_function(dev):
    """set_mixture_of_attention(permute_head=True) re-orders plan and projections together: prefill
    and decode outputs of the stack stay the same (up to GEMM summation order)."""
    from moa_amd.models.llama.modeling_llama import LlamaMixtureAttentionStack
    L, hidden, H, D, B, S = 2, 256, 4, 64, 2, 300
    torch.manual_seed(3)
    base = LlamaMixtureAttentionStack(L, hidden, H, head_dim=D, dtype=torch.float16, device=dev)
    for p in base.parameters():
        p.data = (torch.randn(p.shape) * 0.06).to(dev, torch.float16)
    plan = {"alphas": [[400, 100, 400, 200], [64, 300, 64, 300]], "betas": [[0.1, 0.0, 0.1, 0.3], [0.2, 0.0, 0.2, 0.0]]}
    outs = []
    for permute in (False, True):
        m = copy.deepcopy(base)
        m.set_mixture_of_attention(copy.deepcopy(plan), permute_head=permute, moa_max_new_token=16)
        if permute:
            assert m.moa_config["alphas"][0] == [100, 200, 400, 400]
        cache = m.new_cache(B, S, dev)
        g = torch.Generator().manual_seed(9)
        x = torch.randn(B, S, hidden, generator=g).to(dev, torch.float16)
        res = [m(x, torch.arange(S, device=dev)[None, :], cache)]
        for t in range(3):
            x1 = torch.randn(B, 1, hidden, generator=g).to(dev, torch.float16)
            res.append(m(x1, torch.full((1, 1), S + t, device=dev), cache))
        outs.append(res)
    for a, b in zip(*outs):
        torch.testing.assert_close(a.float(), b.float(), rtol=2e-2, atol=2e-2)
