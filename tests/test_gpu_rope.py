"""GPU parity of the rotary-embedding kernels (moa_rope_fwd, moa_rope_cache_append) through the
Python surface and the C ABI, against oracle.rope_reference (torch on the CPU in the same dtype)
and the cache oracle.  The kernels round where torch rounds, so the bar is bit-exact."""
import ctypes

import numpy as np
import pytest
import torch

from oracle.moa_oracle import (StaticCircularCacheOracle, decode_segments, rope_cos_sin, rope_reference)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _rand(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g).to(dtype)


def _same_bits(a, b):
    a, b = a.cpu().contiguous(), b.cpu().contiguous()
    if a.dtype == torch.float32:
        return torch.equal(a.view(torch.int32), b.view(torch.int32))
    return torch.equal(a.view(torch.int16), b.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("D", [128, 64])
def test_rope_fwd_bit_exact(dev, dtype, D):
    from moa_amd.kernels.rotary import apply_rotary_pos_emb
    B, Hq, Hkv, N = 2, 5, 3, 37
    # the caller's layout: [B, N, H, D] projections viewed as [B, H, N, D]
    q = _rand((B, N, Hq, D), dtype, 1).transpose(1, 2)
    k = _rand((B, N, Hkv, D), dtype, 2).transpose(1, 2)
    pos = torch.arange(N)[None, :] + torch.tensor([[0], [1000]])
    cos, sin = rope_cos_sin(pos, D, dtype=dtype)
    qe, ke = apply_rotary_pos_emb(q.to(dev), k.to(dev), cos.to(dev), sin.to(dev))
    # the result keeps the layout of a dense input (as torch's elementwise evaluation does)
    assert qe.shape == q.shape and ke.shape == k.shape and qe.stride() == q.stride() and ke.stride() == k.stride()
    assert _same_bits(qe, rope_reference(q, cos, sin))
    # contiguous [B, H, N, D] inputs (the kernel then walks tokens before heads)
    qc, kc = q.contiguous(), k.contiguous()
    qe2, ke2 = apply_rotary_pos_emb(qc.to(dev), kc.to(dev), cos.to(dev), sin.to(dev))
    assert qe2.is_contiguous() and _same_bits(qe2, rope_reference(q, cos, sin)) and _same_bits(ke2, rope_reference(k, cos, sin))
    assert _same_bits(ke, rope_reference(k, cos, sin))
    # one shared position table (batch 1) broadcasts; k alone
    cos1, sin1 = cos[:1], sin[:1]
    _, ke1 = apply_rotary_pos_emb(None, k.to(dev), cos1.to(dev), sin1.to(dev))
    assert _same_bits(ke1, rope_reference(k, cos1, sin1))


def test_rope_fwd_in_place_through_the_c_abi(dev):
    from moa_amd import _lib
    lib = _lib.load()
    B, H, N, D = 1, 4, 64, 128
    q = _rand((B, H, N, D), torch.float16, 3)
    cos, sin = rope_cos_sin(torch.arange(N)[None, :], D, dtype=torch.float16)
    qd, cd, sd = q.to(dev), cos.to(dev), sin.to(dev)
    st = _lib.i64_array(qd.stride())
    rc = lib.moa_rope_fwd(qd.data_ptr(), None, qd.data_ptr(), None, st, None, st, None, cd.data_ptr(),
                          sd.data_ptr(), _lib.i64_array([0, D, 1]), B, H, 0, N, D, _lib.MOA_DTYPE_F16,
                          _lib.current_stream_ptr(dev))
    assert rc == 0, _lib.last_error()
    assert _same_bits(qd, rope_reference(q, cos, sin))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_rope_update_decode_steps(dev, dtype):
    """Prompt through rope_update (rope kernel + insert), then decode steps through the fused
    launch with ring wraparound; caches, indices and q bit-exact against oracle compositions."""
    from moa_amd import StaticCircularCache
    B, D, S, steps = 2, 128, 150, 40
    cache_size = [128, 192, 64, 256]
    static = [64, 64, 64, 64]
    H = len(cache_size)
    cache = StaticCircularCache([cache_size], static_size=[static], batch_size=B, head_dim=D, device=dev,
                                dtype=dtype)
    o = StaticCircularCacheOracle(cache_size, static, B, D)
    q = _rand((B, S, H, D), dtype, 10).transpose(1, 2)
    k = _rand((B, S, H, D), dtype, 11).transpose(1, 2)
    v = _rand((B, S, H, D), dtype, 12).transpose(1, 2)
    cos, sin = rope_cos_sin(torch.arange(S)[None, :], D, dtype=dtype)
    qe, kk, vv = cache.rope_update(q.to(dev), k.to(dev), v.to(dev), cos.to(dev), sin.to(dev), 0)
    k_ref = rope_reference(k, cos, sin)
    assert _same_bits(qe, rope_reference(q, cos, sin)) and _same_bits(kk, k_ref) and _same_bits(vv, v)
    o.update_prefill(k_ref.float().numpy(), v.float().numpy())

    def check(tag):
        assert cache.cache_update_index[0].cpu().numpy().tolist() == o.cache_update_index.tolist(), tag
        assert cache.cache_valid_length[0].cpu().numpy().tolist() == o.cache_valid_length.tolist(), tag
        m = o.mask_cache == 1
        assert np.array_equal(cache.mask_cache[0].cpu().numpy(), o.mask_cache), tag
        assert np.array_equal(cache.key_cache[0].float().cpu().numpy()[m], o.key_cache[m]), tag
        assert np.array_equal(cache.value_cache[0].float().cpu().numpy()[m], o.value_cache[m]), tag

    check("prefill")
    for t in range(steps):
        qn = _rand((B, 1, H, D), dtype, 100 + t).transpose(1, 2)
        kn = _rand((B, 1, H, D), dtype, 200 + t).transpose(1, 2)
        vn = _rand((B, 1, H, D), dtype, 300 + t).transpose(1, 2)
        c1, s1 = rope_cos_sin(torch.full((B, 1), S + t), D, dtype=dtype)
        qe, kc, vc = cache.rope_update(qn.to(dev), kn.to(dev), vn.to(dev), c1.to(dev), s1.to(dev), 0)
        assert qe.shape == (B, H, 1, D) and qe.transpose(1, 2).is_contiguous()
        assert _same_bits(qe, rope_reference(qn, c1, s1)), t
        o.update_decode(rope_reference(kn, c1, s1).float().numpy(), vn.float().numpy())
        assert kc is cache.key_cache[0] and vc is cache.value_cache[0]
        check(("decode", t))
    assert cache._kv_len[0] == S + steps == o.kv_len


def test_fused_step_feeds_the_decode_kernel(dev):
    """rope_update (one launch) + mixture_of_sparse_attention against the oracle's decode on the
    oracle's cache: what a decoder layer sees."""
    from moa_amd import StaticCircularCache, mixture_of_sparse_attention
    dtype, B, D, S = torch.float16, 3, 128, 300
    cache_size, static = [128, 320, 192], [64, 64, 64]
    H = len(cache_size)
    cache = StaticCircularCache([cache_size], static_size=[static], batch_size=B, head_dim=D, device=dev,
                                dtype=dtype)
    o = StaticCircularCacheOracle(cache_size, static, B, D)
    k = (_rand((B, H, S, D), dtype, 1), _rand((B, H, S, D), dtype, 2))
    cos, sin = rope_cos_sin(torch.arange(S)[None, :], D, dtype=dtype)
    cache.rope_update(_rand((B, H, S, D), dtype, 3).to(dev), k[0].to(dev), k[1].to(dev), cos.to(dev),
                      sin.to(dev), 0)
    o.update_prefill(rope_reference(k[0], cos, sin).float().numpy(), k[1].float().numpy())
    for t in range(5):
        qn, kn, vn = (_rand((B, H, 1, D), dtype, 50 + 3 * t + i) for i in range(3))
        c1, s1 = rope_cos_sin(torch.full((B, 1), S + t), D, dtype=dtype)
        qe, kc, vc = cache.rope_update(qn.to(dev), kn.to(dev), vn.to(dev), c1.to(dev), s1.to(dev), 0)
        out = mixture_of_sparse_attention(qe, kc, vc, D ** -0.5,
                                          head_start_index=cache.cache_head_start_index[0],
                                          head_valid_length=cache.cache_valid_length[0])
        o.update_decode(rope_reference(kn, c1, s1).float().numpy(), vn.float().numpy())
        ref = decode_segments(rope_reference(qn, c1, s1)[:, :, 0].double().numpy(), o.key_cache, o.value_cache,
                              o.cache_head_start_index, o.cache_valid_length, D ** -0.5)
        got = out[:, 0].float().cpu().numpy()
        assert np.all(np.abs(got - ref) <= 2e-3 + 1e-2 * np.abs(ref)), t


def test_fused_qkv_projection_buffer(dev):
    """q, k and v as views of ONE fused projection output [B, q_len, (Hq + 2 Hkv) D] (the QKV split
    costs no copy: the entry points take strides), prompt and decode step."""
    from moa_amd import StaticCircularCache
    dtype, B, Hq, Hkv, D, S = torch.bfloat16, 2, 8, 2, 64, 130
    cache_size, static = [128, 192], [64, 64]
    cache = StaticCircularCache([cache_size], static_size=[static], batch_size=B, head_dim=D, device=dev, dtype=dtype)
    o = StaticCircularCacheOracle(cache_size, static, B, D)

    def split(qkv):
        n = qkv.shape[1]
        q = qkv[..., : Hq * D].view(B, n, Hq, D).transpose(1, 2)
        k = qkv[..., Hq * D: (Hq + Hkv) * D].view(B, n, Hkv, D).transpose(1, 2)
        v = qkv[..., (Hq + Hkv) * D:].view(B, n, Hkv, D).transpose(1, 2)
        return q, k, v

    for step, n in enumerate([S, 1, 1]):
        qkv = _rand((B, n, (Hq + 2 * Hkv) * D), dtype, 40 + step)
        pos = torch.arange(n)[None, :] + (0 if step == 0 else S + step - 1)
        cos, sin = rope_cos_sin(pos, D, dtype=dtype)
        q, k, v = split(qkv)
        qe, kk, vv = cache.rope_update(*split(qkv.to(dev)), cos.to(dev), sin.to(dev), 0)
        assert _same_bits(qe, rope_reference(q, cos, sin)), step
        k_ref = rope_reference(k, cos, sin).float().numpy()
        if step == 0:
            o.update_prefill(k_ref, v.float().numpy())
        else:
            o.update_decode(k_ref, v.float().numpy())
        m = o.mask_cache == 1
        assert np.array_equal(cache.key_cache[0].float().cpu().numpy()[m], o.key_cache[m]), step
        assert np.array_equal(cache.value_cache[0].float().cpu().numpy()[m], o.value_cache[m]), step
        assert cache.cache_update_index[0].cpu().numpy().tolist() == o.cache_update_index.tolist(), step


def test_rope_errors(dev):
    from moa_amd import _lib
    from moa_amd.kernels.rotary import apply_rotary_pos_emb
    q = torch.zeros(1, 2, 4, 128, dtype=torch.float16, device=dev)
    cos = torch.zeros(1, 4, 128, dtype=torch.float16, device=dev)
    with pytest.raises(AssertionError):
        apply_rotary_pos_emb(q, None, cos.float(), cos.float())          # dtype mismatch
    with pytest.raises(AssertionError):
        apply_rotary_pos_emb(q, None, cos[:, :3], cos[:, :3])            # seq_len mismatch
    with pytest.raises(NotImplementedError):
        apply_rotary_pos_emb(q, None, cos, cos, unsqueeze_dim=2)
    q8 = torch.zeros(1, 2, 4, 8, dtype=torch.float16, device=dev)        # half a row is 8 bytes
    c8 = torch.zeros(1, 4, 8, dtype=torch.float16, device=dev)
    with pytest.raises(NotImplementedError):
        apply_rotary_pos_emb(q8, None, c8, c8)
    with pytest.raises(_lib.MoaKernelError):
        apply_rotary_pos_emb(q.cpu(), None, cos.cpu(), cos.cpu())
