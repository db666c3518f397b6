"""Operands with more than 2**31 elements: every kernel of the path indexes with
64 bits.  The batch is raised until each packed cache tensor (decode, append,
prompt insert) or each q/k/v/o tensor (prefill) crosses 2**31 elements; the
checks look at the far end of the tensors, where a 32-bit offset would have
wrapped, with the same oracles and tolerances as the tests at ordinary sizes."""
import numpy as np
import pytest
import torch

from oracle.moa_oracle import decode_segments, moa_token_mask
from prefill_checks import close_counted, close_stated, masked_attention_gpu

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-3, 1e-2


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _plan(B, D):
    from moa_amd.workloads import elastic_spans, ring_cache_sizes
    cache_size, static_size = ring_cache_sizes(elastic_spans(32, 16384, seed=0))
    assert B * sum(cache_size) * D > 2 ** 31
    return cache_size, static_size


def test_decode_over_2g_elements(dev):
    from moa_amd import mixture_of_sparse_attention
    B, H, D = 112, 32, 128
    sizes, _ = _plan(B, D)
    sizes = np.asarray(sizes)
    sumc = int(sizes.sum())
    gd = torch.Generator(device=dev).manual_seed(5)
    kc = torch.randn(B, sumc, D, generator=gd, device=dev, dtype=torch.float16)
    vc = torch.randn(B, sumc, D, generator=gd, device=dev, dtype=torch.float16)
    q = torch.randn(B, H, 1, D, generator=gd, device=dev, dtype=torch.float16)
    start = np.concatenate([[0], np.cumsum(sizes)[:-1]])
    hs = torch.from_numpy(np.broadcast_to(start, (B, H)).astype(np.int64).copy()).to(dev)
    hv = torch.from_numpy(np.broadcast_to(sizes, (B, H)).astype(np.int64).copy()).to(dev)
    sm = D ** -0.5
    out = mixture_of_sparse_attention(q, kc, vc, sm, head_start_index=hs, head_valid_length=hv)
    first_far_row = 2 ** 31 // (sumc * D)            # batch rows from here on lie past 2**31 elements
    assert first_far_row < B - 2
    rng = np.random.default_rng(5)
    pairs = [(int(rng.integers(first_far_row + 1, B)), int(rng.integers(H))) for _ in range(12)]
    pairs += [(B - 1, H - 1), (B - 1, 0), (first_far_row, int(np.argmax(sizes))), (0, 3)]
    for b, h in pairs:
        s0, n = int(start[h]), int(sizes[h])
        ref = decode_segments(q[b:b + 1, h:h + 1, 0].float().cpu().numpy(),
                              kc[b:b + 1, s0:s0 + n].float().cpu().numpy(),
                              vc[b:b + 1, s0:s0 + n].float().cpu().numpy(),
                              np.array([[0]]), np.array([[n]]), sm)[0, 0]
        got = out[b, 0, h].float().cpu().numpy().astype(np.float64)
        assert (np.abs(got - ref) <= ATOL + RTOL * np.abs(ref)).all(), (b, h)
    dense = mixture_of_sparse_attention(q[B - 2:], kc[B - 2:], vc[B - 2:], sm, head_start_index=hs[B - 2:],
                                        head_valid_length=hv[B - 2:], implementation="sdpa")
    torch.testing.assert_close(out[B - 2:].float(), dense.float(), rtol=RTOL, atol=ATOL)
    vc.fill_(1)
    ones = mixture_of_sparse_attention(q, kc, vc, sm, head_start_index=hs, head_valid_length=hv)
    assert (ones.float() - 1).abs().max().item() <= 1e-3


def test_append_and_rotary_append_over_2g_elements(dev):
    """Decode-step cache writes at B = 112: plain append and the fused rotary + append, against
    torch index ops on the whole tensors (cache_utils.py:1031-1054)."""
    from moa_amd import StaticCircularCache
    from moa_amd.kernels.rotary import apply_rotary_pos_emb
    B, H, D = 112, 32, 128
    cache_size, static_size = _plan(B, D)
    cache = StaticCircularCache([cache_size], static_size=[static_size], batch_size=B, head_dim=D,
                                device=dev, dtype=torch.float16)
    g = torch.Generator(device="cpu").manual_seed(7)
    circ = cache.circular_cache_size[0].cpu()
    off = torch.minimum((torch.rand(B, H, generator=g) * circ[None, :].float()).long(), circ[None, :] - 1)
    off[B - 1, :] = circ - 1      # the last batch row wraps on its next step
    cache.cache_update_index[0] = (cache.circular_cache_head_index[0].cpu()[None, :] + off).to(dev)
    cache.cache_valid_length[0] = cache.cache_max_length[0][None, :].expand(B, -1).contiguous().to(dev)
    cache._kv_len[0] = 16384
    z = torch.zeros(B, 1, H, D, dtype=torch.float16, device=dev).transpose(1, 2)
    cache.update(z, z, 0)
    kc_ref, vc_ref = cache.key_cache[0].clone(), cache.value_cache[0].clone()
    upd_ref = cache.cache_update_index[0].clone()
    ch = cache.circular_cache_head_index[0].to(dev)
    csz = cache.circular_cache_size[0].to(dev)
    bidx = torch.arange(B, device=dev)[:, None]
    gd = torch.Generator(device=dev).manual_seed(8)
    pos = torch.full((B, 1), 16385, device=dev)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, device=dev).float() / D))
    for step in range(3):
        qn = torch.randn(B, 1, H, D, generator=gd, device=dev, dtype=torch.float16).transpose(1, 2)
        kn = torch.randn(B, 1, H, D, generator=gd, device=dev, dtype=torch.float16).transpose(1, 2)
        vn = torch.randn(B, 1, H, D, generator=gd, device=dev, dtype=torch.float16).transpose(1, 2)
        if step == 1:
            cache.update(kn, vn, 0)
            k_written = kn
        else:
            ang = (pos + step).float()[:, :, None] * inv[None, None, :]
            emb = torch.cat([ang, ang], dim=-1)
            cos, sin = emb.cos().to(torch.float16), emb.sin().to(torch.float16)
            q_sep, k_written = apply_rotary_pos_emb(qn, kn, cos, sin)
            q_rot, _, _ = cache.rope_update(qn, kn, vn, cos, sin, 0)
            assert torch.equal(q_rot, q_sep), step
        kc_ref[bidx, upd_ref] = k_written[:, :, -1, :]
        vc_ref[bidx, upd_ref] = vn[:, :, -1, :]
        upd_ref = (upd_ref + 1 - ch[None, :]) % csz[None, :] + ch[None, :]
        assert torch.equal(cache.cache_update_index[0], upd_ref), step
        assert torch.equal(cache.key_cache[0], kc_ref), step
        assert torch.equal(cache.value_cache[0], vc_ref), step
    assert torch.equal(cache.cache_update_index[0][B - 1], ch + 3)


def test_prompt_insert_over_2g_elements(dev):
    """A 16384-token prompt for B = 112 (k, v: 7.5e9 elements each): closed-form ring contents in
    the first and the last batch row, and all batch rows equal (they get equal input)."""
    from moa_amd import StaticCircularCache
    B, H, D, N = 112, 32, 128, 16384
    cache_size, static_size = _plan(B, D)
    cache = StaticCircularCache([cache_size], static_size=[static_size], batch_size=B, head_dim=D,
                                device=dev, dtype=torch.float16)
    t = torch.arange(N, device=dev)
    row = torch.zeros(1, H, N, D, dtype=torch.float16, device=dev)
    row[..., 0] = (t // 128).to(torch.float16)
    row[..., 1] = (t % 128).to(torch.float16)
    row[..., 2] = torch.arange(H, device=dev, dtype=torch.float16)[None, :, None]
    k = row.repeat(B, 1, 1, 1)
    k[:, :, :, 3] = torch.arange(B, device=dev, dtype=torch.float16)[:, None, None]   # the batch row, exact in fp16
    del row
    cache.update(k, k, 0)
    kc = cache.key_cache[0]
    assert torch.equal(cache.value_cache[0], kc)
    assert torch.equal(kc[..., 3], torch.arange(B, device=dev, dtype=torch.float16)[:, None].expand(B, kc.shape[1]))
    assert torch.equal(kc[..., :3], kc[:1, :, :3].expand(B, -1, -1))
    tok = kc[B - 1, :, 0].long() * 128 + kc[B - 1, :, 1].long()
    for h in range(H):
        s, c = static_size[h], cache_size[h] - static_size[h]
        st = int(cache.head_index[0][h])
        expect = torch.empty(s + c, dtype=torch.long, device=dev)
        expect[:s] = torch.arange(s, device=dev)
        ring_tok = torch.arange(N - c, N, device=dev)
        expect[s + (ring_tok - s) % c] = ring_tok
        assert torch.equal(tok[st:st + s + c], expect), h
        assert (kc[B - 1, st:st + s + c, 2] == h).all()
    assert torch.equal(cache.cache_update_index[0][B - 1], cache.cache_update_index[0][0])
    assert torch.equal(cache.cache_valid_length[0].cpu(), torch.tensor(cache_size)[None, :].expand(B, -1))


def test_prefill_over_2g_elements(dev):
    """B = 68 at the benchmark's prefill shape (H = 32, N = 8192, D = 128, bf16): 2.28e9 elements per
    tensor.  V == 1 => O == 1 everywhere; the last batch row (and the first one past 2**31 elements)
    against dense masked attention evaluated with torch ops in fp32 on the GPU."""
    from moa_amd import mixture_of_sparse_attention
    from moa_amd.workloads import elastic_spans
    B, H, N, D = 68, 32, 8192, 128
    assert B * H * N * D > 2 ** 31
    gd = torch.Generator(device=dev).manual_seed(9)
    q = torch.randn(B, N, H, D, generator=gd, device=dev, dtype=torch.bfloat16).transpose(1, 2)
    k = torch.randn(B, N, H, D, generator=gd, device=dev, dtype=torch.bfloat16).transpose(1, 2)
    v = torch.randn(B, N, H, D, generator=gd, device=dev, dtype=torch.bfloat16).transpose(1, 2)
    spans = elastic_spans(H, N, seed=0)
    ns, nl = [1] * H, [s // 64 for s in spans]
    sink = torch.tensor([64] * H, dtype=torch.int64, device=dev)
    local = torch.tensor(spans, dtype=torch.int64, device=dev)
    sm = D ** -0.5
    out = mixture_of_sparse_attention(q, k, v, sm, sink_size=sink, local_size=local)   # [B, N, H, D]
    assert out.shape == (B, N, H, D)
    for b in (B - 1, 2 ** 31 // (H * N * D) + 1):
        for h0 in range(0, H, 8):
            mask = torch.stack([torch.from_numpy(moa_token_mask(N, ns[h], nl[h])) for h in range(h0, h0 + 8)]).to(dev)
            sl = (slice(b, b + 1), slice(h0, h0 + 8))
            got = out[b:b + 1, :, h0:h0 + 8].transpose(1, 2)
            # bf16: against the attention with the weights rounded where the kernel rounds them, and, outliers
            # counted, against the unrounded one (see prefill_checks.py)
            close_stated(got, masked_attention_gpu(q[sl], k[sl], v[sl], mask, sm, torch.bfloat16), (b, h0))
            close_counted(got, masked_attention_gpu(q[sl], k[sl], v[sl], mask, sm),
                          masked_attention_gpu(q[sl], k[sl], v[sl].abs(), mask, sm), ("over 2g", b, h0))
    del out
    v.fill_(1)
    ones = mixture_of_sparse_attention(q, k, v, sm, sink_size=sink, local_size=local)
    assert (ones.float().sub_(1).abs_().max().item()) <= 8e-3   # bf16 output spacing near 1
