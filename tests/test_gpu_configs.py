"""The two end-to-end configurations at FULL size on the attention path of a decoder
(moa_amd.models.llama.modeling_llama.LlamaMixtureAttentionStack: projections, rotary embedding, cache,
sparse prefill, ring decode; norms, MLPs and LM head are not on the path):

  * 7B shape:  32 layers, hidden 4096, 32 heads of 128, bf16, batch 8, a 16384-token prompt, then 256
    decode steps; every (layer, head) has its own span from the elastic rule (alpha in [64, 2048]).
  * 70B shape: 80 layers, hidden 8192, 64 query heads on 8 kv heads of 128 (grouped-query attention,
    spans per kv head), bf16, batch 4, a 32768-token prompt, spans with alpha in [256, 8192], then 128
    decode steps.

No CPU oracle can redo these sizes whole, so the checks are of three kinds:
  (1) closed forms over EVERY layer: ring pointers, valid lengths, masks after prompt + steps;
  (2) two sampled layers, bit-exact: every cache row holds the token the ring definition says
      (slot of token t: start + t for t < s, else start + s + (t - s) mod c; kept tokens are
      {0..s-1} U {p-c+1..p}), V rows against the recorded projections, K rows against torch's own
      evaluation of the rotary embedding of the recorded projections;
  (3) the same layers, arithmetic: sampled (batch row, kv head) rings of the last decode step against
      the CPU oracle (decode_segments, incl. the largest ring); the smallest- and largest-span kv heads
      of the prompt pass against dense masked attention in fp32 on the GPU; V == 1 => O == 1 in
      prefill and decode; the last decode steps replayed from a HIP graph equal the eager ones bit
      for bit (outputs and all caches).
Tolerances as everywhere: 2e-3 + 1e-2 |ref| (see prefill_checks.py for the bf16 weight rounding)."""
import copy

import numpy as np
import pytest
import torch

from oracle.moa_oracle import decode_segments, moa_token_mask
from prefill_checks import ATOL, RTOL, close_counted, close_stated, masked_attention_gpu

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _rotate_half(x):
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def _mask_rows(N, ns, nl, r0, r1, dev):
    """Rows [r0, r1) of the oracle's moa_token_mask(N, ns, nl), built on the GPU (the whole mask of a
    32768-token prompt is 1 GiB); keys up to r1 only, the rest is causally dead."""
    i = torch.arange(r0, r1, device=dev)[:, None]
    j = torch.arange(r1, device=dev)[None, :]
    return (j <= i) & ((j // 64 < ns) | (j // 64 >= i // 64 + 1 - nl))


def test_mask_rows_is_the_oracle_mask(dev):
    for N, ns, nl in ((700, 1, 3), (1000, 0, 1), (640, 2, 0), (900, 1, 99)):
        want = torch.from_numpy(moa_token_mask(N, ns, nl))
        for r0, r1 in ((0, 256), (256, N), (0, N)):
            assert torch.equal(_mask_rows(N, ns, nl, r0, r1, dev).cpu(), want[r0:r1, :r1])
            assert not want[r0:r1, r1:].any()


class _Recorder:
    """Wraps the cache's rope_update and the layer's attention call for the sampled layers: keeps the
    un-rotated k and v of every token, and q / output of the prompt pass and of every decode step."""

    def __init__(self, cache, layers):
        self.layers = set(layers)
        self.k_raw = {l: [] for l in layers}
        self.v_raw = {l: [] for l in layers}
        self.prefill = {}
        self.decode = {l: [] for l in layers}
        self.current = None
        self.cache = cache
        self._rope_update = cache.rope_update
        cache.rope_update = self.rope_update

    def rope_update(self, q, k, v, cos, sin, layer_idx, attention_mask=None):
        self.current = layer_idx
        if layer_idx in self.layers:
            self.k_raw[layer_idx].append(k.clone())
            self.v_raw[layer_idx].append(v.clone())
        return self._rope_update(q, k, v, cos, sin, layer_idx, attention_mask)

    def attention(self, real):
        def wrapped(query, key, value, **kw):
            out = real(query, key, value, **kw)
            l = self.current
            if l in self.layers:
                if query.shape[-2] > 1:
                    self.prefill[l] = (query, key, value, out)
                else:
                    self.decode[l].append((query.clone(), out.clone()))
            return out
        return wrapped


def _run_config(dev, monkeypatch, L, Hq, Hkv, B, N, steps, alpha_range, sampled, row_block):
    from moa_amd import mixture_of_sparse_attention
    from moa_amd.models.llama import modeling_llama
    from moa_amd.models.llama.modeling_llama import LlamaMixtureAttentionStack, rotary_cos_sin
    from moa_amd.workloads import elastic_spans

    D, dtype = 128, torch.bfloat16
    G = Hq // Hkv
    hidden = Hq * D
    torch.manual_seed(0)
    model = LlamaMixtureAttentionStack(L, hidden, Hq, num_key_value_heads=Hkv, head_dim=D, dtype=dtype, device=dev)
    for p in model.parameters():
        p.data.normal_(0.0, hidden ** -0.5)
    for layer in model.layers:       # the stack has no norms: small output projections keep the residual stream O(1)
        layer.o_proj.weight.data.mul_(L ** -0.5)
    plan = {"alphas": [[64 + s for s in elastic_spans(Hkv, N, seed=l, alpha_range=alpha_range)] for l in range(L)],
            "betas": [[0.0] * Hkv for _ in range(L)]}
    model.set_mixture_of_attention(plan, permute_head=True, moa_max_new_token=steps)
    cache = model.new_cache(B, N, dev)
    rec = _Recorder(cache, sampled)
    monkeypatch.setattr(modeling_llama, "mixture_of_sparse_attention", rec.attention(mixture_of_sparse_attention))

    gen = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn(B, N, hidden, generator=gen, device=dev, dtype=dtype)
    h = model(x, torch.arange(N, device=dev)[None, :], cache)
    assert torch.isfinite(h.float()).all()
    del x, h
    xs = [torch.randn(B, 1, hidden, generator=gen, device=dev, dtype=dtype) for _ in range(steps)]
    n_graph = 4
    eager_out = []
    cache_g = None
    for t in range(steps):
        if t == steps - n_graph:
            # a second copy of all caches, to be driven by graph replays from here on
            del cache.rope_update                         # (the instance attribute: deepcopy must not copy the recorder)
            cache_g = copy.deepcopy(cache)
            cache.rope_update = rec.rope_update
        y = model(xs[t], torch.full((1, 1), N + t, device=dev, dtype=torch.int64), cache)
        if t >= steps - n_graph:
            eager_out.append(y)
    torch.cuda.synchronize()
    total = N + steps
    p_last = total - 1

    # ---- (1) closed forms over every layer -------------------------------------------------------
    for l in range(L):
        size = cache.cache_max_length[l].cpu().numpy()
        s = cache.static_cache_size[l].cpu().numpy()
        c = size - s
        start = cache.head_index[l].cpu().numpy()[:-1]
        assert (c > 0).all() and (size <= total).all()
        want_ptr = start + s + (total - s) % c
        assert np.array_equal(cache.cache_update_index[l].cpu().numpy(), np.broadcast_to(want_ptr, (B, Hkv))), l
        assert np.array_equal(cache.cache_valid_length[l].cpu().numpy(), np.broadcast_to(size, (B, Hkv))), l
        assert bool((cache.mask_cache[l] == 1).all()), l
        assert cache.get_seq_length(l) == total

    # ---- (2) sampled layers: which token sits in which row, bit for bit ---------------------------
    pos = torch.arange(total, device=dev)[None, :]
    cos, sin = rotary_cos_sin(pos, D, dtype)                          # [1, total, D]
    for l in sampled:
        v_hist = torch.cat(rec.v_raw[l], dim=2)                       # [B, Hkv, total, D]
        k_hist = torch.cat(rec.k_raw[l], dim=2)
        assert v_hist.shape == (B, Hkv, total, D)
        k_rot = k_hist * cos[:, None] + _rotate_half(k_hist) * sin[:, None]   # torch's evaluation, bf16 per op
        size = cache.cache_max_length[l].tolist()
        s_l = cache.static_cache_size[l].tolist()
        start = cache.head_index[l].tolist()
        for hk in range(Hkv):
            s, c = s_l[hk], size[hk] - s_l[hk]
            kept = list(range(s)) + list(range(p_last - c + 1, p_last + 1))
            assert len(kept) == size[hk]
            tok = torch.tensor(kept, device=dev)
            slot = torch.where(tok < s, tok, s + (tok - s) % c) + start[hk]
            assert slot.unique().numel() == size[hk]                  # the kept tokens fill the ring exactly
            assert torch.equal(cache.value_cache[l][:, slot], v_hist[:, hk, tok]), (l, hk)
            assert torch.equal(cache.key_cache[l][:, slot], k_rot[:, hk, tok]), (l, hk)
        del v_hist, k_hist, k_rot

    # ---- (3a) last decode step of the sampled layers against the CPU oracle ------------------------
    name = None if G == 1 else "bf16"
    for l in sampled:
        q_last, o_last = rec.decode[l][-1]                            # [B, Hq, 1, D], [B, 1, Hq, D]
        size = cache.cache_max_length[l].tolist()
        picks = sorted({int(np.argmax(size)), int(np.argmin(size)), Hkv // 2})
        hs = cache.cache_head_start_index[l].cpu().numpy()
        hv = cache.cache_valid_length[l].cpu().numpy()
        for b in (0, B - 1):
            for hk in picks:
                seg = slice(hs[b, hk], hs[b, hk] + hv[b, hk])
                kc = cache.key_cache[l][b, seg].float().cpu().numpy()[None]
                vc = cache.value_cache[l][b, seg].float().cpu().numpy()[None]
                qn = q_last[b, hk * G:(hk + 1) * G, 0].float().cpu().numpy()[None]
                got = o_last[b, 0, hk * G:(hk + 1) * G][None]
                one = (np.array([[0]]), np.array([[hv[b, hk]]]))
                ref = decode_segments(qn, kc, vc, *one, D ** -0.5, group=G, p_dtype=name)
                close_stated(got, torch.from_numpy(ref), ("decode", l, b, hk, size[hk]))
                if name is not None:
                    close_counted(got, torch.from_numpy(decode_segments(qn, kc, vc, *one, D ** -0.5, group=G)),
                                  torch.from_numpy(decode_segments(qn, kc, vc, *one, D ** -0.5, group=G, abs_v=True)),
                                  ("decode, exact", l, b, hk))
        # V == 1 => O == 1 over the real keys of the step
        ones = mixture_of_sparse_attention(q_last, cache.key_cache[l], torch.ones_like(cache.value_cache[l]),
                                           D ** -0.5, head_start_index=cache.cache_head_start_index[l],
                                           head_valid_length=cache.cache_valid_length[l])
        assert (ones.float() - 1).abs().max().item() <= 8e-3          # bf16 output spacing near 1

    # ---- (3b) the prompt pass of the sampled layers ------------------------------------------------
    for l in sampled:
        q, k, v, out = rec.prefill[l]                                 # [B,Hq,N,D], [B,Hkv,N,D] x2, [B,N,Hq,D]
        ns = (cache.static_cache_size[l] // 64).tolist()
        nl = (cache.circular_cache_size[l] // 64).tolist()
        ones = mixture_of_sparse_attention(q, k, torch.ones_like(v), D ** -0.5,
                                           sink_size=cache.static_cache_size[l],
                                           local_size=cache.circular_cache_size[l])
        assert (ones.float() - 1).abs().max().item() <= 8e-3
        del ones
        b = B - 1
        outside = elements = 0
        for hk in sorted({int(np.argmin(nl)), int(np.argmax(nl))}):
            hq = slice(hk * G, (hk + 1) * G)
            for r0 in range(0, N, row_block):
                r1 = min(N, r0 + row_block)
                rows = slice(r0, r1)
                m = _mask_rows(N, ns[hk], nl[hk], r0, r1, dev)[None].expand(G, -1, -1)
                kk = k[b:b + 1, hk:hk + 1, :r1].expand(1, G, r1, D)
                vv = v[b:b + 1, hk:hk + 1, :r1].expand(1, G, r1, D)
                qq = q[b:b + 1, hq, rows]
                got = out[b:b + 1, rows, hq].transpose(1, 2)
                close_stated(got, masked_attention_gpu(qq, kk, vv, m, D ** -0.5, torch.bfloat16),
                             ("prefill, weights rounded", l, hk, r0))
                outside += close_counted(got, masked_attention_gpu(qq, kk, vv, m, D ** -0.5),
                                         masked_attention_gpu(qq, kk, vv.abs(), m, D ** -0.5), ("prefill", l, hk, r0))
                elements += got.numel()
        assert outside <= 1e-5 * elements, (outside, elements)
    rec.prefill.clear()

    # ---- (3c) the last steps again, replayed from a HIP graph --------------------------------------
    x_static = xs[steps - n_graph].clone()
    pos_static = torch.full((1, 1), N + steps - n_graph, device=dev, dtype=torch.int64)
    monkeypatch.setattr(modeling_llama, "mixture_of_sparse_attention", mixture_of_sparse_attention)

    def step():
        y = model(x_static, pos_static, cache_g)
        pos_static.add_(1)
        return y

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_static = step()
    for i in range(n_graph):
        x_static.copy_(xs[steps - n_graph + i])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_static, eager_out[i]), i
    for l in range(L):
        assert torch.equal(cache_g.key_cache[l], cache.key_cache[l]), l
        assert torch.equal(cache_g.value_cache[l], cache.value_cache[l]), l
        assert torch.equal(cache_g.cache_update_index[l], cache.cache_update_index[l]), l
        assert torch.equal(cache_g.cache_valid_length[l], cache.cache_valid_length[l]), l


def test_7b_shape_end_to_end_at_full_size(dev, monkeypatch):
    _run_config(dev, monkeypatch, L=32, Hq=32, Hkv=32, B=8, N=16384, steps=256, alpha_range=(64.0, 2048.0),
                sampled=(0, 31), row_block=4096)


def test_70b_grouped_query_shape_end_to_end_at_full_size(dev, monkeypatch):
    _run_config(dev, monkeypatch, L=80, Hq=64, Hkv=8, B=4, N=32768, steps=128, alpha_range=(256.0, 8192.0),
                sampled=(0, 79), row_block=2048)
