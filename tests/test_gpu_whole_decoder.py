"""The two end-to-end configurations as WHOLE decoders at full size: embedding, per layer RMSNorm +
attention + RMSNorm + SwiGLU, final norm, LM head, greedy decoding, random bf16 weights
(LlamaMixtureForCausalLM; the reference's model forward is MoA/models/llama/modeling_llama.py:52-204 and
its efficiency script drives prompt + greedy steps the same way, scripts/evaluate/effieicency_test.py:548-562).

  7B shape : 32 layers, hidden 4096, 32 heads, FFN 11008, vocab 32000, B=8, 16384 prompt ids, 256 steps
  70B shape: 80 layers, hidden 8192, 64 query heads on 8 kv heads, FFN 28672, vocab 128256, B=4,
             32768 prompt ids, alpha in [256, 8192], 128 steps

Checked: finite logits throughout; ring pointers, valid lengths, masks and lengths of EVERY layer against
the closed form after prompt + steps; the last four greedy steps replayed from a HIP graph on a copy of
the caches give the logits, the tokens and the cache contents of eager execution, bit for bit.  What the
attention kernels compute at these sizes is checked against the oracle in test_gpu_configs.py."""
import copy

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _run(dev, L, hidden, Hq, Hkv, ffn, vocab, B, N, steps, alpha_range, n_graph=4):
    from moa_amd.models.llama.modeling_llama import LlamaMixtureForCausalLM
    from moa_amd.workloads import elastic_spans

    D, dtype = 128, torch.bfloat16
    model = LlamaMixtureForCausalLM(L, hidden, Hq, Hkv, ffn, vocab, head_dim=D, dtype=dtype, device=dev)
    gen = torch.Generator(device=dev).manual_seed(0)
    for p in model.parameters():
        if p.dim() > 1:
            p.data.normal_(0.0, 0.02, generator=gen)
    plan = {"alphas": [[64 + s for s in elastic_spans(Hkv, N, seed=l, alpha_range=alpha_range)] for l in range(L)],
            "betas": [[0.0] * Hkv for _ in range(L)]}
    model.set_mixture_of_attention(plan, permute_head=True, moa_max_new_token=steps)
    ids = torch.randint(0, vocab, (B, N), generator=torch.Generator().manual_seed(5)).to(dev)

    logits, cache = model(ids)
    assert logits.shape == (B, vocab)
    finite = torch.isfinite(logits.float()).all()
    tok = logits.argmax(-1, keepdim=True)
    del logits, ids
    eager_logits, eager_toks = [], []
    cache_g = tok_g = None
    for t in range(steps):
        if t == steps - n_graph:
            cache_g = copy.deepcopy(cache)     # to be driven by graph replays from here on
            tok_g = tok.clone()
        logits, _ = model(tok, cache, position_ids=torch.full((1, 1), N + t, device=dev, dtype=torch.int64))
        finite = finite & torch.isfinite(logits.float()).all()
        tok = logits.argmax(-1, keepdim=True)
        if t >= steps - n_graph:
            eager_logits.append(logits.clone())
            eager_toks.append(tok.clone())
    torch.cuda.synchronize()
    assert bool(finite)
    total = N + steps

    # ---- every layer's ring bookkeeping against the closed form ----------------------------------
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

    # ---- the last steps again, replayed from a HIP graph on the copied caches --------------------
    tok_s = tok_g.clone()
    pos_s = torch.full((1, 1), N + steps - n_graph, device=dev, dtype=torch.int64)

    def step():
        lg, _ = model(tok_s, cache_g, position_ids=pos_s)
        tok_s.copy_(lg.argmax(-1, keepdim=True))
        pos_s.add_(1)
        return lg

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        lg_s = step()
    for i in range(n_graph):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(lg_s, eager_logits[i]), i
        assert torch.equal(tok_s, eager_toks[i]), i
    for l in range(L):
        assert torch.equal(cache_g.key_cache[l], cache.key_cache[l]), l
        assert torch.equal(cache_g.value_cache[l], cache.value_cache[l]), l
        assert torch.equal(cache_g.cache_update_index[l], cache.cache_update_index[l]), l
        assert torch.equal(cache_g.cache_valid_length[l], cache.cache_valid_length[l]), l


def test_7b_whole_decoder_at_full_size(dev):
    _run(dev, L=32, hidden=4096, Hq=32, Hkv=32, ffn=11008, vocab=32000, B=8, N=16384, steps=256,
         alpha_range=(64.0, 2048.0))
    torch.cuda.empty_cache()


def test_70b_whole_decoder_at_full_size(dev):
    free, _ = torch.cuda.mem_get_info(dev)
    if free < 200 * 2 ** 30:
        pytest.skip("needs about 200 GB of free device memory (141 GB of weights)")
    _run(dev, L=80, hidden=8192, Hq=64, Hkv=8, ffn=28672, vocab=128256, B=4, N=32768, steps=128,
         alpha_range=(256.0, 8192.0))
    torch.cuda.empty_cache()
