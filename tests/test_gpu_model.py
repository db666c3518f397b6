"""The whole-decoder harness (moa_amd.models.llama.modeling_llama.LlamaMixtureForCausalLM) on the
GPU: properties that hold for any weights.

* With rings that hold every token, decoding token by token must give the logits of a one-shot
  prompt pass over the same tokens (prefill kernel vs. cache insert + append + decode kernels, both
  dense causal then).
* Grouped-query attention equals multi-head attention whose k/v projections repeat each kv head
  (the reference's way to run such models, scripts/helper/gqa_to_mha.py).
* Head permutation leaves the model's function unchanged (reference modeling_llama.py:373-398).
"""
import copy

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _model(dev, heads=4, kv_heads=2, seed=0, dtype=torch.float16):
    from moa_amd.models.llama.modeling_llama import LlamaMixtureForCausalLM
    torch.manual_seed(seed)
    m = LlamaMixtureForCausalLM(num_layers=2, hidden_size=256, num_heads=heads, num_key_value_heads=kv_heads,
                                intermediate_size=512, vocab_size=1000, head_dim=64, dtype=dtype, device=dev)
    for p in m.parameters():
        if p.dim() > 1:
            p.data.normal_(0.0, 0.05)
    return m


def _plan(layers, kv_heads, alpha):
    return {"alphas": [[alpha] * kv_heads for _ in range(layers)], "betas": [[0.0] * kv_heads for _ in range(layers)]}


@pytest.mark.parametrize("heads,kv_heads", [(4, 4), (4, 2), (4, 1), (6, 2)])
def test_incremental_decoding_matches_one_shot_prompt(dev, heads, kv_heads):
    m = _model(dev, heads=heads, kv_heads=kv_heads)
    m.set_mixture_of_attention(_plan(2, kv_heads, 4096.0), moa_max_new_token=64)   # rings hold everything
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, 1000, (2, 137), generator=g).to(dev)
    new = m.generate_greedy(ids, 6)
    assert new.shape == (2, 6)
    logits, cache = m(ids)
    for t in range(6):
        assert torch.equal(logits.argmax(-1), new[:, t])
        one_shot, _ = m(torch.cat([ids, new[:, :t]], dim=1))
        torch.testing.assert_close(logits.float(), one_shot.float(), rtol=2e-2, atol=2e-2)
        logits, cache = m(new[:, t:t + 1], cache)
    assert cache.get_seq_length() == 137 + 6


def test_grouped_query_equals_repeated_kv_heads(dev):
    gqa = _model(dev, heads=4, kv_heads=2, seed=3)
    mha = _model(dev, heads=4, kv_heads=4, seed=3)
    mha.load_state_dict({k: v for k, v in gqa.state_dict().items() if "k_proj" not in k and "v_proj" not in k},
                        strict=False)
    for lg, lm in zip(gqa.layers, mha.layers):
        for name in ("k_proj", "v_proj"):
            w = getattr(lg.self_attn, name).weight.data.view(2, 64, 256)
            getattr(lm.self_attn, name).weight.data.copy_(w.repeat_interleave(2, dim=0).reshape(256, 256))
    alphas = [[192.0, 448.0], [320.0, 128.0]]
    gqa.set_mixture_of_attention({"alphas": alphas, "betas": [[0.0, 0.0]] * 2}, moa_max_new_token=8)
    mha.set_mixture_of_attention({"alphas": [[a for a in row for _ in range(2)] for row in alphas],
                                  "betas": [[0.0] * 4] * 2}, moa_max_new_token=8)
    ids = torch.randint(0, 1000, (2, 700), generator=torch.Generator().manual_seed(4)).to(dev)
    lg, cg = gqa(ids)
    lm, cm = mha(ids)
    torch.testing.assert_close(lg.float(), lm.float(), rtol=2e-2, atol=2e-2)
    for _ in range(4):
        nxt = lg.argmax(-1, keepdim=True)
        lg, cg = gqa(nxt, cg)
        lm, cm = mha(nxt, cm)
        torch.testing.assert_close(lg.float(), lm.float(), rtol=2e-2, atol=2e-2)


def test_head_permutation_keeps_the_function(dev):
    a = _model(dev, heads=4, kv_heads=4, seed=5)
    b = copy.deepcopy(a)
    plan = {"alphas": [[448.0, 128.0, 448.0, 128.0], [256.0, 256.0, 640.0, 128.0]], "betas": [[0.0] * 4] * 2}
    a.set_mixture_of_attention(plan, permute_head=False, moa_max_new_token=8)
    b.set_mixture_of_attention(plan, permute_head=True, moa_max_new_token=8)
    assert b.moa_config["alphas"][0] != plan["alphas"][0]          # the heads did move
    ids = torch.randint(0, 1000, (1, 900), generator=torch.Generator().manual_seed(6)).to(dev)
    la, ca = a(ids)
    lb, cb = b(ids)
    torch.testing.assert_close(la.float(), lb.float(), rtol=2e-2, atol=2e-2)
    for _ in range(3):
        nxt = la.argmax(-1, keepdim=True)
        la, ca = a(nxt, ca)
        lb, cb = b(nxt, cb)
        torch.testing.assert_close(la.float(), lb.float(), rtol=2e-2, atol=2e-2)
