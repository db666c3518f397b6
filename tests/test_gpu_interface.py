"""update_model_function / set_mixture_of_attention on a real transformers Llama (the installed release,
random weights, no download): the way the reference's scripts switch a loaded model to the MoA attention
path (MoA/models/interface.py:3-28, scripts/evaluate/effieicency_test.py:335-343).

With windows that cover the whole sequence the MoA path is plain causal attention, so the patched model
must reproduce the unpatched model's logits (transformers' own attention and rotary embedding): in the
prompt pass, in token-by-token decoding through the StaticCircularCache, with and without head permutation,
with grouped-query attention."""
import copy

import pytest
import torch

pytestmark = pytest.mark.gpu

transformers = pytest.importorskip("transformers")


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _hf_model(dev, heads, kv_heads, seed):
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(seed)
    cfg = LlamaConfig(hidden_size=heads * 64, num_attention_heads=heads, num_key_value_heads=kv_heads,
                      num_hidden_layers=2, intermediate_size=512, vocab_size=1000, max_position_embeddings=4096)
    cfg._attn_implementation = "eager"
    return LlamaForCausalLM(cfg).to(dev, torch.float16).eval()


@pytest.mark.parametrize("heads,kv_heads,permute", [(4, 4, False), (4, 4, True), (4, 2, True)])
def test_patched_transformers_llama_matches_dense_attention(dev, heads, kv_heads, permute):
    from moa_amd import StaticCircularCache
    from moa_amd.models.interface import update_model_function
    ref = _hf_model(dev, heads, kv_heads, seed=7)
    moa = copy.deepcopy(ref)
    moa = update_model_function(moa, "lmsys/vicuna-7b-v1.5-16k")
    # distinct (alpha, beta) pairs per head so that the permutation moves heads; all windows cover the sequence
    plan = {"alphas": [[4096.0 + 64 * ((kv_heads - 1 - h + l) % kv_heads) for h in range(kv_heads)] for l in range(2)],
            "betas": [[0.0] * kv_heads for _ in range(2)]}
    moa.model.set_mixture_of_attention(plan, permute_head=permute, moa_max_new_token=64)
    if permute:
        assert moa.model.moa_config["alphas"][0] != plan["alphas"][0]
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, 1000, (2, 300), generator=g).to(dev)
    with torch.no_grad():
        want = ref(input_ids=ids).logits[:, -1]
        out = moa(input_ids=ids, use_cache=True)
    cache = out.past_key_values
    assert isinstance(cache, StaticCircularCache) and cache.get_seq_length() == 300
    assert out.logits.shape == (2, 1, 1000)                  # last_hidden_only: the lm_head sees one position
    torch.testing.assert_close(out.logits[:, -1].float(), want.float(), rtol=2e-2, atol=2e-2)
    seq = ids
    for _ in range(4):
        nxt = out.logits[:, -1].argmax(-1, keepdim=True)
        seq = torch.cat([seq, nxt], dim=1)
        with torch.no_grad():
            out = moa(input_ids=nxt, past_key_values=cache, use_cache=True)
            want = ref(input_ids=seq).logits[:, -1]
        assert out.past_key_values is cache
        torch.testing.assert_close(out.logits[:, -1].float(), want.float(), rtol=2e-2, atol=2e-2)
    assert cache.get_seq_length() == 304


def test_sparse_plan_runs_and_keeps_only_the_rings(dev):
    """A real sparse plan on the patched model: the cache holds sink + window rows per head, not the
    sequence, and decoding continues past the ring size."""
    from moa_amd.models.interface import update_model_function
    moa = update_model_function(_hf_model(dev, 4, 2, seed=9), "meta-llama/Llama-2-7b")
    moa.model.set_mixture_of_attention({"alphas": [[128.0, 256.0], [192.0, 128.0]], "betas": [[0.0, 0.0]] * 2},
                                       permute_head=True, moa_max_new_token=8)
    ids = torch.randint(0, 1000, (1, 700), generator=torch.Generator().manual_seed(2)).to(dev)
    with torch.no_grad():
        out = moa(input_ids=ids, use_cache=True)
        cache = out.past_key_values
        assert cache.layer_cache_size == [128 + 256, 128 + 192]
        for _ in range(5):
            out = moa(input_ids=out.logits[:, -1].argmax(-1, keepdim=True), past_key_values=cache, use_cache=True)
    assert torch.isfinite(out.logits.float()).all()
    assert cache.cache_valid_length[0].tolist() == [[128, 256]]


def test_unknown_model_names_are_refused():
    from moa_amd.models.interface import update_model_function
    with pytest.raises(NotImplementedError):
        update_model_function(object(), "mistralai/Mistral-7B")


@pytest.mark.parametrize("mode", ["prefill", "decode", "whole"])
def test_efficiency_cli_modes(dev, mode, golden_dir):
    """python -m moa_amd.efficiency_test: the reference's three test modes and printed figures
    (scripts/evaluate/effieicency_test.py:548-562), here on the tiny shape."""
    import io
    from moa_amd import efficiency_test
    args = efficiency_test.parse_args(["--prefill_len", "300", "--decode_len", "5", "--batch_size", "2", "--num_iters", "2",
                                       "--model_name", "tiny-llama", "--test_mode", mode, "--cuda_event", "--cuda_cache"])
    out = io.StringIO()
    res = efficiency_test.run_model(args, out=out)
    text = out.getvalue()
    assert "input_shape: (2, 300)" in text and "Start testing" in text and "Elapsed time:" in text and "per iter:" in text
    assert res["per_iter_ms"] == pytest.approx(res["elapsed_ms"] / 2)
    if mode == "prefill":
        assert res["per_token_ms"] == pytest.approx(res["elapsed_ms"] / 2 / 2 / 300)
    if mode == "decode":
        assert "throughput:" in text
        assert res["throughput_tokens_per_s"] == pytest.approx(2 * 5 * 2 / (res["elapsed_ms"] / 1000))
    if mode == "whole":
        assert "iter 1 done" in text
    assert res["max_memory_mb"] > 0
