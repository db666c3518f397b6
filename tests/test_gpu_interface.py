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


def test_generate_on_the_patched_model(dev, capsys):
    """transformers' own ``generate`` drives the patched model, as the reference's scripts do
    (scripts/evaluate/chat_demo.py:72, batch_inference.py:89, retrieval_evaluate.py:53): it hands over
    its own empty cache, which the model forward replaces by a StaticCircularCache at the prompt
    (reference modeling_llama.py:93-112) and gets back in the outputs.  Greedy tokens equal those of the
    step-by-step loop on the same model; ``moa_verbose`` prints the cache summary when the cache is built
    (:95-104)."""
    from moa_amd import StaticCircularCache
    from moa_amd.models.interface import update_model_function
    moa = update_model_function(_hf_model(dev, 4, 2, seed=11), "lmsys/vicuna-7b-v1.5-16k")
    plan = {"alphas": [[192.0, 256.0], [128.0, 192.0]], "betas": [[0.0, 0.0]] * 2}
    moa.model.set_mixture_of_attention(plan, permute_head=True, moa_verbose=True, moa_max_new_token=16)
    ids = torch.randint(0, 1000, (2, 300), generator=torch.Generator().manual_seed(3)).to(dev)
    new = 6
    with torch.no_grad():
        got = moa.generate(ids, max_new_tokens=new, do_sample=False, pad_token_id=0)
    assert got.shape == (2, 300 + new) and torch.equal(got[:, :300], ids)
    text = capsys.readouterr().out
    assert "Cache configuration" in text and "cache_size" in text       # moa_verbose
    with torch.no_grad():
        out = moa(input_ids=ids, use_cache=True)
        cache = out.past_key_values
        assert isinstance(cache, StaticCircularCache)
        want = []
        for _ in range(new):
            nxt = out.logits[:, -1].argmax(-1, keepdim=True)
            want.append(nxt)
            out = moa(input_ids=nxt, past_key_values=cache, use_cache=True)
    assert torch.equal(got[:, 300:], torch.cat(want, dim=1))
    # a left-padded batch goes through generate as well (mask with zeros, per-row positions): the rings
    # hold the valid tokens only
    mask = torch.ones(2, 300, dtype=torch.int64, device=dev)
    mask[1, :100] = 0
    moa.model.moa_verbose = False
    with torch.no_grad():
        res = moa.generate(ids, attention_mask=mask, max_new_tokens=3, do_sample=False, pad_token_id=0,
                           return_dict_in_generate=True)
    assert res.sequences.shape == (2, 303)
    cache = res.past_key_values
    assert isinstance(cache, StaticCircularCache)
    # 3 tokens generated, the last of them not yet fed back: prompt + 2 positions seen
    assert cache.get_seq_length() == 302
    sizes = cache.cache_max_length[0].tolist()
    assert cache.cache_valid_length[0].tolist() == [[min(302, c) for c in sizes], [min(202, c) for c in sizes]]


def test_model_forward_arguments(dev):
    """return_dict=False, output_hidden_states, cache_position and output_attentions behave as in the
    reference's model forward (modeling_llama.py:64-70,114-129,183-198)."""
    from moa_amd.models.interface import update_model_function
    moa = update_model_function(_hf_model(dev, 4, 4, seed=5), "llama")
    moa.model.set_mixture_of_attention({"alphas": [[512.0] * 4] * 2, "betas": [[0.0] * 4] * 2}, last_hidden_only=False)
    ids = torch.randint(0, 1000, (1, 130), generator=torch.Generator().manual_seed(4)).to(dev)
    with torch.no_grad():
        a = moa.model(input_ids=ids, use_cache=True, output_hidden_states=True)
        assert a.last_hidden_state.shape == (1, 130, 256) and len(a.hidden_states) == 3
        b = moa.model(input_ids=ids, use_cache=True, return_dict=False)
        assert isinstance(b, tuple) and torch.equal(b[0], a.last_hidden_state)
        c = moa.model(input_ids=ids, use_cache=True, cache_position=torch.arange(130, device=dev))
        assert torch.equal(c.last_hidden_state, a.last_hidden_state)
        with pytest.raises(NotImplementedError):
            moa.model(input_ids=ids, output_attentions=True)


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
