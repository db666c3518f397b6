"""The PRODUCT's copies of the plan -> cache-size rule and of the cache constructor
(moa_amd.attention.cache_utils), on the CPU, against the vectors the reference's own code wrote
(tests/golden/cache_update_vectors.json; made by tests/golden/make_cache_vectors.py) and against the
oracle's copies.  Neither needs a GPU: the rule is host arithmetic and the constructor only lays out
index tensors (reference: MoA/attention/cache_utils.py:1183-1239 and :698-769)."""
import json
import os

import numpy as np
import pytest
import torch

from moa_amd.attention.cache_utils import StaticCircularCache, moa_config_to_cache_config
from oracle import moa_oracle


@pytest.fixture(scope="module")
def golden(golden_dir):
    return json.load(open(os.path.join(golden_dir, "cache_update_vectors.json")))


def test_plan_rule_single_heads(golden):
    rows = [p for p in golden["plans"] if "alpha" in p]
    assert len(rows) == 7
    for p in rows:
        plan = {"alphas": [[p["alpha"]]], "betas": [[p["beta"]]]}
        r = moa_config_to_cache_config(plan, p["seq_len"], p["max_new_token"], verbose=False)
        assert r == {"cache_size": [[p["cache_size"]]], "static_size": [[p["static_size"]]]}, p
        assert r == moa_oracle.moa_config_to_cache_config(plan, p["seq_len"], p["max_new_token"])


def _check_rows(plan, rows):
    for p in rows:
        r = moa_config_to_cache_config(plan, p["seq_len"], p["max_new_token"], verbose=False)
        assert r["cache_size"][0] == p["cache_size_layer0"]
        assert r["cache_size"][-1] == p["cache_size_last"]
        assert int(np.sum(r["cache_size"])) == p["cache_size_sum"]
        assert int(np.sum(r["static_size"])) == p["static_size_sum"]
        assert r == moa_oracle.moa_config_to_cache_config(plan, p["seq_len"], p["max_new_token"])


def test_plan_rule_shipped_vicuna_7b(golden, golden_dir):
    plan = json.load(open(os.path.join(golden_dir, "plan_vicuna-7b-v1.5-16k_moa_alpha_beta.json")))
    rows = [p for p in golden["plans"] if p.get("plan_file", "").startswith("examples/lmsys--vicuna-7b")]
    assert len(rows) == 2
    _check_rows(plan, rows)


def test_plan_rule_shipped_llama3_70b(golden):
    """examples/gradientai--Llama-3-70B-Instruct-262k/streamingllm_alpha_beta.json of the reference is
    80 layers x 64 heads of alpha = 0, beta = 0.5 (a uniform plan, written out here instead of copied)."""
    plan = {"alphas": [[0.0] * 64 for _ in range(80)], "betas": [[0.5] * 64 for _ in range(80)]}
    rows = [p for p in golden["plans"] if "Llama-3-70B" in p.get("plan_file", "")]
    assert len(rows) == 2
    _check_rows(plan, rows)


def test_plan_rule_options():
    """minimum_cache_size is applied after the clamp to the sequence (a cache may exceed it), sizes are
    rounded up to split_size, sink_size caps the static part (reference :1224-1237)."""
    plan = {"alphas": [[0, 1000, 5]], "betas": [[0.0, 0.0, 0.01]]}
    r = moa_config_to_cache_config(plan, 100, 28, sink_size=96, minimum_cache_size=80, split_size=32, verbose=False)
    assert r == {"cache_size": [[96, 128, 96]], "static_size": [[96, 96, 96]]}
    assert r == moa_oracle.moa_config_to_cache_config(plan, 100, 28, sink_size=96, minimum_cache_size=80,
                                                      split_size=32)


def test_constructor_against_reference_vectors(golden):
    for case in golden["cases"]:
        B = case["B"]
        c = StaticCircularCache([case["cache_size"]], static_size=[case["static_size"]], batch_size=B,
                                head_dim=case["D"], device="cpu", dtype=torch.float32)
        ctor, tag = case["ctor"], case["name"]
        assert c.cache_head_start_index[0].tolist() == ctor["head_start"], tag
        assert c.head_index[0].tolist() == ctor["head_index"], tag
        assert c.circular_cache_head_index[0].tolist() == ctor["circular_head"], tag
        assert c.circular_cache_size[0].tolist() == ctor["circular_size"], tag
        assert c.cache_update_index[0].tolist() == ctor["update_index"], tag
        assert c.cache_max_length[0].tolist() == case["cache_size"], tag
        assert c.static_cache_size[0].tolist() == case["static_size"], tag
        assert c.cache_valid_length[0].tolist() == [[0] * len(case["cache_size"])] * B, tag
        assert c.mask_cache[0].shape == (B, sum(case["cache_size"])) and not c.mask_cache[0].any(), tag
        for t in (c.cache_head_start_index[0], c.cache_update_index[0], c.cache_valid_length[0], c.mask_cache[0]):
            assert t.dtype == torch.int64 and t.is_contiguous(), tag
        assert len(c) == 1 and c.get_seq_length(0) == 0


def test_constructor_several_layers_and_default_static():
    c = StaticCircularCache([[128, 64], [64, 192, 64]], batch_size=2, head_dim=64)
    assert len(c) == 2 and c.dtype == torch.float16
    assert c.static_cache_size[1].tolist() == [0, 0, 0]
    assert c.circular_cache_size[1].tolist() == [64, 192, 64]
    assert c.head_index[1].tolist() == [0, 64, 256, 320]
    assert c.layer_cache_size == [192, 320]
    with pytest.raises(AssertionError):
        StaticCircularCache([[64]], static_size=[[65]])


def test_capturing_a_decode_step_too_early_is_refused(monkeypatch):
    """A decode step recorded into a graph bakes in kv_len, which decides whether a head has left its
    static part: capture is only allowed once every head has (host logic, checked without a GPU)."""
    c = StaticCircularCache([[128, 192]], static_size=[[64, 32]], batch_size=1, head_dim=64)
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: True)
    for kv_len, ok in ((0, False), (40, False), (63, False), (64, True), (500, True)):
        c._kv_len[0] = kv_len
        if ok:
            c._check_capture(0, "cpu")
        else:
            with pytest.raises(RuntimeError, match="static"):
                c._check_capture(0, "cpu")
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: False)
    c._kv_len[0] = 0
    c._check_capture(0, "cpu")


def test_update_model_function_binds_like_the_reference():
    """Host logic of the wrapper binding (MoA/models/interface.py:3-28): Llama-family names get
    set_mixture_of_attention bound to model.model, others raise; the plan is stored (and re-ordered with
    the projections when heads are permuted)."""
    from types import SimpleNamespace
    from torch import nn
    from moa_amd.models.interface import update_model_function
    from moa_amd.models.llama.modeling_llama import LlamaMixtureAttention

    layers = nn.ModuleList(nn.Module() for _ in range(2))
    for i, l in enumerate(layers):
        l.self_attn = LlamaMixtureAttention(64, 4, 2, head_dim=16, layer_idx=i, dtype=torch.float32)
    inner = nn.Module()
    inner.layers = layers
    model = SimpleNamespace(model=inner)
    with pytest.raises(NotImplementedError):
        update_model_function(model, "gpt2")
    assert update_model_function(model, "lmsys/longchat-7b") is model
    w_before = layers[0].self_attn.k_proj.weight.data.clone()
    inner.set_mixture_of_attention({"alphas": [[512.0, 128.0], [64.0, 64.0]], "betas": [[0.0, 0.0]] * 2},
                                   permute_head=True, moa_max_new_token=16)
    assert inner.use_moa and inner.moa_max_new_token == 16 and inner.last_hidden_only
    assert inner.moa_config["alphas"] == [[128.0, 512.0], [64.0, 64.0]]          # layer 0: heads swapped
    w_after = layers[0].self_attn.k_proj.weight.data
    assert torch.equal(w_after.view(2, 16, 64)[0], w_before.view(2, 16, 64)[1])
    assert torch.equal(layers[1].self_attn.k_proj.weight.data.view(2, 16, 64)[0],
                       layers[1].self_attn.k_proj.weight.data.view(2, 16, 64)[0])
    with pytest.raises(NotImplementedError):
        inner.use_block_sparse_attention_lut()


def test_efficiency_cli_arguments():
    from moa_amd import efficiency_test
    a = efficiency_test.parse_args(["--prefill_len", "4096"])
    assert (a.test_mode, a.num_iters, a.batch_size, a.decode_len, a.model_name) == (
        "whole", 1, 1, None, "lmsys/vicuna-7b-v1.5-16k")
    assert efficiency_test.shape_of("lmsys/vicuna-7b-v1.5-16k")[0] == "7b"
    assert efficiency_test.shape_of("lmsys/vicuna-13b-v1.5-16k")[1][:4] == (40, 5120, 40, 40)
    assert efficiency_test.shape_of("gradientai/Llama-3-70B-Instruct-262k")[1][2:4] == (64, 8)
    with pytest.raises(NotImplementedError):
        efficiency_test.shape_of("gpt2")


def test_cache_summary_columns():
    """The reference's cache summary (MoA/attention/cache_utils.py:1241-1293): per layer and for the model,
    (mean, min, max) of cache_size, static_size, circular_size and ratio = cache / (seq_len + max_new_token)."""
    from moa_amd.attention.cache_utils import cache_config_summary, format_cache_summary
    layers, model = cache_config_summary([[128, 1024, 128], [2624, 1152, 2560]], [[64] * 3] * 2, 5120)
    assert layers[0]["cache_size"] == (pytest.approx(1280 / 3), 128, 1024)
    assert layers[1]["circular_size"] == (pytest.approx(2048.0), 1088, 2560)
    assert layers[0]["ratio"][2] == pytest.approx(0.2) and layers[0]["raw_cache_size"][0] == 5120
    assert model["cache_size"] == (pytest.approx(7616 / 6), 128, 2624) and model["static_size"] == (64, 64, 64)
    text = format_cache_summary(layers, model)
    assert text.splitlines()[0].split()[:2] == ["layer_id", "raw_cache_size"] and "circular_size" in text
