"""Writes tests/golden/cache_update_vectors.json from the reference's own
StaticCircularCache (CPU tensors).  Runs only where the reference checkout is
mounted; the committed JSON is what the tests read.

The reference targets transformers 4.44, whose ``Cache`` base class is an empty
shell; the installed release's ``Cache`` needs layer arguments and has
read-only ``batch_size`` properties.  For this process only, the name
``transformers.cache_utils.Cache`` is therefore bound to an empty base class
before the reference module is imported.  Nothing of the reference is modified
and none of the cache arithmetic lives in that base class.

Usage:  python tests/golden/make_cache_vectors.py [/root/reference]
"""
import json
import os
import sys

import numpy as np
import torch

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, ref)

import transformers.cache_utils as _tcu  # noqa: E402



class _EmptyCacheBase:
    def __init__(self, *a, **k):
        pass


_tcu.Cache = _EmptyCacheBase

from MoA.attention.cache_utils import StaticCircularCache, moa_config_to_cache_config  # noqa: E402


def payload(B, H, S, D, base):
    """token id encoded in the payload: value = base + h*1000 + t  (exact in fp32)."""
    t = torch.arange(S, dtype=torch.float32)[None, None, :, None]
    h = torch.arange(H, dtype=torch.float32)[None, :, None, None] * 1000.0
    b = torch.arange(B, dtype=torch.float32)[:, None, None, None] * 100000.0
    return (base + b + h + t).expand(B, H, S, D).contiguous()


def snapshot(c, step):
    if c.key_cache[0].device.type != "meta":
        # the value payload is always key + 0.5 where the mask is set; store keys only
        m = c.mask_cache[0] == 1
        assert torch.equal(c.value_cache[0][:, :, 0][m], c.key_cache[0][:, :, 0][m] + 0.5)
    return {
        "step": step,
        "update_index": c.cache_update_index[0].tolist(),
        "valid_length": c.cache_valid_length[0].tolist(),
        "mask_cache": c.mask_cache[0].tolist(),
        "key_col0": c.key_cache[0][:, :, 0].tolist() if c.key_cache[0].device.type != "meta" else None,
        "kv_len": c._kv_len[0],
    }


def run_case(name, cache_size, static_size, B, D, prefill_lens, S, n_decode, use_mask, snap_every=1):
    c = StaticCircularCache(cache_size=[cache_size], static_size=[static_size], batch_size=B,
                            head_dim=D, device="cpu", dtype=torch.float32)
    H = len(cache_size)
    case = {"name": name, "cache_size": cache_size, "static_size": static_size, "B": B, "D": D,
            "S": S, "prefill_lens": prefill_lens, "n_decode": n_decode, "use_mask": use_mask,
            "ctor": {
                "head_start": c.cache_head_start_index[0].tolist(),
                "head_index": c.head_index[0].tolist(),
                "circular_head": c.circular_cache_head_index[0].tolist(),
                "circular_size": c.circular_cache_size[0].tolist(),
                "update_index": c.cache_update_index[0].tolist(),
            },
            "steps": []}
    am = None
    if use_mask:
        am = torch.zeros(B, S, dtype=torch.int64)
        for i, n in enumerate(prefill_lens):
            am[i, S - n:] = 1
    base = 0.0
    if S > 0:
        k = payload(B, H, S, D, base)
        c.update(k, k + 0.5, 0, am)
        case["steps"].append(snapshot(c, 0))
    pos = S
    for i in range(n_decode):
        k = payload(B, H, 1, D, float(pos))
        if am is not None:
            am = torch.cat([am, torch.ones(B, 1, dtype=torch.int64)], dim=-1)
        c.update(k, k + 0.5, 0, am)
        if (i + 1) % snap_every == 0 or i == n_decode - 1:
            case["steps"].append(snapshot(c, i + 1))
        pos += 1
    return case


cases = []
# the reference's own demo (cache_utils.py:1301-1371): left-padded rows 14, 9, 5
cases.append(run_case("reference_demo", [5, 10], [2, 3], 3, 4, [14, 9, 5], 14, 9, True))
# a left-padded row whose valid tokens do not fill its static part: the reference then
# enters the ring early because its token counter includes padding (cache_utils.py:1041-1045,1139)
cases.append(run_case("padded_short_row", [5, 10], [2, 3], 3, 4, [12, 2, 1], 12, 8, True))
# same sizes, no mask
cases.append(run_case("demo_no_mask", [5, 10], [2, 3], 3, 4, [14, 14, 14], 14, 9, False))
# prompt shorter than static part of one head, then decode through the static->ring switch
cases.append(run_case("short_prompt", [8, 6, 12], [4, 2, 5], 2, 2, [3, 3], 3, 14, False))
# prompt between s and s+c
cases.append(run_case("mid_prompt", [8, 6, 12], [4, 2, 5], 2, 2, [7, 7], 7, 12, False))
# long prompt, many wraps
cases.append(run_case("long_prompt", [8, 6, 12], [4, 2, 5], 2, 2, [40, 40], 40, 20, False))
# decode only from an empty cache
cases.append(run_case("decode_only", [6, 4], [2, 1], 2, 2, [], 0, 15, False))
# 64-multiple sizes like production (sink 64)
cases.append(run_case("prod_like", [128, 256, 192], [64, 64, 64], 1, 1, [300], 300, 70, False, snap_every=23))
# static 0 (pure ring)
cases.append(run_case("pure_ring", [4, 7], [0, 0], 1, 1, [10], 10, 9, False))

plans = []
for a, b, n, mn in [(0, 0.5, 1024, 1024), (-1024, 0.125, 1024, 1024), (1024, 1.0, 1024, 1024),
                    (100.7, 0.3, 900, 100), (0, 0, 10, 10), (8192, 0.0, 4096, 1024), (-1024, 1.0, 16384, 1024)]:
    r = moa_config_to_cache_config({"alphas": [[a]], "betas": [[b]]}, n, max_new_token=mn, verbose=False)
    plans.append({"alpha": a, "beta": b, "seq_len": n, "max_new_token": mn,
                  "cache_size": r["cache_size"][0][0], "static_size": r["static_size"][0][0]})
for rel in ["examples/lmsys--vicuna-7b-v1.5-16k/moa_alpha_beta.json",
            "examples/gradientai--Llama-3-70B-Instruct-262k/streamingllm_alpha_beta.json"]:
    plan = json.load(open(os.path.join(ref, rel)))
    for n in (4096, 16384):
        r = moa_config_to_cache_config(plan, n, verbose=False)
        plans.append({"plan_file": rel, "seq_len": n, "max_new_token": 1024,
                      "cache_size_layer0": r["cache_size"][0], "cache_size_last": r["cache_size"][-1],
                      "cache_size_sum": int(np.sum(r["cache_size"])), "static_size_sum": int(np.sum(r["static_size"]))})

out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cache_update_vectors.json")
json.dump({"cases": cases, "plans": plans}, open(out, "w"))
print("wrote", out, os.path.getsize(out), "bytes")
