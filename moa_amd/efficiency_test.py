#!/usr/bin/env python3
"""Efficiency test of a MoA model on the GPU: the three modes of the reference's
scripts/evaluate/effieicency_test.py (``--test_mode prefill | decode | whole``) with its argument names
and its printed figures (elapsed / per iter / per token, and for decode
``throughput = batch_size * decode_len * num_iters / seconds``, :548-562).

    python -m moa_amd.efficiency_test --prefill_len 16384 --decode_len 64 --batch_size 8 \\
        --moa_config tests/golden/plan_vicuna-7b-v1.5-16k_moa_alpha_beta.json --test_mode decode --cuda_event

There is no network here, so instead of downloading a checkpoint ``--model_name`` picks the SHAPE of a
Llama-family decoder (names containing 7b / 13b / 70b, or ``tiny``), built with random weights from
moa_amd.models.llama.modeling_llama.LlamaMixtureForCausalLM; prompts are random token ids.  Without
``--moa_config`` every head gets the synthetic elastic plan of the benchmark (64 sinks + window
alpha + beta * N).  Only the attention path runs in libmoa_hip.so; norms, MLP and LM head are torch.
"""
from __future__ import annotations

import argparse
import json
import random
import sys
import time

SHAPES = {   # layers, hidden, query heads, kv heads, FFN, vocab
    "7b": (32, 4096, 32, 32, 11008, 32000),
    "13b": (40, 5120, 40, 40, 13824, 32000),
    "70b": (80, 8192, 64, 8, 28672, 128256),
    "tiny": (2, 512, 4, 2, 1024, 1000),
}


def parse_args(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--prefill_len", type=int, required=True)
    ap.add_argument("--model_name", type=str, default="lmsys/vicuna-7b-v1.5-16k",
                    help="picks the decoder shape by the size in the name (7b, 13b, 70b, tiny); weights are random")
    ap.add_argument("--dtype", choices=["fp16", "bf16"], default="fp16")
    ap.add_argument("--moa_config", type=str, default=None, help="the path to moa configuration file")
    ap.add_argument("--num_iters", type=int, default=1)
    ap.add_argument("--batch_size", type=int, default=1)
    ap.add_argument("--decode_len", type=int, default=None, help="decoding max len. if None, just do prefilling")
    ap.add_argument("--cuda_event", action="store_true")
    ap.add_argument("--cuda_cache", action="store_true")
    ap.add_argument("--test_mode", type=str, choices=["decode", "prefill", "whole"], default="whole")
    ap.add_argument("--moa_verbose", action="store_true", help="print the cache configuration of the plan")
    return ap.parse_args(argv)


def shape_of(model_name: str):
    low = model_name.lower()
    for key in ("70b", "13b", "7b", "tiny"):
        if key in low:
            return key, SHAPES[key]
    raise NotImplementedError("Model {} not implemented".format(model_name))


def build_model(args, torch, device):
    from moa_amd.attention.cache_utils import moa_config_to_cache_config
    from moa_amd.models.llama.modeling_llama import LlamaMixtureForCausalLM
    from moa_amd.workloads import elastic_spans

    key, (L, hidden, Hq, Hkv, ffn, vocab) = shape_of(args.model_name)
    dtype = torch.float16 if args.dtype == "fp16" else torch.bfloat16
    head_dim = 128
    if args.moa_config is not None:
        with open(args.moa_config, "r") as f:
            moa_config = json.load(f)
        assert len(moa_config["alphas"]) == L and len(moa_config["alphas"][0]) == Hkv, (
            f"the plan is for {len(moa_config['alphas'])} layers x {len(moa_config['alphas'][0])} heads, "
            f"{args.model_name} has {L} x {Hkv}")
    else:
        moa_config = {"alphas": [[64 + s for s in elastic_spans(Hkv, args.prefill_len, seed=l)] for l in range(L)],
                      "betas": [[0.0] * Hkv for _ in range(L)]}
    model = LlamaMixtureForCausalLM(L, hidden, Hq, Hkv, ffn, vocab, head_dim=head_dim, dtype=dtype, device=device)
    for p in model.parameters():
        if p.dim() > 1:
            p.data.normal_(0.0, 0.02)
    max_new = (args.decode_len or 0) + 8
    model.set_mixture_of_attention(moa_config, permute_head=True, moa_max_new_token=max_new)
    if args.moa_verbose:
        moa_config_to_cache_config(model.moa_config, args.prefill_len, max_new_token=max_new, verbose=True)
    return model, vocab


def fake_decode(model, torch, logits, cache, max_len, batch_size, vocab, device):
    """The reference's decode loop (:74-91): the first token is the prompt pass's argmax, every later one a
    random id (the same for all batch rows), max_len - 1 model calls."""
    pred = logits.argmax(dim=-1, keepdim=True)
    for _ in range(max_len - 1):
        logits, cache = model(pred, cache)
        pred = torch.full((batch_size, 1), random.randint(0, vocab - 1), device=device, dtype=torch.long)
    return cache


def run_model(args, out=sys.stdout):
    import torch

    if not torch.cuda.is_available():
        raise SystemExit("efficiency_test: no GPU visible (moa_amd has no CPU path)")
    if args.test_mode in ("decode", "whole") and not args.decode_len:
        raise SystemExit("efficiency_test: --decode_len is needed for --test_mode decode and whole")
    device = torch.device("cuda:0")
    model, vocab = build_model(args, torch, device)
    num_iters = args.num_iters
    gen = torch.Generator().manual_seed(0)
    input_ids = torch.randint(0, vocab, (args.batch_size, args.prefill_len), generator=gen).to(device)
    print(f"input_shape: {tuple(input_ids.shape)}", file=out)

    for _ in range(2):   # warmup
        model(input_ids)
    prefilled = []
    if args.test_mode == "decode":   # generate the past key value states
        for _ in range(num_iters):
            prefilled.append(model(input_ids))
    print("Start testing", file=out)
    if args.cuda_cache:
        torch.cuda.empty_cache()
        torch.cuda.reset_peak_memory_stats()
    torch.cuda.synchronize()
    start_event, end_event = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start_event.record()
    t0 = time.perf_counter()
    for i in range(num_iters):
        if args.test_mode == "prefill":
            model(input_ids)
        elif args.test_mode == "decode":
            logits, cache = prefilled[i]
            fake_decode(model, torch, logits, cache, args.decode_len, args.batch_size, vocab, device)
        else:
            logits, cache = model(input_ids)
            fake_decode(model, torch, logits, cache, args.decode_len, args.batch_size, vocab, device)
            print(f"iter {i} done", file=out)
    end_event.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    elapsed_time_ms = start_event.elapsed_time(end_event) if args.cuda_event else wall_ms
    result = {"elapsed_ms": elapsed_time_ms, "per_iter_ms": elapsed_time_ms / num_iters}
    print(f"Elapsed time: {elapsed_time_ms} ms", file=out)
    print(f"per iter: {elapsed_time_ms / num_iters} ms", file=out)
    if args.test_mode == "prefill":
        print(f"input shape: {tuple(input_ids.shape)}", file=out)
        result["per_token_ms"] = elapsed_time_ms / num_iters / args.batch_size / input_ids.shape[1]
        print(f"per token: {result['per_token_ms']} ms", file=out)
    if args.test_mode == "decode":
        result["per_token_ms"] = elapsed_time_ms / num_iters / args.decode_len / args.batch_size
        result["throughput_tokens_per_s"] = args.batch_size * args.decode_len * num_iters / (elapsed_time_ms / 1000)
        print(f"per token: {result['per_token_ms']} ms", file=out)
        print(f"throughput: {result['throughput_tokens_per_s']} tokens/s", file=out)
    if args.cuda_cache:
        result["max_memory_mb"] = torch.cuda.max_memory_allocated() // 2 ** 20
        print(f"Max memory: {result['max_memory_mb']} MB", file=out)
    return result


if __name__ == "__main__":
    run_model(parse_args())
