#!/usr/bin/env python3
"""Benchmark of the MoA sparse-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L]

Headline workload (the configuration the metric is quoted on):
decode step + cache append at the 7B shape -- batch 64, 32 heads, head_dim 128,
fp16, logical context 16384, every (layer, head) with its own ring of
64 sinks + elastic window.  One "step" generates one token for the whole batch
through the attention path of all L=32 layers: per layer one fused ring append
(moa_cache_append) and one split-K decode attention (moa_decode_fwd).  The
projections/MLP of a full decoder are not part of this path and not run.

value = batch * steps / wall seconds (whole job, inputs resident in HBM).

Also measured, outside the timed region, and reported in the same JSON line:
  * sparse prefill: B=4, H=32, D=128, N=8192, bf16 -> ms/layer,
    TFLOP/s on live (unmasked) work, fraction of the dense bf16 MFMA peak;
  * the append kernel alone (us, GB/s);
  * cpu_baseline: the CPU oracle's restatement of the reference's dense
    debug decode on a bounded sample, on this box's host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
# HBM bytes moved by one decode launch divided by its algorithmic bytes, from two rocprofv3 --pmc runs
# (FETCH_SIZE, WRITE_SIZE) scaled by a 1 GiB copy kernel's readings; see
# profiles/hbm_traffic_decode_and_prefill.txt.  bench.py cannot profile itself, so the ratio is carried here.
DECODE_TRAFFIC_RATIO = 1.003
MFMA_PEAK_TFLOPS = 2500.0      # MI355X dense bf16 / fp16


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=32, help="decoder layers in one decode step")
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--ctx", type=int, default=16384)
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--prefill-iters", type=int, default=20)
    ap.add_argument("--plan", default=None,
                    help='with --only e2e: a plan file in the reference\'s JSON format {"alphas": [L][H], "betas": [L][H]} '
                         "(e.g. tests/golden/plan_vicuna-7b-v1.5-16k_moa_alpha_beta.json) instead of the synthetic plan")
    ap.add_argument("--shape", choices=["7b", "70b"], default="7b",
                    help="with --only e2e: 7b = 32 layers, 32 heads, B=8, 16k prompt, fp16; 70b = 80 layers, 64 query "
                         "heads on 8 kv heads, hidden 8192, B=4, 32k prompt, bf16 (the largest config)")
    ap.add_argument("--new-tokens", type=int, default=64, help="with --only e2e-full: decode steps to time")
    ap.add_argument("--test_mode", choices=["prefill", "decode", "whole"], default=None,
                    help="run moa_amd.efficiency_test (the reference's efficiency script: same modes and printed "
                         "figures) on the whole decoder of --shape at that config's batch and prompt length, "
                         "--new-tokens decode steps; not the contract line")
    ap.add_argument("--no-e2e", action="store_true",
                    help="skip the whole-decoder runs of the two end-to-end configurations in the default line")
    ap.add_argument("--only", choices=["decode", "prefill", "copy", "e2e", "e2e-full", "gqa", "prompt"], default=None,
                    help="profiling aid: run one part only and print its figures (not the contract line)")
    return ap.parse_args()


def build_decode_state(torch, dev, layers, B, H, D, ctx, dtype):
    """Per layer: a StaticCircularCache in the state right after a ctx-token
    prompt (rings full, write pointers uniformly random in the ring, one row on
    its last slot so that the first step wraps), K/V ~ N(0,1)."""
    from moa_amd import StaticCircularCache
    from moa_amd.workloads import elastic_spans, ring_cache_sizes

    cache_size, static_size = [], []
    for l in range(layers):
        cs, ss = ring_cache_sizes(elastic_spans(H, ctx, seed=l))
        cache_size.append(cs)
        static_size.append(ss)
    cache = StaticCircularCache(cache_size, static_size=static_size, batch_size=B, head_dim=D,
                                device=dev, dtype=dtype)
    gen = torch.Generator(device=dev).manual_seed(1234)
    rows_total = 0
    for l in range(layers):
        sumc = cache.layer_cache_size[l]
        rows_total += sumc * B
        cache.key_cache[l] = torch.empty(B, sumc, D, dtype=dtype, device=dev).normal_(generator=gen)
        cache.value_cache[l] = torch.empty(B, sumc, D, dtype=dtype, device=dev).normal_(generator=gen)
        circ = cache.circular_cache_size[l]
        off = (torch.rand(B, H, generator=gen, device=dev) * circ[None, :].float()).long()
        off = torch.minimum(off, circ[None, :] - 1)
        off[0, :] = circ - 1
        cache.cache_update_index[l] = (cache.circular_cache_head_index[l][None, :] + off).contiguous()
        cache.cache_valid_length[l] = cache.cache_max_length[l][None, :].expand(B, -1).contiguous()
        cache.mask_cache[l].fill_(1)
        cache._kv_len[l] = ctx
    return cache, rows_total


def bench_decode(torch, dev, args):
    from moa_amd import mixture_of_sparse_attention
    from moa_amd.workloads import append_bytes, decode_bytes

    B, H, D, L = args.batch, 32, 128, args.layers
    dtype = torch.float16
    free, _ = torch.cuda.mem_get_info(dev)
    # K+V bytes of one layer at these spans (~5.2 GB at B=64); keep 10% headroom
    from moa_amd.workloads import elastic_spans, ring_cache_sizes
    need = sum(sum(ring_cache_sizes(elastic_spans(H, args.ctx, seed=l))[0]) for l in range(L)) * B * D * 2 * 2
    distinct = L
    if need > 0.9 * free:
        distinct = max(1, int(L * 0.9 * free / need))
    cache, rows_total = build_decode_state(torch, dev, distinct, B, H, D, args.ctx, dtype)
    gen = torch.Generator(device=dev).manual_seed(99)
    # per layer inputs of one step: q and the new k, v as the model hands them over
    # ([B, 1, H, D] projections viewed [B, H, 1, D])
    qs = [torch.randn(B, 1, H, D, generator=gen, device=dev, dtype=dtype).transpose(1, 2) for _ in range(L)]
    kn = [torch.randn(B, 1, H, D, generator=gen, device=dev, dtype=dtype).transpose(1, 2) for _ in range(L)]
    vn = [torch.randn(B, 1, H, D, generator=gen, device=dev, dtype=dtype).transpose(1, 2) for _ in range(L)]
    sm = D ** -0.5

    def one_step(events=None):
        for l in range(L):
            c = l % distinct
            if events is not None:
                e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
                e0.record()
            kc, vc = cache.update(kn[l], vn[l], c)
            if events is not None:
                e1.record()
            mixture_of_sparse_attention(qs[l], kc, vc, sm,
                                        head_start_index=cache.cache_head_start_index[c],
                                        head_valid_length=cache.cache_valid_length[c])
            if events is not None:
                e2.record()
                events.append((e0, e1, e2))

    for _ in range(args.warmup):
        one_step()
    torch.cuda.synchronize(dev)
    events = []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one_step(events)
    torch.cuda.synchronize(dev)
    wall = time.perf_counter() - t0

    # the same step with the rotary embedding of q and k folded into the append launch
    # (StaticCircularCache.rope_update: what a caller that owns the projections runs)
    ang = torch.rand(1, 1, D, generator=gen, device=dev) * 6.28
    cos, sin = ang.cos().to(dtype), ang.sin().to(dtype)

    def fused_step():
        for l in range(L):
            c = l % distinct
            qe, kc, vc = cache.rope_update(qs[l], kn[l], vn[l], cos, sin, c)
            mixture_of_sparse_attention(qe, kc, vc, sm, head_start_index=cache.cache_head_start_index[c],
                                        head_valid_length=cache.cache_valid_length[c])

    fused_step()
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fused_step()
    torch.cuda.synchronize(dev)
    fused_wall = time.perf_counter() - t0

    app_ms = sum(e0.elapsed_time(e1) for e0, e1, _ in events) / len(events)
    dec_ms = sum(e1.elapsed_time(e2) for _, e1, e2 in events) / len(events)
    rows_per_layer = rows_total / distinct
    dec_bytes = decode_bytes(int(rows_per_layer), B, H, D)
    app_bytes = append_bytes(B, H, D)
    return {
        "wall_s": wall,
        "tokens_per_s": B * args.steps / wall,
        "ms_per_step": wall / args.steps * 1e3,
        "fused_rotary_step": {"workload": "the same step with the rotary embedding of q and k fused into the append launch",
                              "ms_per_step": fused_wall / args.steps * 1e3,
                              "tokens_per_s": B * args.steps / fused_wall},
        "decode_ms": dec_ms,
        "decode_bytes": dec_bytes,
        "decode_gbs": dec_bytes / (dec_ms * 1e-3) / 1e9,
        "append_us": app_ms * 1e3,
        "append_bytes": app_bytes,
        "append_gbs": app_bytes / (app_ms * 1e-3) / 1e9,
        "distinct_layer_caches": distinct,
        "kv_rows_per_layer": int(rows_per_layer),
        "cache": cache,
    }


def bench_rope_append(torch, dev, args, cache, iters=50):
    """The step in front of the decode kernel at the headline shape: rotary embedding of q and k
    plus the ring append, as ONE launch (StaticCircularCache.rope_update) and as the two launches
    it replaces (rotary kernel, then append)."""
    from moa_amd.kernels.rotary import apply_rotary_pos_emb
    from moa_amd.workloads import rope_append_bytes

    B, H, D = args.batch, 32, 128
    dtype = torch.float16
    gen = torch.Generator(device=dev).manual_seed(5)
    q, k, v = (torch.randn(B, 1, H, D, generator=gen, device=dev, dtype=dtype).transpose(1, 2) for _ in range(3))
    ang = torch.rand(B, 1, D, generator=gen, device=dev) * 6.28
    cos, sin = ang.cos().to(dtype), ang.sin().to(dtype)

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize(dev)
        evs = []
        for _ in range(iters):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            evs.append((e0, e1))
        torch.cuda.synchronize(dev)
        ms = sorted(a.elapsed_time(b) for a, b in evs)
        return ms[len(ms) // 2] * 1e3

    def separate():
        qe, ke = apply_rotary_pos_emb(q, k, cos, sin)
        cache.update(ke, v, 0)

    fused_us = timed(lambda: cache.rope_update(q, k, v, cos, sin, 0))
    separate_us = timed(separate)
    nbytes = rope_append_bytes(B, H, D)
    return {"fused_us": fused_us, "separate_us": separate_us, "bytes": nbytes,
            "GB/s": nbytes / (fused_us * 1e-6) / 1e9}


C5_ALPHA_RANGE = (256.0, 8192.0)   # the largest config draws alpha from [256, 8192] (the others from [64, 2048])


def bench_decode_gqa(torch, dev, args, iters=5, layers=8):
    """Decode attention at the grouped-query shape of the largest config (B=4, 64 query heads on 8
    rings of head_dim 128, bf16, 32k context: 64 sinks + elastic window per ring, alpha in
    [256, 8192]): the matrix-core kernel.  K+V bytes of the valid rows per launch over the mean
    HIP-event time around the call."""
    import numpy as np
    from moa_amd import mixture_of_sparse_attention
    from moa_amd.workloads import elastic_spans, ring_cache_sizes
    out = {}
    for B in (4, 64):
        Hkv, G, D, ctx = 8, 8, 128, 32768
        caches = []
        for l in range(layers):
            sizes, _ = ring_cache_sizes(elastic_spans(Hkv, ctx, seed=l, alpha_range=C5_ALPHA_RANGE))
            sizes = np.asarray(sizes)
            sumc = int(sizes.sum())
            kc = torch.randn(B, sumc, D, device=dev, dtype=torch.bfloat16)
            vc = torch.randn(B, sumc, D, device=dev, dtype=torch.bfloat16)
            start = np.concatenate([[0], np.cumsum(sizes)[:-1]])
            hs = torch.from_numpy(np.broadcast_to(start, (B, Hkv)).astype(np.int64).copy()).to(dev)
            hv = torch.from_numpy(np.broadcast_to(sizes, (B, Hkv)).astype(np.int64).copy()).to(dev)
            caches.append((kc, vc, hs, hv, sumc))
        q = torch.randn(B, Hkv * G, 1, D, device=dev, dtype=torch.bfloat16)
        sm = D ** -0.5
        for kc, vc, hs, hv, _ in caches:
            mixture_of_sparse_attention(q, kc, vc, sm, head_start_index=hs, head_valid_length=hv)
        torch.cuda.synchronize(dev)
        # isolated calls: the queue is empty before each, so the host's launch path is in the figure
        ms, byts = 0.0, 0
        for _ in range(iters):
            for kc, vc, hs, hv, sumc in caches:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                mixture_of_sparse_attention(q, kc, vc, sm, head_start_index=hs, head_valid_length=hv)
                e1.record()
                torch.cuda.synchronize(dev)
                ms += e0.elapsed_time(e1)
                byts += B * sumc * D * 2 * 2
        n = iters * len(caches)
        # back to back, as the layers of a decode step follow each other (the headline loop is timed this way)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            for kc, vc, hs, hv, sumc in caches:
                mixture_of_sparse_attention(q, kc, vc, sm, head_start_index=hs, head_valid_length=hv)
        e1.record()
        torch.cuda.synchronize(dev)
        stream_ms = e0.elapsed_time(e1)
        out[f"B{B}"] = {"us_per_launch": stream_ms / n * 1e3, "GB/s": byts / (stream_ms * 1e-3) / 1e9,
                        "frac_of_hbm_peak": byts / (stream_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                        "us_per_isolated_launch": ms / n * 1e3,
                        "timing": "launches back to back over 8 layers' rings (queue kept full, like the layers of a "
                                  "decode step); isolated = queue empty before every call"}
        del caches
        torch.cuda.empty_cache()
    out["workload"] = ("decode attention, 64 query heads on 8 rings, D=128, bf16, 32k context, ring = 64 sinks + elastic "
                       "window (alpha U[256,8192], beta U[0,0.5])")
    return out


def bench_e2e(torch, dev, args, new_tokens=32):
    """The attention path of a decoder end to end: q/k/v/o projections (library GEMMs), rotary
    embedding + cache update, sparse prefill of the prompt, then new_tokens decode steps.  Norms, MLPs
    and the LM head are not on the path and are left out.  Shapes: 7b = 32 layers, hidden 4096, 32
    heads of 128, B=8, 16k prompt, fp16; 70b = 80 layers, hidden 8192, 64 query heads on 8 kv heads,
    B=4, 32k prompt, bf16.  Random weights; the plan is synthetic (elastic spans per kv head) unless
    --plan names a plan file, whose layer and head counts then set the shape (head dim stays 128)."""
    from moa_amd.models.llama.modeling_llama import LlamaMixtureAttentionStack
    from moa_amd.workloads import elastic_spans

    D = 128
    if args.shape == "70b":
        L, Hq, H, batch, n_ctx, dtype = 80, 64, 8, 4, 32768, torch.bfloat16
    else:
        L, Hq, H, batch, n_ctx, dtype = args.layers, 32, 32, 8, 16384, torch.float16
    plan = None
    if args.plan:
        with open(args.plan) as f:
            plan = json.load(f)
        L, H = len(plan["alphas"]), len(plan["alphas"][0])
        Hq = H
    hidden = Hq * D
    model = LlamaMixtureAttentionStack(L, hidden, Hq, num_key_value_heads=H, head_dim=D, dtype=dtype, device=dev)
    for p in model.parameters():
        p.data.normal_(0.0, hidden ** -0.5)
    for layer in model.layers:       # the stack has no norms: small output projections keep the residual stream O(1)
        layer.o_proj.weight.data.mul_(L ** -0.5)
    # a plan whose cache sizes are sink (64) + the elastic window at n_ctx
    if plan is None:
        plan = {"alphas": [[64 + s for s in elastic_spans(H, n_ctx, seed=l)] for l in range(L)],
                "betas": [[0.0] * H for _ in range(L)]}
    model.set_mixture_of_attention(plan, permute_head=True, moa_max_new_token=new_tokens)
    gen = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn(batch, n_ctx, hidden, generator=gen, device=dev, dtype=dtype)
    pos = torch.arange(n_ctx, device=dev)[None, :]
    times = []
    for _ in range(2):   # first pass warms up
        cache = model.new_cache(batch, n_ctx, dev)
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        h = model(x, pos, cache)
        torch.cuda.synchronize(dev)
        times.append(time.perf_counter() - t0)
    prefill_s = times[-1]
    x1 = h[:, -1:, :].contiguous()
    pos1 = torch.full((1, 1), n_ctx, device=dev, dtype=torch.int64)

    def step():
        y = model(x1, pos1, cache)
        pos1.add_(1)
        return y

    for _ in range(3):
        step()
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for _ in range(3, new_tokens):
        step()
    torch.cuda.synchronize(dev)
    dec_s = (time.perf_counter() - t0) / (new_tokens - 3)
    # the same step captured once in a HIP graph and replayed (the library only enqueues kernels;
    # the position advances on the device)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for _ in range(new_tokens):
        graph.replay()
    torch.cuda.synchronize(dev)
    graph_s = (time.perf_counter() - t0) / new_tokens
    kept = sum(cache.layer_cache_size) / (L * H * (n_ctx + new_tokens))
    return {"workload": f"attention path of a decoder: L={L}, {Hq} query heads on {H} kv heads, D={D}, B={batch}, "
                        f"prompt {n_ctx}, {str(dtype).split('.')[-1]}",
            "plan": os.path.basename(args.plan) if args.plan else "synthetic elastic spans",
            "kv_kept_fraction": kept,
            "prefill_s": prefill_s, "prefill_tokens_per_s": batch * n_ctx / prefill_s,
            "decode_ms_per_step": dec_s * 1e3, "decode_tokens_per_s": batch / dec_s,
            "graph_decode_ms_per_step": graph_s * 1e3, "graph_decode_tokens_per_s": batch / graph_s}


def bench_e2e_full(torch, dev, args):
    """The whole decoder of the two end-to-end configs with random bf16 weights: embedding, per
    layer RMSNorm + attention + RMSNorm + SwiGLU, final norm, LM head, greedy decoding.  7b: 32
    layers, hidden 4096, 32 heads, FFN 11008, vocab 32000, B=8, 16384-token prompt, spans from alpha
    in [64, 2048]; 70b: 80 layers, hidden 8192, 64 query heads on 8 kv heads, FFN 28672, vocab 128256,
    B=4, 32768-token prompt, spans from alpha in [256, 8192]; beta in [0, 0.5] for both.  Only the
    attention runs in libmoa_hip.so; norms, MLP and LM head are torch (library GEMMs)."""
    from moa_amd.models.llama.modeling_llama import LlamaMixtureForCausalLM
    from moa_amd.workloads import elastic_spans

    D, dtype = 128, torch.bfloat16
    if args.shape == "70b":
        L, hidden, Hq, H, ffn, vocab, batch, n_ctx, arange = 80, 8192, 64, 8, 28672, 128256, 4, 32768, (256.0, 8192.0)
    else:
        L, hidden, Hq, H, ffn, vocab, batch, n_ctx, arange = 32, 4096, 32, 32, 11008, 32000, 8, 16384, (64.0, 2048.0)
    new_tokens = args.new_tokens
    model = LlamaMixtureForCausalLM(L, hidden, Hq, H, ffn, vocab, head_dim=D, dtype=dtype, device=dev)
    for p in model.parameters():
        if p.dim() > 1:
            p.data.normal_(0.0, 0.02)
    plan = {"alphas": [[64 + s for s in elastic_spans(H, n_ctx, seed=l, alpha_range=arange)] for l in range(L)],
            "betas": [[0.0] * H for _ in range(L)]}
    model.set_mixture_of_attention(plan, permute_head=True, moa_max_new_token=new_tokens + 8)
    ids = torch.randint(0, vocab, (batch, n_ctx), generator=torch.Generator().manual_seed(5)).to(dev)
    times = []
    for _ in range(2):   # first pass warms up
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        logits, cache = model(ids)
        torch.cuda.synchronize(dev)
        times.append(time.perf_counter() - t0)
    prefill_s = times[-1]
    tok = logits.argmax(-1, keepdim=True)
    pos = torch.full((1, 1), n_ctx, device=dev, dtype=torch.int64)

    def step():
        lg, _ = model(tok, cache, position_ids=pos)
        tok.copy_(lg.argmax(-1, keepdim=True))
        pos.add_(1)

    for _ in range(3):
        step()
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for _ in range(new_tokens):
        step()
    torch.cuda.synchronize(dev)
    dec_s = (time.perf_counter() - t0) / new_tokens
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for _ in range(2):
        graph.replay()
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for _ in range(new_tokens):
        graph.replay()
    torch.cuda.synchronize(dev)
    graph_s = (time.perf_counter() - t0) / new_tokens
    n_param = sum(p.numel() for p in model.parameters())
    return {"workload": f"whole decoder: L={L}, hidden {hidden}, {Hq} query heads on {H} kv heads, FFN {ffn}, vocab {vocab}, "
                        f"B={batch}, prompt {n_ctx}, bf16, random weights, greedy",
            "parameters": n_param,
            "kv_kept_fraction": sum(cache.layer_cache_size) / (L * H * (n_ctx + new_tokens + 8)),
            "prefill_s": prefill_s, "prefill_tokens_per_s": batch * n_ctx / prefill_s,
            "decode_steps_timed": new_tokens,
            "decode_ms_per_step": dec_s * 1e3, "decode_tokens_per_s": batch / dec_s,
            "graph_decode_ms_per_step": graph_s * 1e3, "graph_decode_tokens_per_s": batch / graph_s}


def bench_prefill(torch, dev, args, B=4, Hq=32, Hkv=32, N=8192, iters=None, alpha_range=(64.0, 2048.0)):
    """One sparse prefill layer: the headline shape (B=4, 32 heads, N=8192) by default; the grouped-
    query shape of the largest config with Hq=64, Hkv=8, N=32768 (spans per kv head, alpha in
    [256, 8192])."""
    from moa_amd import mixture_of_sparse_attention
    from moa_amd.workloads import elastic_spans, prefill_work

    D = 128
    H = Hkv
    dtype = torch.bfloat16
    spans = elastic_spans(H, N, seed=0, alpha_range=alpha_range)
    sink = torch.full((H,), 64, dtype=torch.int64, device=dev)
    local = torch.tensor(spans, dtype=torch.int64, device=dev)
    gen = torch.Generator(device=dev).manual_seed(7)
    # the model's projections are [B, N, H, D]; the operator sees them as [B, H, N, D] views
    q = torch.randn(B, N, Hq, D, generator=gen, device=dev, dtype=dtype).transpose(1, 2)
    k, v = (torch.randn(B, N, H, D, generator=gen, device=dev, dtype=dtype).transpose(1, 2) for _ in range(2))
    sm = D ** -0.5
    flops, tile_flops, tiles = prefill_work(N, [1] * H, [s // 64 for s in spans], B, D)
    flops, tile_flops = flops * (Hq // Hkv), tile_flops * (Hq // Hkv)
    for _ in range(5 if iters is None else 2):
        mixture_of_sparse_attention(q, k, v, sm, sink_size=sink, local_size=local)
    torch.cuda.synchronize(dev)
    evs = []
    for _ in range(args.prefill_iters if iters is None else iters):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        mixture_of_sparse_attention(q, k, v, sm, sink_size=sink, local_size=local)
        e1.record()
        evs.append((e0, e1))
    torch.cuda.synchronize(dev)
    ms = sorted(e0.elapsed_time(e1) for e0, e1 in evs)
    med = ms[len(ms) // 2]
    return {
        "workload": f"B={B},Hq={Hq},Hkv={Hkv},D=128,N={N},bf16,sink=64,window=elastic(seed 0, alpha "
                    f"U[{alpha_range[0]:g},{alpha_range[1]:g}], beta U[0,0.5])",
        "ms_per_layer": med,
        "ms_min": ms[0],
        "flops_live": flops,
        "flops_tiles": tile_flops,
        "tflops_live": flops / (med * 1e-3) / 1e12,
        "tflops_tiles": tile_flops / (med * 1e-3) / 1e12,
        "mfma_frac": flops / (med * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS,
        "mfma_peak_tflops": MFMA_PEAK_TFLOPS,
    }


def bench_prompt_side(torch, dev, iters=6):
    """The kernels between the projections and the attention in a prompt pass, at the layer shape of the
    7B end-to-end config (B=8, 32 heads, N=16384, D=128, bf16): the rotary embedding of q and k
    (moa_rope_fwd) and the bulk insert of the rotated k and of v into the rings
    (moa_cache_prefill_insert), without and with an attention mask (two batch rows left-padded).
    Algorithmic bytes: rotary = q and k read and written once + cos and sin; insert = the rows that are
    kept (per head min(N, cache size)) of k and of v read and written once + the ring bookkeeping."""
    from moa_amd import StaticCircularCache
    from moa_amd.kernels.rotary import apply_rotary_pos_emb
    from moa_amd.models.llama.modeling_llama import rotary_cos_sin
    from moa_amd.workloads import elastic_spans, ring_cache_sizes

    B, H, N, D, dtype = 8, 32, 16384, 128, torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(3)
    q, k, v = (torch.randn(B, N, H, D, generator=gen, device=dev, dtype=dtype).transpose(1, 2) for _ in range(3))
    cos, sin = rotary_cos_sin(torch.arange(N, device=dev)[None, :], D, dtype)
    cs, ss = ring_cache_sizes(elastic_spans(H, N, seed=0))

    def timed(fn, n):
        out = []
        for _ in range(n):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize(dev)
            out.append(e0.elapsed_time(e1))
        out.sort()
        return out[len(out) // 2] * 1e3   # us

    res = {"workload": f"B={B},H={H},N={N},D={D},bf16; rings = 64 sinks + elastic window (seed 0)"}
    for _ in range(2):
        apply_rotary_pos_emb(q, k, cos, sin)
    rope_us = timed(lambda: apply_rotary_pos_emb(q, k, cos, sin), iters)
    rope_bytes = 2 * (q.numel() + k.numel()) * 2 + 2 * cos.numel() * 2
    res["rope_prefill"] = {"us": rope_us, "bytes": rope_bytes, "GB/s": rope_bytes / rope_us / 1e3,
                           "frac_of_hbm_peak": rope_bytes / rope_us / 1e3 / HBM_PEAK_GBS,
                           "note": "includes torch's allocation of the two outputs (caching allocator, no hipMalloc after the first call)"}
    mask = torch.ones(B, N, dtype=torch.int64, device=dev)
    mask[1, :1000] = 0
    mask[5, :7777] = 0

    def insert_bytes(valid):   # valid tokens per batch row
        kept = sum(min(nv, c) for nv in valid for c in cs)
        return 2 * 2 * kept * D * 2 + 3 * 8 * B * H + 8 * kept

    for name, am, ins_bytes in (("prefill_insert", None, insert_bytes([N] * B)),
                                ("prefill_insert_masked", mask, insert_bytes(mask.sum(1).tolist()) + 8 * B * N)):
        us = []
        for i in range(iters + 1):
            cache = StaticCircularCache([cs], batch_size=B, head_dim=D, static_size=[ss], device=dev, dtype=dtype)
            cache._to_device(0, dev)      # the K/V allocation stays outside the timed region
            torch.cuda.synchronize(dev)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            cache.update(k, v, 0, attention_mask=am)
            e1.record()
            torch.cuda.synchronize(dev)
            if i:
                us.append(e0.elapsed_time(e1) * 1e3)
            del cache
        us.sort()
        med = us[len(us) // 2]
        res[name] = {"us": med, "bytes": ins_bytes, "GB/s": ins_bytes / med / 1e3,
                     "frac_of_hbm_peak": ins_bytes / med / 1e3 / HBM_PEAK_GBS}
    return res


def bench_prefill_c1(torch, dev, iters=20):
    """The CPU-reference configuration on the GPU kernel (fp16: the kernel has no fp32 path), to put a
    GPU time beside cpu_baseline.prefill_c1."""
    from moa_amd import mixture_of_sparse_attention
    from moa_amd.workloads import uniform_block_windows
    B, H, N, D = 1, 32, 2048, 64
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(B, N, H, D, generator=g).to(dev, torch.float16).transpose(1, 2) for _ in range(3))
    sink = torch.full((H,), 64, dtype=torch.int64, device=dev)
    local = torch.tensor(uniform_block_windows(H, seed=0), dtype=torch.int64, device=dev)
    for _ in range(3):
        mixture_of_sparse_attention(q, k, v, D ** -0.5, sink_size=sink, local_size=local)
    torch.cuda.synchronize(dev)
    evs = []
    for _ in range(iters):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        mixture_of_sparse_attention(q, k, v, D ** -0.5, sink_size=sink, local_size=local)
        e1.record()
        evs.append((e0, e1))
    torch.cuda.synchronize(dev)
    ms = sorted(a.elapsed_time(b) for a, b in evs)
    return {"workload": "B=1,H=32,D=64,N=2048,fp16,sink=64,window uniform in {256..1024}", "ms": ms[len(ms) // 2]}


def cpu_baseline(torch, args, budget_s=12.0):
    """The CPU oracle's restatement of the reference's dense debug decode
    (grouped SDPA over the packed cache, fp32, torch CPU threads), on whole
    batch rows of the same workload until ~budget_s of CPU time is spent.
    Scaled to tokens/s of the full step (all layers)."""
    import numpy as np
    from oracle.moa_oracle import decode_grouped_sdpa
    from moa_amd.workloads import elastic_spans, ring_cache_sizes

    H, D, L = 32, 128, args.layers
    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(5)
    spent = 0.0
    per_layer = []
    l = 0
    while spent < budget_s and len(per_layer) < 16 * L:
        sizes, _ = ring_cache_sizes(elastic_spans(H, args.ctx, seed=l % L))
        sumc = sum(sizes)
        kc = torch.randn(1, sumc, D, generator=g)
        vc = torch.randn(1, sumc, D, generator=g)
        hi = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
        for _ in range(4):   # four sequences' steps on this layer's cache (new query each)
            q = torch.randn(1, H, 1, D, generator=g)
            t0 = time.perf_counter()
            decode_grouped_sdpa(q, kc, vc, hi, D ** -0.5)
            dt = time.perf_counter() - t0
            per_layer.append(dt)
            spent += dt
        l += 1
    mean_layer = sum(per_layer) / len(per_layer)
    # one token of ONE sequence costs L layer passes; the batch is B such sequences
    tok_s = 1.0 / (mean_layer * L)
    return {
        "prefill_c1": cpu_prefill_c1(torch),
        "prefill_c2": cpu_prefill_c2_slice(torch),
        "append": cpu_append(torch, args),
        "value": tok_s,
        "unit": "tokens/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{len(per_layer)} (batch row, layer) decode passes of the same spans ({spent:.1f} s of CPU time), fp32 "
                  f"grouped SDPA on CPU; tokens/s = 1 / (mean pass time * {L} layers)",
    }


def cpu_prefill_c1(torch):
    """The CPU-reference configuration in full: one layer, B=1, 32 heads, head_dim 64, N=2048, fp32,
    64 sinks + a window from {256,...,1024} per head, through the oracle's dense masked attention
    (torch SDPA with a boolean mask, the arithmetic of the reference's dense path)."""
    from oracle.moa_oracle import count_live_pairs, prefill_masked_dense
    from moa_amd.workloads import uniform_block_windows
    B, H, N, D = 1, 32, 2048, 64
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(B, H, N, D, generator=g) for _ in range(3))
    ns, nl = [1] * H, [w // 64 for w in uniform_block_windows(H, seed=0)]
    prefill_masked_dense(q[:, :2], k[:, :2], v[:, :2], D ** -0.5, ns[:2], nl[:2])   # warm-up
    t0 = time.perf_counter()
    prefill_masked_dense(q, k, v, D ** -0.5, ns, nl)
    dt = time.perf_counter() - t0
    pairs = sum(count_live_pairs(N, a, b)[0] for a, b in zip(ns, nl))
    return {"seconds": dt, "cores": torch.get_num_threads(), "kind": "port",
            "workload": "B=1,H=32,D=64,N=2048,fp32,sink=64,window uniform in {256..1024}: dense masked SDPA, whole config",
            "gflops_live": 4.0 * D * pairs * B / dt / 1e9,
            "gflops_dense_causal": 4.0 * D * H * B * (N * (N + 1) / 2) / dt / 1e9}


def cpu_prefill_c2_slice(torch, heads=4):
    """A slice of the prefill benchmark configuration (B=4, H=32, D=128, N=8192) on the host cores: ONE
    batch row and the first `heads` heads through the oracle's dense masked attention in fp32 (the
    arithmetic of the reference's dense path), scaled linearly to the whole configuration (the work of
    a (batch row, head) pair on the dense path does not depend on its span)."""
    from oracle.moa_oracle import prefill_masked_dense
    from moa_amd.workloads import elastic_spans, prefill_work
    B, H, N, D = 4, 32, 8192, 128
    spans = elastic_spans(H, N, seed=0)
    g = torch.Generator().manual_seed(7)
    q, k, v = (torch.randn(1, heads, N, D, generator=g).to(torch.bfloat16).float() for _ in range(3))
    ns, nl = [1] * heads, [s // 64 for s in spans[:heads]]
    t0 = time.perf_counter()
    prefill_masked_dense(q, k, v, D ** -0.5, ns, nl)
    dt = time.perf_counter() - t0
    scale = B * H / heads
    flops_live, _, _ = prefill_work(N, [1] * H, [s // 64 for s in spans], B, D)
    return {"seconds_slice": dt, "seconds_whole_config_scaled": dt * scale, "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"1 of {B} batch rows x {heads} of {H} heads of B=4,H=32,D=128,N=8192 (bf16 values in fp32), dense masked SDPA; "
                      f"scaled by {scale:g} to the whole configuration",
            "gflops_live_scaled": flops_live / (dt * scale) / 1e9}


def cpu_append(torch, args, rows=8, steps=20):
    """The reference's decode-branch cache update (about 15 indexing operations per layer and step,
    MoA/attention/cache_utils.py:1020-1058) as the oracle restates it with numpy, on `rows` batch rows
    of one layer of the headline shape; the time of a whole batch is that times batch / rows (the work
    is per batch row)."""
    import numpy as np
    from oracle.moa_oracle import StaticCircularCacheOracle
    from moa_amd.workloads import elastic_spans, ring_cache_sizes
    H, D = 32, 128
    cs, ss = ring_cache_sizes(elastic_spans(H, args.ctx, seed=0))
    o = StaticCircularCacheOracle(cs, ss, rows, D, dtype=np.float16)
    o.cache_valid_length[:] = np.asarray(cs)[None, :]
    o.cache_update_index[:] = o.circular_cache_head_index[None, :]
    o.kv_len = args.ctx
    rng = np.random.default_rng(0)
    kn = rng.standard_normal((rows, H, 1, D)).astype(np.float16)
    o.update_decode(kn, kn)
    t0 = time.perf_counter()
    for _ in range(steps):
        o.update_decode(kn, kn)
    dt = (time.perf_counter() - t0) / steps
    return {"us_per_layer_step": dt * 1e6 * args.batch / rows, "cores": 1, "kind": "port",
            "sample": f"{steps} decode-branch updates of {rows} batch rows of one layer (H=32, D=128, fp16, ctx "
                      f"{args.ctx}), numpy index operations; scaled by {args.batch}/{rows} to the whole batch"}


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the path has no collectives); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    from moa_amd import _lib
    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.test_mode:
        from moa_amd import efficiency_test
        batch, prompt = (4, 32768) if args.shape == "70b" else (8, 16384)
        efficiency_test.run_model(efficiency_test.parse_args(
            ["--prefill_len", str(prompt), "--decode_len", str(args.new_tokens), "--batch_size", str(batch),
             "--model_name", args.shape, "--dtype", "bf16", "--test_mode", args.test_mode, "--cuda_event", "--cuda_cache"]
            + (["--moa_config", args.plan] if args.plan else [])))
        return
    if args.only == "copy":
        # calibration for the HBM traffic counters: a plain device copy of known size (1 GiB read,
        # 1 GiB written per launch by torch's elementwise copy kernel)
        n = 1 << 30
        x = torch.empty(n, dtype=torch.uint8, device=dev).random_(0, 255)
        y = torch.empty_like(x)
        for _ in range(5):
            y.copy_(x)
        torch.cuda.synchronize(dev)
        print(json.dumps({"copy_bytes_read": n, "copy_bytes_written": n, "launches": 5}))
        return
    if args.only == "e2e":
        print(json.dumps({"e2e": bench_e2e(torch, dev, args)}))
        return
    if args.only == "e2e-full":
        print(json.dumps({"e2e_full": bench_e2e_full(torch, dev, args)}))
        return
    if args.only == "prefill":
        print(json.dumps({"prefill": bench_prefill(torch, dev, args)}))
        return
    if args.only == "gqa":
        print(json.dumps({"decode_gqa": bench_decode_gqa(torch, dev, args)}))
        return
    if args.only == "prompt":
        print(json.dumps({"prompt_side": bench_prompt_side(torch, dev)}))
        return
    dec = bench_decode(torch, dev, args)
    rope = bench_rope_append(torch, dev, args, dec["cache"])
    del dec["cache"]
    if args.only == "decode":
        print(json.dumps({"decode": dec}))
        return
    torch.cuda.empty_cache()
    pre = None
    if not args.no_prefill:
        try:
            pre = bench_prefill(torch, dev, args)
            pre["cpu_reference_config"] = bench_prefill_c1(torch, dev)
            pre["grouped_query_32k"] = bench_prefill(torch, dev, args, B=1, Hq=64, Hkv=8, N=32768, iters=5,
                                                     alpha_range=C5_ALPHA_RANGE)
        except NotImplementedError as e:
            pre = {"error": str(e)}
    torch.cuda.empty_cache()
    gqa = bench_decode_gqa(torch, dev, args)
    prompt_side = bench_prompt_side(torch, dev)
    torch.cuda.empty_cache()
    e2e = None
    if not args.no_e2e:
        # the two end-to-end configurations as whole decoders (prompt pass, then greedy steps, eager and
        # replayed from a HIP graph): 7B shape with 256 steps, 70B grouped-query shape with 128
        import argparse as _ap
        e2e = {}
        for key, shape, steps in (("c4_7b", "7b", 256), ("c5_70b", "70b", 128)):
            try:
                e2e[key] = bench_e2e_full(torch, dev, _ap.Namespace(shape=shape, new_tokens=steps))
            except torch.cuda.OutOfMemoryError as e:   # a smaller card: say so instead of failing the line
                e2e[key] = {"error": "out of device memory: " + str(e)[:200]}
            torch.cuda.empty_cache()
    cpu = None if args.no_cpu else cpu_baseline(torch, args)

    line = {
        "metric": "decode tok/s (7B-shape, 16k ctx, bs64) + sparse prefill ms/layer; % roofline",
        "value": dec["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dec["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": f"decode+append: B={args.batch}, H=32, D=128, fp16, ctx={args.ctx}, "
                        f"{args.layers} layers/step, ring=64 sinks+elastic window (alpha U[64,2048], beta U[0,0.5]), "
                        "attention path only",
            "layers_per_step": args.layers,
            "distinct_layer_caches": dec["distinct_layer_caches"],
            "kv_rows_per_layer": dec["kv_rows_per_layer"],
        },
        "roofline": {
            "kernel": "decode_split_kernel (+merge)",
            "bound": "hbm",
            "achieved": dec["decode_gbs"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": dec["decode_gbs"] / HBM_PEAK_GBS,
            "traffic": DECODE_TRAFFIC_RATIO * dec["decode_bytes"],
            "traffic_source": "profiles/hbm_traffic_decode_and_prefill.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, "
                              "copy-kernel scaled; measured ratio to algorithmic bytes)",
            "bytes_per_launch": dec["decode_bytes"],
            "ms_per_launch": dec["decode_ms"],
        },
        "cpu_baseline": cpu,
        "append": {"us": dec["append_us"], "bytes": dec["append_bytes"], "GB/s": dec["append_gbs"]},
        "fused_rotary_step": dec["fused_rotary_step"],
        "rope_append": rope,
        "prefill": pre,
        "decode_gqa": gqa,
        "prompt_side": prompt_side,
        "e2e": e2e,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
