"""GPU parity of the block-sparse prefill kernel (mixture_of_sparse_attention ->
moa_prefill -> ctypes -> libmoa_hip.so) against the CPU oracle.

Tolerance: |out - oracle| <= 2e-3 + 1e-2 * |oracle|, the bound this path is specified with (max-abs
2e-3, relative 1e-2), applied the way the reference's tests apply theirs (assert_close).  fp16 is
compared with the oracle's dense masked attention in fp32; bf16 with the oracle that rounds the
softmax weights to bf16 where the kernel (and the reference's kernel, in fp16) rounds them, and, with
the outliers counted, with the unrounded one: see prefill_checks.py.  The reference has no bf16 prefill
to compare with (its kernel asserts fp16, MoA/kernels/block_sparse_attention_prefill.py:645-646)."""
import warnings

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle.moa_oracle import moa_token_mask, prefill_masked_dense, prefill_p_rounded
from prefill_checks import (check_prefill, close_counted, close_stated, masked_attention_gpu, stats)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _close(out, ref, tag):
    """fp16 results (and bf16 ones that no weight rounding can move) against a reference, every element."""
    close_stated(out, ref, tag)


def _qkv(B, H, N, D, dtype, dev, seed, hkv=None):
    g = torch.Generator().manual_seed(seed)
    hkv = hkv or H
    # projections come out as [B, N, H, D]; the operator gets [B, H, N, D] views of them
    q = torch.randn(B, N, H, D, generator=g).to(dev, dtype).transpose(1, 2)
    k = torch.randn(B, N, hkv, D, generator=g).to(dev, dtype).transpose(1, 2)
    v = torch.randn(B, N, hkv, D, generator=g).to(dev, dtype).transpose(1, 2)
    return q, k, v


def _run(q, k, v, sm, ns, nl, dev):
    from moa_amd import mixture_of_sparse_attention
    H = k.shape[1]
    sink = torch.tensor([x * 64 for x in ns], dtype=torch.int64, device=dev)
    local = torch.tensor([x * 64 for x in nl], dtype=torch.int64, device=dev)
    out = mixture_of_sparse_attention(q, k, v, sm, sink_size=sink, local_size=local)
    B, Hq, N, D = q.shape
    assert out.shape == (B, N, Hq, D) and out.dtype == q.dtype and out.is_contiguous()
    return out.transpose(1, 2)   # [B,H,N,D] like the oracle


def test_reference_prefill_test(dev):
    """The reference's own prefill test (tests/attention_kernel_test.py:35-76):
    uniform [0,1) fp16 data, B=2, H=4, N=128, D=128, sm_scale 0.1, sink 64 + local 64
    (dense causal), "sdpa" against "moa" at rtol = atol = 1e-3, output [B, N, H, D]."""
    from moa_amd import mixture_of_sparse_attention
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.rand(2, 4, 128, 128, generator=g).to(dev, torch.float16) for _ in range(3))
    sink = torch.full((4,), 64, dtype=torch.int64, device=dev)
    local = torch.full((4,), 64, dtype=torch.int64, device=dev)
    out = {}
    for impl in ("sdpa", "moa"):
        out[impl] = mixture_of_sparse_attention(q, k, v, 0.1, attention_dropout=0.0, implementation=impl,
                                                local_size=local, sink_size=sink)
        assert out[impl].shape == (2, 128, 4, 128)
    torch.testing.assert_close(out["sdpa"], out["moa"], rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("N", [64 * 5, 200, 333, 1000, 128, 65])
def test_small_against_oracle(dev, dtype, D, N):
    H = 6
    ns = [1, 0, 2, 1, 0, 3]
    nl = [2, 1, 1, 0, 3, 5]
    q, k, v = _qkv(2, H, N, D, dtype, dev, seed=N + D)
    sm = D ** -0.5
    out = _run(q, k, v, sm, ns, nl, dev)
    check_prefill(out, q, k, v, sm, ns, nl, (dtype, D, N))


@pytest.mark.parametrize("seed", range(24))
def test_random_plans_against_oracle(dev, seed):
    """Random lengths (ragged and long enough for several 256-row query tiles), random sink and band
    block counts per head incl. 0 and more than there are blocks: the tile schedule (sinks, rotated
    band, wrap, repeated last tile) against the dense masked oracle."""
    rng = np.random.default_rng(1000 + seed)
    D = int(rng.choice([64, 128]))
    dtype = [torch.float16, torch.bfloat16][seed % 2]
    N = int(rng.integers(65, 1800))
    nb = -(-N // 64)
    H = int(rng.integers(1, 7))
    ns = [int(x) for x in rng.integers(0, min(nb, 6) + 2, size=H)]
    nl = [int(x) for x in rng.integers(0, nb + 3, size=H)]
    if seed % 5 == 0:
        nl = [int(x) for x in rng.integers(0, 4, size=H)]      # narrow bands: many dead tiles per query tile
    q, k, v = _qkv(1 + seed % 2, H, N, D, dtype, dev, seed=seed)
    sm = D ** -0.5
    out = _run(q, k, v, sm, ns, nl, dev)
    check_prefill(out, q, k, v, sm, ns, nl, (seed, N, D, ns, nl))


@pytest.mark.parametrize("layout", ["fused_qkv", "contiguous_bhnd"])
def test_operand_layouts(dev, layout):
    """q, k, v as the three column slices of ONE fused projection output [B, N, (Hq + 2 Hkv) D] (token
    stride is that of the fused row, the slices start at different 16-byte-aligned offsets), and as
    contiguous [B, H, N, D] tensors (what a caller gets after .contiguous()): the operator takes both
    through their strides, without a copy."""
    B, Hq, Hkv, N, D = 2, 8, 2, 333, 128
    dtype = torch.float16
    g = torch.Generator().manual_seed(11)
    if layout == "fused_qkv":
        fused = torch.randn(B, N, (Hq + 2 * Hkv) * D, generator=g).to(dev, dtype)
        q = fused[..., :Hq * D].view(B, N, Hq, D).transpose(1, 2)
        k = fused[..., Hq * D:(Hq + Hkv) * D].view(B, N, Hkv, D).transpose(1, 2)
        v = fused[..., (Hq + Hkv) * D:].view(B, N, Hkv, D).transpose(1, 2)
        assert q.stride(2) == (Hq + 2 * Hkv) * D and not k.is_contiguous()
    else:
        q = torch.randn(B, Hq, N, D, generator=g).to(dev, dtype)
        k = torch.randn(B, Hkv, N, D, generator=g).to(dev, dtype)
        v = torch.randn(B, Hkv, N, D, generator=g).to(dev, dtype)
    ns, nl = [1, 0], [2, 4]
    sm = D ** -0.5
    out = _run(q, k, v, sm, ns, nl, dev)
    check_prefill(out, q, k, v, sm, ns, nl, ("layout", layout))


def test_dead_rows_are_zero(dev):
    """ns = nl = 0 sees nothing; nl = 0 with sinks sees only sink blocks."""
    q, k, v = _qkv(1, 2, 256, 128, torch.float16, dev, seed=3)
    out = _run(q, k, v, 0.1, [0, 1], [0, 0], dev)
    assert not out[:, 0].any()
    ref = prefill_masked_dense(q, k, v, 0.1, [0, 1], [0, 0])
    _close(out, ref, "dead")


def test_wide_windows_reduce_to_causal(dev):
    q, k, v = _qkv(1, 3, 1024, 128, torch.bfloat16, dev, seed=4)
    out = _run(q, k, v, 128 ** -0.5, [0, 16, 1], [16, 0, 99], dev)
    ref = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True, scale=128 ** -0.5)
    # nothing is masked but the future: the oracle's masks must reduce to the library's causal attention
    torch.testing.assert_close(prefill_masked_dense(q, k, v, 128 ** -0.5, [0, 16, 1], [16, 0, 99]), ref.cpu(),
                               rtol=1e-5, atol=1e-5)
    check_prefill(out, q, k, v, 128 ** -0.5, [0, 16, 1], [16, 0, 99], "causal")


@pytest.mark.parametrize("G", [4, 3])
def test_gqa(dev, G):
    """G query heads per kv head (2 kv heads): equals MHA with each kv head repeated G times."""
    q, k, v = _qkv(2, 2 * G, 448, 128, torch.float16, dev, seed=5, hkv=2)
    ns, nl = [1, 2], [2, 3]
    out = _run(q, k, v, 0.09, ns, nl, dev)
    kr, vr = k.repeat_interleave(G, dim=1), v.repeat_interleave(G, dim=1)
    ref = prefill_masked_dense(q, kr, vr, 0.09, [1] * G + [2] * G, [2] * G + [3] * G)
    _close(out, ref, ("gqa", G))


def test_many_heads_with_equal_and_extreme_spans(dev):
    """The span-sorted work schedule: 40 heads (13B shape, not a multiple of the 8 XCDs) with tied
    spans, heads that see nothing, heads wider than the prompt and block counts far out of range;
    every head against the oracle, and the result must not depend on the order of the heads."""
    B, H, N, D = 1, 40, 640, 64
    nb = N // 64
    rng = np.random.default_rng(11)
    ns = [int(x) for x in rng.integers(0, 3, size=H)]
    nl = [int(x) for x in rng.choice([0, 1, 2, 2, 2, 5, 5, nb, nb + 7], size=H)]
    ns[3], nl[3] = 0, 0
    q, k, v = _qkv(B, H, N, D, torch.float16, dev, seed=12)
    out = _run(q, k, v, D ** -0.5, ns, nl, dev)
    ref = prefill_masked_dense(q, k, v, D ** -0.5, ns, nl)
    _close(out, ref, "many heads")
    assert not out[:, 3].any()
    perm = [int(x) for x in rng.permutation(H)]
    outp = _run(q[:, perm], k[:, perm], v[:, perm], D ** -0.5, [ns[i] for i in perm], [nl[i] for i in perm], dev)
    assert torch.equal(outp, out[:, perm])
    # counts beyond the prompt (and negative ones) select the same tiles as their clamped values
    from moa_amd.kernels.mixture_of_attention import moa_prefill
    big = torch.tensor([10 ** 12 if n >= nb else n for n in nl], dtype=torch.int64, device=dev)
    neg = torch.tensor([-5 if n == 0 else n for n in ns], dtype=torch.int64, device=dev)
    out2 = moa_prefill(q.transpose(1, 2), k, v, num_global_blocks=neg, num_band_blocks=big, sm_scale=D ** -0.5)
    assert torch.equal(out2.transpose(1, 2), out)


def test_many_launches_in_flight_on_two_streams(dev):
    """The work queue of a launch is one of 256 slots of a device array, handed out in turn and cleared by
    the launch's last work-group.  600 launches of two different shapes, alternating between two streams
    with nothing waiting in between (so launches overlap and the slots go round more than twice): every
    result must equal that of the same call made alone, bit for bit."""
    shapes = [(2, 6, 700, 64, torch.float16, [1, 0, 2, 1, 1, 3], [2, 5, 1, 11, 3, 4]),
              (1, 4, 1300, 128, torch.bfloat16, [1, 1, 0, 2], [4, 21, 2, 7])]
    cases = []
    for i, (B, H, N, D, dtype, ns, nl) in enumerate(shapes):
        q, k, v = _qkv(B, H, N, D, dtype, dev, seed=70 + i)
        alone = _run(q, k, v, D ** -0.5, ns, nl, dev).clone()
        cases.append((q, k, v, D ** -0.5, ns, nl, alone))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = []
    for i in range(600):
        q, k, v, sm, ns, nl, alone = cases[i % 2]
        with torch.cuda.stream(streams[(i // 2) % 2]):
            outs.append((i % 2, _run(q, k, v, sm, ns, nl, dev)))
    torch.cuda.synchronize()
    for i, (c, out) in enumerate(outs):
        assert torch.equal(out, cases[c][6]), i


def test_gqa_70b_shape(dev):
    """The largest config's head layout: 64 query heads on 8 kv heads, head_dim 128, bf16 (its
    32k-token prompt shortened to 4096 so that the CPU oracle finishes in seconds)."""
    B, Hq, Hkv, N, D = 1, 64, 8, 4096, 128
    q, k, v = _qkv(B, Hq, N, D, torch.bfloat16, dev, seed=13, hkv=Hkv)
    ns, nl = [1] * Hkv, [4, 9, 17, 33, 2, 64, 12, 25]
    out = _run(q, k, v, D ** -0.5, ns, nl, dev)
    for hk in (0, 3, 5):
        sl = slice(hk * 8, hk * 8 + 8)
        check_prefill(out[:, sl], q[:, sl], k[:, hk:hk + 1], v[:, hk:hk + 1], D ** -0.5, [ns[hk]], [nl[hk]], ("70b", hk))


def test_more_heads_than_the_sorted_schedule_covers(dev):
    """Beyond 512 kv heads the span sort is skipped and heads are taken in the given order."""
    B, H, N, D = 1, 520, 128, 64
    rng = np.random.default_rng(21)
    ns = [int(x) for x in rng.integers(0, 2, size=H)]
    nl = [int(x) for x in rng.integers(0, 3, size=H)]
    q, k, v = _qkv(B, H, N, D, torch.float16, dev, seed=22)
    out = _run(q, k, v, D ** -0.5, ns, nl, dev)
    ref = prefill_masked_dense(q, k, v, D ** -0.5, ns, nl)
    _close(out, ref, "520 heads")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_peaked_and_drifting_scores(dev, dtype):
    """Scores in the hundreds (one-hot-like softmax) and a row maximum that keeps growing along the
    keys, so that the lazily updated softmax reference is rescaled many times."""
    B, H, N, D = 1, 4, 768, 128
    q, k, v = _qkv(B, H, N, D, dtype, dev, seed=31)
    q = (q * 6).contiguous()
    ramp = torch.linspace(0.2, 3.0, N, device=dev)[None, None, :, None]
    k = (k * ramp.to(dtype)).contiguous()          # later keys are larger: the running max drifts upward
    ns, nl = [1, 0, 2, 1], [12, 3, 5, 1]
    out = _run(q, k, v, D ** -0.5, ns, nl, dev)
    check_prefill(out, q, k, v, D ** -0.5, ns, nl, ("peaked", dtype))


def test_short_prompt_falls_back_to_dense(dev):
    """N <= 64: dense causal with a warning (mixture_of_attention.py:412-415), whatever the spans."""
    from moa_amd import mixture_of_sparse_attention
    q, k, v = _qkv(2, 3, 40, 64, torch.float16, dev, seed=6)
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        out = mixture_of_sparse_attention(q, k, v, 0.125)
        assert any("Falling back to dense" in str(x.message) for x in w)
    ref = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True, scale=0.125)
    _close(out.transpose(1, 2), ref, "short")


def test_invariants(dev):
    q, k, v = _qkv(2, 4, 704, 128, torch.float16, dev, seed=7)
    ns, nl = [1, 1, 0, 2], [3, 1, 4, 2]
    out = _run(q, k, v, 0.09, ns, nl, dev)
    ones = _run(q, k, torch.ones_like(v), 0.09, ns, nl, dev)
    assert (ones.float() - 1).abs().max().item() <= 1e-3
    perm = [2, 0, 3, 1]
    outp = _run(q[:, perm], k[:, perm], v[:, perm], 0.09, [ns[i] for i in perm], [nl[i] for i in perm], dev)
    assert torch.equal(outp, out[:, perm])
    outb = _run(q[1:], k[1:], v[1:], 0.09, ns, nl, dev)
    assert torch.equal(outb, out[1:])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_negative_and_zero_softmax_scale(dev, dtype):
    """The reference takes any float as sm_scale.  A negative one prefers the LEAST similar keys; zero
    gives uniform weights over the visible keys."""
    q, k, v = _qkv(1, 3, 400, 128, dtype, dev, seed=50)
    ns, nl = [1, 0, 1], [2, 3, 1]
    for sm in (-0.11, 0.0):
        out = _run(q, k, v, sm, ns, nl, dev)
        check_prefill(out, q, k, v, sm, ns, nl, ("scale", sm, dtype))


def test_cpu_reference_config(dev):
    """The CPU-reference configuration: one layer, 32 heads, head_dim 64, batch 1, seq 2048, 64 sinks,
    per-head window from {256,...,1024}; inputs N(0,1).  The GPU path runs it in
    fp16 (the config's fp32 is the oracle's arithmetic); whole output against the oracle."""
    from moa_amd.workloads import uniform_block_windows
    B, H, N, D = 1, 32, 2048, 64
    q, k, v = _qkv(B, H, N, D, torch.float16, dev, seed=0)
    win = uniform_block_windows(H, seed=0)
    ns, nl = [1] * H, [w // 64 for w in win]
    sm = D ** -0.5
    out = _run(q, k, v, sm, ns, nl, dev)
    ref = prefill_masked_dense(q, k, v, sm, ns, nl)
    _close(out, ref, "C1")


def test_prefill_config_scale(dev):
    """The benchmark's prefill configuration at full size (B=4, H=32, D=128, N=8192, bf16, elastic spans):
    (a) V == 1 => O == 1 everywhere; (b) three whole heads against the CPU oracle;
    (c) one batch element against torch's dense masked attention in fp32 on the GPU."""
    from moa_amd.workloads import elastic_spans
    B, H, N, D = 4, 32, 8192, 128
    q, k, v = _qkv(B, H, N, D, torch.bfloat16, dev, seed=1)
    spans = elastic_spans(H, N, seed=0)
    ns, nl = [1] * H, [s // 64 for s in spans]
    sm = D ** -0.5
    out = _run(q, k, v, sm, ns, nl, dev)
    ones = _run(q, k, torch.ones_like(v), sm, ns, nl, dev)
    assert (ones.float() - 1).abs().max().item() <= 8e-3   # bf16 output spacing near 1
    for b, h in [(0, int(np.argmin(nl))), (3, int(np.argmax(nl))), (2, 17)]:
        check_prefill(out[b:b + 1, h:h + 1], q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], sm,
                      [ns[h]], [nl[h]], ("config scale", b, h), max_fraction=1e-5)
    # one whole batch element on the GPU: the same two comparisons with torch ops in fp32
    b = 1
    outside = 0
    for h0 in range(0, H, 8):
        sl = (slice(b, b + 1), slice(h0, h0 + 8))
        mask = torch.stack([torch.from_numpy(moa_token_mask(N, ns[h], nl[h])) for h in range(h0, h0 + 8)]).to(dev)
        ref_p = masked_attention_gpu(q[sl], k[sl], v[sl], mask, sm, torch.bfloat16)
        close_stated(out[sl], ref_p, ("gpu dense, weights rounded", h0))
        ref = masked_attention_gpu(q[sl], k[sl], v[sl], mask, sm)
        ref_absv = masked_attention_gpu(q[sl], k[sl], v[sl].abs(), mask, sm)
        outside += close_counted(out[sl], ref, ref_absv, ("gpu dense", h0), max_fraction=1e-5)
    print(f"config scale, batch element 1: {outside} of {H * N * D} elements outside 2e-3 + 1e-2 |ref| "
          f"against the unrounded fp32 attention")


def test_gpu_restatement_of_the_rounded_oracle(dev):
    """masked_attention_gpu (used where the CPU oracle is too slow) against the CPU oracle."""
    B, H, N, D = 1, 3, 333, 64
    q, k, v = _qkv(B, H, N, D, torch.bfloat16, dev, seed=40)
    ns, nl = [1, 0, 2], [2, 1, 3]
    mask = torch.stack([torch.from_numpy(moa_token_mask(N, ns[h], nl[h])) for h in range(H)]).to(dev)
    for name, dt in ((None, None), ("bf16", torch.bfloat16), ("f16", torch.float16)):
        want = prefill_p_rounded(q, k, v, D ** -0.5, ns, nl, name)
        got = masked_attention_gpu(q, k, v, mask, D ** -0.5, dt).double().cpu().numpy()
        # fp32 scores against fp64 ones: a weight that sits on a rounding boundary may go the other way
        assert np.abs(got - want).max() < 1e-3 and np.mean(np.abs(got - want)) < 2e-6, name


def test_report_bf16_outliers(dev):
    """Not a check of its own: prints what the bf16 comparisons made so far in this process (prefill and
    grouped-query decode) measured against the exact oracle."""
    total = sum(x["elements"] for x in stats)
    outside = sum(x["outside_stated_bound"] for x in stats)
    worst = max((x["max_abs_err"] for x in stats), default=0.0)
    print(f"bf16 results against the exact oracle: {outside} of {total} elements outside "
          f"2e-3 + 1e-2 |ref| in {len(stats)} comparisons, largest error {worst:.3e}")
    for x in stats:
        if x["outside_stated_bound"]:
            print("   ", x)
    assert total > 0


def test_errors(dev):
    from moa_amd import mixture_of_sparse_attention
    q = torch.zeros(1, 2, 128, 128, dtype=torch.float32, device=dev)
    s = torch.tensor([64, 64], device=dev)
    with pytest.raises(AssertionError):   # fp32 (reference: block_sparse_attention_prefill.py:645-646)
        mixture_of_sparse_attention(q, q, q, 1.0, sink_size=s, local_size=s)
    q96 = torch.zeros(1, 2, 128, 96, dtype=torch.float16, device=dev)
    with pytest.raises(NotImplementedError):
        mixture_of_sparse_attention(q96, q96, q96, 1.0, sink_size=s, local_size=s)
    qa = torch.zeros(1, 2, 128, 128, dtype=torch.float16, device=dev)
    kb = torch.zeros(1, 2, 128, 64, dtype=torch.float16, device=dev)
    with pytest.raises(AssertionError):
        mixture_of_sparse_attention(qa, kb, qa, 1.0, sink_size=s, local_size=s)
