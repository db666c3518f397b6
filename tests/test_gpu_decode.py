"""GPU parity of the split-K decode kernel (moa_decode -> ctypes ->
libmoa_hip.so) against the fp64 CPU oracle.

Tolerance (fp16/bf16 inputs, fp32 softmax, output rounded to the input dtype):
|out - oracle| <= 2e-3 + 1e-2 * |oracle|, the bound this path is specified with
(max-abs 2e-3, relative 1e-2), applied the way the reference's tests apply theirs (assert_close)."""
import numpy as np
import pytest
import torch

from oracle.moa_oracle import decode_segments
from prefill_checks import close_counted, close_stated

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-3, 1e-2


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _close(out, ref, tag):
    out = np.asarray(out, dtype=np.float64)
    err = np.abs(out - ref)
    bound = ATOL + RTOL * np.abs(ref)
    assert np.isfinite(out).all(), tag
    assert (err <= bound).all(), (tag, float(err.max()), float((err - bound).max()))


def _close_grouped(out, q, kc, vc, hs, hv, sm, G, tag):
    """The grouped-query kernel (matrix cores) rounds the softmax weights to the input type in front of
    P.V: the stated bound against the oracle that rounds them at the same place; against the exact
    oracle the stated bound for fp16 and, for bf16, the a-priori bound of that rounding with the
    elements outside the stated bound counted (prefill_checks.py)."""
    qn, kn, vn = q.float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy()
    name = "bf16" if out.dtype == torch.bfloat16 else "f16"
    close_stated(out, torch.from_numpy(decode_segments(qn, kn, vn, hs, hv, sm, group=G, p_dtype=name)),
                 (tag, "weights rounded"))
    ref = decode_segments(qn, kn, vn, hs, hv, sm, group=G)
    if name == "f16":
        close_stated(out, torch.from_numpy(ref), tag)
    else:
        close_counted(out, torch.from_numpy(ref),
                      torch.from_numpy(decode_segments(qn, kn, vn, hs, hv, sm, group=G, abs_v=True)), tag)


def _case(rng, B, sizes, D, dtype, dev, fill="full", scale=1.0):
    sizes = np.asarray(sizes)
    H = len(sizes)
    start = np.concatenate([[0], np.cumsum(sizes)[:-1]])
    sumc = int(sizes.sum())
    kc = torch.from_numpy(rng.standard_normal((B, sumc, D)).astype(np.float32) * scale).to(dev, dtype)
    vc = torch.from_numpy(rng.standard_normal((B, sumc, D)).astype(np.float32)).to(dev, dtype)
    q = torch.from_numpy(rng.standard_normal((B, H, 1, D)).astype(np.float32)).to(dev, dtype)
    hs = np.broadcast_to(start, (B, H)).astype(np.int64).copy()
    if fill == "full":
        hv = np.broadcast_to(sizes, (B, H)).astype(np.int64).copy()
    else:
        hv = rng.integers(0, sizes + 1, size=(B, H)).astype(np.int64)
    return q, kc, vc, hs, hv


def _run(q, kc, vc, hs, hv, sm_scale, dev):
    from moa_amd import mixture_of_sparse_attention
    out = mixture_of_sparse_attention(q, kc, vc, sm_scale, head_start_index=torch.from_numpy(hs).to(dev),
                                      head_valid_length=torch.from_numpy(hv).to(dev))
    B, H = hs.shape
    assert out.shape == (B, 1, H, q.shape[-1]) and out.dtype == q.dtype
    ref = decode_segments(q[:, :, 0].float().cpu().numpy(), kc.float().cpu().numpy(),
                          vc.float().cpu().numpy(), hs, hv, sm_scale)
    return out[:, 0].float().cpu().numpy(), ref


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [128, 64])
def test_heterogeneous_heads(dev, dtype, D):
    rng = np.random.default_rng(D + (1 if dtype == torch.bfloat16 else 0))
    # one-chunk heads, multi-chunk heads, sizes off the chunk grid
    sizes = [64, 128, 512, 576, 1024, 1344, 3008, 192, 640, 2112]
    q, kc, vc, hs, hv = _case(rng, 3, sizes, D, dtype, dev)
    out, ref = _run(q, kc, vc, hs, hv, D ** -0.5, dev)
    _close(out, ref, ("full", D, dtype))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_partial_fill_and_empty_heads(dev, dtype):
    rng = np.random.default_rng(7)
    sizes = [128, 640, 64, 1472, 257, 35, 1000]
    q, kc, vc, hs, hv = _case(rng, 4, sizes, 128, dtype, dev, fill="partial")
    hv[0, 0] = 0
    hv[1, 3] = 0
    hv[2, 5] = 1
    hv[3, 6] = 513
    # rows outside the valid part must be ignored, whatever they hold
    for b in range(4):
        for h in range(len(sizes)):
            s0, n = int(hs[b, h]), int(hv[b, h])
            kc[b, s0 + n:s0 + sizes[h]] = float("nan")
            vc[b, s0 + n:s0 + sizes[h]] = float("inf")
    out, ref = _run(q, kc, vc, hs, hv, 0.09, dev)
    _close(out, ref, "partial")
    assert not out[0, 0].any() and not out[1, 3].any()


@pytest.mark.parametrize("B", [64, 40])
@pytest.mark.parametrize("D", [128, 64])
def test_partial_fill_with_a_large_grid(dev, D, B):
    """Grids beyond the small-grid variant (half-length chunks): batch 64 takes the load-pipelined
    loop, batch 40 the plain loop with full-length chunks.  Ragged valid lengths, an empty head,
    lengths around the half-batch of rows the pipelined loop works in."""
    rng = np.random.default_rng(77 + D + B)
    sizes = [64, 576, 1344, 192, 2112, 128]
    q, kc, vc, hs, hv = _case(rng, B, sizes, D, torch.float16, dev, fill="partial")
    hv[0, :] = [1, 15, 16, 17, 33, 0]
    hv[1, :] = [31, 32, 63, 64, 65, 127]
    out, ref = _run(q, kc, vc, hs, hv, D ** -0.5, dev)
    _close(out, ref, ("large grid", D))


def test_peaked_softmax(dev):
    """Large score range: the running max must carry across chunks and waves."""
    rng = np.random.default_rng(11)
    q, kc, vc, hs, hv = _case(rng, 2, [2048, 700], 128, torch.float16, dev, scale=3.0)
    out, ref = _run(q, kc, vc, hs, hv, 0.3, dev)
    _close(out, ref, "peaked")


def test_ring_order_invariance_and_ones(dev):
    rng = np.random.default_rng(12)
    sizes = [320, 1088]
    q, kc, vc, hs, hv = _case(rng, 2, sizes, 128, torch.float16, dev)
    out, _ = _run(q, kc, vc, hs, hv, 0.1, dev)
    kc2, vc2 = kc.clone(), vc.clone()
    for h, n in enumerate(sizes):
        s0 = int(hs[0, h])
        shift = int(rng.integers(1, n))
        kc2[:, s0:s0 + n] = torch.roll(kc[:, s0:s0 + n], shift, dims=1)
        vc2[:, s0:s0 + n] = torch.roll(vc[:, s0:s0 + n], shift, dims=1)
    out2, _ = _run(q, kc2, vc2, hs, hv, 0.1, dev)
    assert np.abs(out - out2).max() <= 2e-3
    out3, _ = _run(q, kc, torch.ones_like(vc), hs, hv, 0.1, dev)
    assert np.abs(out3 - 1.0).max() <= 1e-3


def test_reference_decode_test_shape(dev):
    """Shape of the reference's decode test (tests/attention_kernel_test.py:78-138:
    bsz 2, one head, cache 64, head_dim 128, uniform [0,1) data), "moa" against the
    "sdpa" debug implementation at the reference's tolerance 1e-3."""
    from moa_amd import mixture_of_sparse_attention
    g = torch.Generator(device="cpu").manual_seed(0)
    q = torch.rand(2, 1, 1, 128, generator=g).to(dev, torch.float16)
    k = torch.rand(2, 64, 128, generator=g).to(dev, torch.float16)
    v = torch.rand(2, 64, 128, generator=g).to(dev, torch.float16)
    hs = torch.zeros(2, 1, dtype=torch.int64, device=dev)
    hv = torch.full((2, 1), 64, dtype=torch.int64, device=dev)
    outs = {}
    for impl in ("sdpa", "moa"):
        outs[impl] = mixture_of_sparse_attention(q, k, v, 1.0, attention_mask=None, attention_dropout=0.0,
                                                 head_start_index=hs, head_valid_length=hv,
                                                 implementation=impl)
        assert outs[impl].shape == (2, 1, 1, 128)
    torch.testing.assert_close(outs["sdpa"], outs["moa"], rtol=1e-3, atol=1e-3)


def test_many_heads_and_batch_one(dev):
    rng = np.random.default_rng(13)
    sizes = list(rng.integers(1, 12, size=64) * 64)
    q, kc, vc, hs, hv = _case(rng, 1, sizes, 128, torch.bfloat16, dev)
    out, ref = _run(q, kc, vc, hs, hv, 128 ** -0.5, dev)
    _close(out, ref, "64 heads")


def test_decode_config_scale(dev):
    """Benchmark-size decode config (B=64, H=32, D=128, fp16, rings 64 + elastic
    window at N=16384, full).  Checked (a) against the fp64 oracle on sampled
    (b, h) pairs, (b) V == 1 => O == 1 everywhere, (c) against the grouped dense
    debug path on the GPU for two whole batch rows."""
    from moa_amd import mixture_of_sparse_attention
    from moa_amd.workloads import elastic_spans, ring_cache_sizes
    B, H, D = 64, 32, 128
    spans = elastic_spans(H, 16384, seed=0)
    sizes, _ = ring_cache_sizes(spans)
    sizes = np.asarray(sizes)
    sumc = int(sizes.sum())
    gd = torch.Generator(device=dev).manual_seed(0)
    kc = torch.randn(B, sumc, D, generator=gd, device=dev, dtype=torch.float16)
    vc = torch.randn(B, sumc, D, generator=gd, device=dev, dtype=torch.float16)
    q = torch.randn(B, H, 1, D, generator=gd, device=dev, dtype=torch.float16)
    start = np.concatenate([[0], np.cumsum(sizes)[:-1]])
    hs = torch.from_numpy(np.broadcast_to(start, (B, H)).astype(np.int64).copy()).to(dev)
    hv = torch.from_numpy(np.broadcast_to(sizes, (B, H)).astype(np.int64).copy()).to(dev)
    sm = D ** -0.5
    out = mixture_of_sparse_attention(q, kc, vc, sm, head_start_index=hs, head_valid_length=hv)
    assert out.shape == (B, 1, H, D)
    rng = np.random.default_rng(0)
    pairs = [(int(rng.integers(B)), int(rng.integers(H))) for _ in range(24)] + [(0, int(np.argmax(sizes))), (63, int(np.argmin(sizes)))]
    for b, h in pairs:
        s0, n = int(start[h]), int(sizes[h])
        ref = decode_segments(q[b:b + 1, h:h + 1, 0].float().cpu().numpy(),
                              kc[b:b + 1, s0:s0 + n].float().cpu().numpy(),
                              vc[b:b + 1, s0:s0 + n].float().cpu().numpy(),
                              np.array([[0]]), np.array([[n]]), sm)
        _close(out[b, 0, h].float().cpu().numpy(), ref[0, 0], (b, h))
    ones = mixture_of_sparse_attention(q, kc, torch.ones_like(vc), sm, head_start_index=hs, head_valid_length=hv)
    assert (ones.float() - 1).abs().max().item() <= 1e-3
    dense = mixture_of_sparse_attention(q[:2], kc[:2], vc[:2], sm, head_start_index=hs[:2],
                                        head_valid_length=hv[:2], implementation="sdpa")
    torch.testing.assert_close(out[:2].float(), dense.float(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("G", [2, 3, 4, 5, 7, 8])
@pytest.mark.parametrize("D", [128, 64])
def test_grouped_query_decode(dev, dtype, G, D):
    """G query heads per ring (not in the reference, whose caller asserts one kv group,
    MoA/models/llama/modeling_llama.py:220-224): query head h reads ring h // G, like the prefill
    kernel and the oracle's decode_segments(group=G)."""
    from moa_amd import mixture_of_sparse_attention
    rng = np.random.default_rng(100 * G + D)
    sizes = [64, 576, 1344, 192, 2112, 35]
    B, Hkv = 2, len(sizes)
    _, kc, vc, hs, hv = _case(rng, B, sizes, D, dtype, dev, fill="partial")
    hv[0, 1] = 0                                   # an empty ring: its G outputs are zero
    q = torch.from_numpy(rng.standard_normal((B, Hkv * G, 1, D)).astype(np.float32)).to(dev, dtype)
    out = mixture_of_sparse_attention(q, kc, vc, D ** -0.5, head_start_index=torch.from_numpy(hs).to(dev),
                                      head_valid_length=torch.from_numpy(hv).to(dev))
    assert out.shape == (B, 1, Hkv * G, D)
    _close_grouped(out[:, 0], q[:, :, 0], kc, vc, hs, hv, D ** -0.5, G, ("gqa", G, D, dtype))
    assert not out[0, 0, G:2 * G].any()
    # the same rings read by one query head each (G = 1, the vector-ALU kernel, weights in fp32; G >= 2
    # runs on the matrix cores with the weights rounded to the input type) give the same rows within the
    # tolerance in fp16 (bf16 weights differ by up to 2^-8 each: covered by _close_grouped above)
    for g in (0, G - 1) if dtype == torch.float16 else ():
        q1 = q[:, g::G].contiguous()
        out1 = mixture_of_sparse_attention(q1, kc, vc, D ** -0.5, head_start_index=torch.from_numpy(hs).to(dev),
                                           head_valid_length=torch.from_numpy(hv).to(dev))
        torch.testing.assert_close(out1[:, 0].float(), out[:, 0, g::G].float(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("B", [2, 48])            # a grid smaller and larger than the chip
@pytest.mark.parametrize("G", [2, 8])
def test_grouped_query_boundaries_and_invariants(dev, G, B):
    """The matrix-core kernel's edges: valid lengths around its 32-key tile, a wave's share (512
    rows) and its 2048-row chunk; scores that keep raising the running max (keys grow along the
    ring); the order of the rows inside a ring does not matter; V == 1 gives O == 1."""
    from moa_amd import mixture_of_sparse_attention
    rng = np.random.default_rng(7 + G)
    D, dtype = 128, torch.float16
    lens = [1, 31, 32, 33, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 2047, 2048, 2049, 4097, 100]
    sizes = [max(64, -(-n // 64) * 64) for n in lens]
    Hkv = len(sizes)
    _, kc, vc, hs, hv = _case(rng, B, sizes, D, dtype, dev)
    hv[:] = np.asarray(lens)[None, :]
    hv[1, 3] = 0
    ramp = torch.linspace(0.2, 3.0, kc.shape[1], device=dev)[None, :, None]
    kc = (kc.float() * ramp).to(dtype)                      # later rows score higher: many rescales
    q = torch.from_numpy(rng.standard_normal((B, Hkv * G, 1, D)).astype(np.float32) * 2).to(dev, dtype)
    hs_t, hv_t = torch.from_numpy(hs).to(dev), torch.from_numpy(hv).to(dev)
    out = mixture_of_sparse_attention(q, kc, vc, D ** -0.5, head_start_index=hs_t, head_valid_length=hv_t)
    rows = [0, 1, B - 1]                                    # the CPU oracle on three batch rows
    _close_grouped(out[rows, 0], q[rows][:, :, 0], kc[rows], vc[rows], hs[rows], hv[rows], D ** -0.5, G,
                   ("gqa edges", G, B))
    # reverse the valid rows of every ring (K and V alike): same softmax, same output
    kc2, vc2 = kc.clone(), vc.clone()
    for b in rows:
        for h in range(Hkv):
            s0, n = int(hs[b, h]), int(hv[b, h])
            kc2[b, s0:s0 + n] = kc[b, s0:s0 + n].flip(0)
            vc2[b, s0:s0 + n] = vc[b, s0:s0 + n].flip(0)
    out2 = mixture_of_sparse_attention(q, kc2, vc2, D ** -0.5, head_start_index=hs_t, head_valid_length=hv_t)
    torch.testing.assert_close(out2.float(), out.float(), rtol=RTOL, atol=ATOL)
    ones = mixture_of_sparse_attention(q, kc, torch.ones_like(vc), D ** -0.5, head_start_index=hs_t,
                                       head_valid_length=hv_t)
    expect = torch.ones_like(ones)
    expect[1, 0, 3 * G:4 * G] = 0                           # the empty ring
    assert (ones.float() - expect.float()).abs().max().item() <= 1e-3


@pytest.mark.parametrize("B", [1, 2])
def test_grouped_query_small_batch_even_split(dev, B):
    """Batch 1 and 2 at the largest config's ring sizes (8 rings of 2 k to 24 k rows, 8 query heads each,
    bf16): too few 2048-row chunks for the chip, so the kernel splits every batch row evenly into its share
    of 256 chunks, with a chunk length per ring found on the device from the valid lengths.  The batch rows
    are filled differently (full; partly, with one empty ring and one of a single row), so each has its own
    table; whole output against the oracle."""
    from moa_amd import mixture_of_sparse_attention
    from moa_amd.workloads import elastic_spans, ring_cache_sizes
    rng = np.random.default_rng(300 + B)
    G, D, dtype = 8, 128, torch.bfloat16
    sizes = ring_cache_sizes(elastic_spans(8, 32768, seed=3, alpha_range=(256.0, 8192.0)))[0]
    Hkv = len(sizes)
    _, kc, vc, hs, hv = _case(rng, B, sizes, D, dtype, dev)
    if B > 1:
        hv[1] = np.maximum(1, (hv[1] * rng.uniform(0.05, 0.9, size=Hkv)).astype(np.int64))
        hv[1, 2], hv[1, 5] = 0, 1
    q = torch.from_numpy(rng.standard_normal((B, Hkv * G, 1, D)).astype(np.float32)).to(dev, dtype)
    out = mixture_of_sparse_attention(q, kc, vc, D ** -0.5, head_start_index=torch.from_numpy(hs).to(dev),
                                      head_valid_length=torch.from_numpy(hv).to(dev))
    _close_grouped(out[:, 0], q[:, :, 0], kc, vc, hs, hv, D ** -0.5, G, ("gqa even split", B))
    if B > 1:
        assert not out[1, 0, 2 * G:3 * G].any()


@pytest.mark.parametrize("seed", range(16))
def test_random_layouts(dev, seed):
    """Segments anywhere in the packed row (gaps between them, not in head order), random valid
    lengths incl. 0, 1..8 query heads per ring, both head dims and dtypes."""
    from moa_amd import mixture_of_sparse_attention
    rng = np.random.default_rng(500 + seed)
    D = int(rng.choice([64, 128]))
    dtype = [torch.float16, torch.bfloat16][seed % 2]
    G = int(rng.integers(1, 9))
    B, Hkv = int(rng.integers(1, 4)), int(rng.integers(1, 9))
    cap = rng.integers(1, 3000, size=Hkv)
    gaps = rng.integers(0, 200, size=Hkv + 1)
    order = rng.permutation(Hkv)
    start = np.zeros(Hkv, dtype=np.int64)
    pos = int(gaps[0])
    for j, h in enumerate(order):
        start[h] = pos
        pos += int(cap[h]) + int(gaps[j + 1])
    sumc = pos
    hs = np.broadcast_to(start, (B, Hkv)).copy()
    hv = rng.integers(0, cap + 1, size=(B, Hkv)).astype(np.int64)
    hv[rng.integers(B), rng.integers(Hkv)] = 0
    kc = torch.from_numpy(rng.standard_normal((B, sumc, D)).astype(np.float32)).to(dev, dtype)
    vc = torch.from_numpy(rng.standard_normal((B, sumc, D)).astype(np.float32)).to(dev, dtype)
    q = torch.from_numpy(rng.standard_normal((B, Hkv * G, 1, D)).astype(np.float32)).to(dev, dtype)
    out = mixture_of_sparse_attention(q, kc, vc, D ** -0.5, head_start_index=torch.from_numpy(hs).to(dev),
                                      head_valid_length=torch.from_numpy(hv).to(dev))
    if G > 1:
        _close_grouped(out[:, 0], q[:, :, 0], kc, vc, hs, hv, D ** -0.5, G, ("random layout", seed, G, D))
        return
    ref = decode_segments(q[:, :, 0].float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy(),
                          hs, hv, D ** -0.5, group=G)
    _close(out[:, 0].float().cpu().numpy(), ref, ("random layout", seed, G, D))


def test_grouped_query_70b_shape(dev):
    """The 70B shape of the largest config: 64 query heads on 8 rings, head_dim 128, B = 4."""
    from moa_amd import mixture_of_sparse_attention
    rng = np.random.default_rng(5)
    sizes = [4096, 1024, 8192, 2048, 6144, 512, 3072, 7168]
    q_, kc, vc, hs, hv = _case(rng, 4, sizes, 128, torch.bfloat16, dev)
    q = torch.from_numpy(rng.standard_normal((4, 64, 1, 128)).astype(np.float32)).to(dev, torch.bfloat16)
    out = mixture_of_sparse_attention(q, kc, vc, 128 ** -0.5, head_start_index=torch.from_numpy(hs).to(dev),
                                      head_valid_length=torch.from_numpy(hv).to(dev))
    _close_grouped(out[:, 0], q[:, :, 0], kc, vc, hs, hv, 128 ** -0.5, 8, "70b")


def test_maximum_head_count(dev):
    """256 rings per batch row is the limit of the chunk table; one more is refused."""
    from moa_amd import mixture_of_sparse_attention
    rng = np.random.default_rng(31)
    sizes = [int(x) for x in rng.choice([64, 128, 576], size=256)]
    q, kc, vc, hs, hv = _case(rng, 2, sizes, 64, torch.float16, dev, fill="partial")
    out, ref = _run(q, kc, vc, hs, hv, 0.125, dev)
    _close(out, ref, "256 heads")
    q2 = torch.zeros(1, 257, 1, 64, dtype=torch.float16, device=dev)
    k2 = torch.zeros(1, 257 * 64, 64, dtype=torch.float16, device=dev)
    hs2 = (torch.arange(257, device=dev) * 64)[None, :]
    hv2 = torch.full((1, 257), 64, device=dev)
    with pytest.raises(NotImplementedError):
        mixture_of_sparse_attention(q2, k2, k2, 0.125, head_start_index=hs2, head_valid_length=hv2)


@pytest.mark.parametrize("G", [1, 4])
def test_overlapping_segments_stay_defined(dev, G):
    """Valid lengths that exceed the rings (what the cache's bookkeeping holds after a second prompt
    insert, as in the reference: cache_utils.py:1136-1138 does not clamp): the segments overlap, a batch
    row has more chunks than partial slots, and the chunk table is cut at the slot count in every kernel
    alike.  Every output element must be written and finite; heads in front of the cut are exact."""
    from moa_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(77 + G)
    B, H, D, C = 2, 4, 128, 256
    sumC = H * C
    dtype = torch.float16
    kc = torch.from_numpy(rng.standard_normal((B, sumC, D)).astype(np.float32)).to(dev, dtype)
    vc = torch.from_numpy(rng.standard_normal((B, sumC, D)).astype(np.float32)).to(dev, dtype)
    q = torch.from_numpy(rng.standard_normal((B, H * G, D)).astype(np.float32)).to(dev, dtype)
    hs = np.broadcast_to(np.arange(H) * C, (B, H)).astype(np.int64).copy()
    hv = (sumC - hs).astype(np.int64)                      # every head runs to the end of the row
    hv[1, 0] = 5 * sumC                                    # and one far beyond it
    o = torch.full((B, H * G, D), float("nan"), dtype=dtype, device=dev)
    need = lib.moa_decode_workspace_bytes(B, H * G, H, D, sumC)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    hs_d, hv_d = torch.from_numpy(hs).to(dev), torch.from_numpy(hv).to(dev)
    rc = lib.moa_decode_fwd(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), o.data_ptr(), ws.data_ptr(), ws.numel(),
                            hs_d.data_ptr(), hv_d.data_ptr(), B, H * G, H, D, sumC, D ** -0.5,
                            _lib.dtype_code(dtype), _lib.current_stream_ptr(dev))
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all()
    # head 0 of batch row 0 spans the whole row and lies in front of the cut for every chunk length
    hv_clamped = np.minimum(hv, sumC - hs)
    name = None if G == 1 else "f16"
    ref = decode_segments(q.float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy(), hs,
                          hv_clamped, D ** -0.5, group=G, p_dtype=name)
    err = np.abs(o[0, :G].float().cpu().numpy() - ref[0, :G])
    assert (err <= ATOL + RTOL * np.abs(ref[0, :G])).all(), float(err.max())


def test_errors(dev):
    from moa_amd import mixture_of_sparse_attention
    q = torch.zeros(1, 2, 1, 128, dtype=torch.float32, device=dev)
    k = torch.zeros(1, 256, 128, dtype=torch.float32, device=dev)
    hs = torch.tensor([[0, 128]], device=dev)
    hv = torch.tensor([[128, 128]], device=dev)
    with pytest.raises(AssertionError):      # fp32 is not a decode dtype (reference: mixture_of_attention.py:215-216)
        mixture_of_sparse_attention(q, k, k, 1.0, head_start_index=hs, head_valid_length=hv)
    with pytest.raises(NotImplementedError):
        mixture_of_sparse_attention(q.half(), k.half(), k.half(), 1.0, head_start_index=hs,
                                    head_valid_length=hv, implementation="nope")
    q96 = torch.zeros(1, 2, 1, 96, dtype=torch.float16, device=dev)
    k96 = torch.zeros(1, 256, 96, dtype=torch.float16, device=dev)
    with pytest.raises(NotImplementedError):  # head_dim 96 is not covered
        mixture_of_sparse_attention(q96, k96, k96, 1.0, head_start_index=hs, head_valid_length=hv)
    q18 = torch.zeros(1, 18, 1, 128, dtype=torch.float16, device=dev)
    with pytest.raises(NotImplementedError):  # 9 query heads per ring: more than the kernel's 8
        mixture_of_sparse_attention(q18, k.half(), k.half(), 1.0, head_start_index=hs, head_valid_length=hv)
    q3 = torch.zeros(1, 3, 1, 128, dtype=torch.float16, device=dev)
    with pytest.raises(AssertionError):       # 3 query heads do not divide over 2 rings
        mixture_of_sparse_attention(q3, k.half(), k.half(), 1.0, head_start_index=hs, head_valid_length=hv)
