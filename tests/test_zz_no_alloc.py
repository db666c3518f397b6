"""moa_decode_fwd_noalloc (the decode entry point that allocates nothing: its split-K partials live
in a scratch array inside the library's device image) against moa_decode_fwd with a caller-owned
workspace, both called through the raw C ABI.

The two share their kernels and their launch geometry, so the outputs must be bit-identical, which
is inside the decode bound |out - ref| <= 2e-3 + 1e-2 |ref| by a wide margin; the workspace path is
itself checked against the fp64 oracle here, at that bound.  Every case makes two calls in a row,
the second on a smaller input, so that whatever the first call left in the shared scratch is there
when the second runs."""
import numpy as np
import pytest
import torch

from oracle.moa_oracle import decode_segments

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-3, 1e-2


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _inputs(rng, B, sizes, G, D, dtype, dev, partial):
    sizes = np.asarray(sizes)
    H = len(sizes)
    start = np.concatenate([[0], np.cumsum(sizes)[:-1]])
    sumc = int(sizes.sum())
    kc = torch.from_numpy(rng.standard_normal((B, sumc, D)).astype(np.float32)).to(dev, dtype)
    vc = torch.from_numpy(rng.standard_normal((B, sumc, D)).astype(np.float32)).to(dev, dtype)
    q = torch.from_numpy(rng.standard_normal((B, H * G, D)).astype(np.float32)).to(dev, dtype)
    hs = np.broadcast_to(start, (B, H)).astype(np.int64).copy()
    hv = np.broadcast_to(sizes, (B, H)).astype(np.int64).copy()
    if partial:
        hv = rng.integers(0, sizes + 1, size=(B, H)).astype(np.int64)
        hv[0, 0] = 0
    return q, kc, vc, hs, hv


def _both(q, kc, vc, hs, hv, sm_scale, dev):
    """(output of moa_decode_fwd_noalloc, output of moa_decode_fwd) through ctypes."""
    from moa_amd import _lib
    lib = _lib.load()
    B, Hq, D = q.shape
    Hkv = hs.shape[1]
    sumC = kc.shape[1]
    hs_d, hv_d = torch.from_numpy(hs).to(dev), torch.from_numpy(hv).to(dev)
    stream = _lib.current_stream_ptr(dev)
    code = _lib.dtype_code(q.dtype)
    need = lib.moa_decode_workspace_bytes(B, Hq, Hkv, D, sumC)
    assert need <= _lib.MOA_DECODE_NOALLOC_MAX_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    o_ws = torch.full_like(q, float("nan"))
    o_na = torch.full_like(q, float("nan"))
    rc = lib.moa_decode_fwd(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), o_ws.data_ptr(), ws.data_ptr(), ws.numel(),
                            hs_d.data_ptr(), hv_d.data_ptr(), B, Hq, Hkv, D, sumC, sm_scale, code, stream)
    assert rc == 0, _lib.last_error()
    rc = lib.moa_decode_fwd_noalloc(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), o_na.data_ptr(),
                                    hs_d.data_ptr(), hv_d.data_ptr(), B, Hq, Hkv, D, sumC, sm_scale, code, stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    return o_na, o_ws


def _check(q, kc, vc, hs, hv, G, dev, tag):
    D = q.shape[-1]
    sm = D ** -0.5
    o_na, o_ws = _both(q, kc, vc, hs, hv, sm, dev)
    assert torch.isfinite(o_na.float()).all(), tag
    assert torch.equal(o_na, o_ws), (tag, (o_na.float() - o_ws.float()).abs().max().item())
    # with several query heads per ring the kernel rounds the softmax weights to the input type in front
    # of P.V; the oracle does it at the same place
    name = None if G == 1 else ("bf16" if q.dtype == torch.bfloat16 else "f16")
    ref = decode_segments(q.float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy(), hs, hv, sm,
                          group=G, p_dtype=name)
    err = np.abs(o_na.float().cpu().numpy() - ref)
    assert (err <= ATOL + RTOL * np.abs(ref)).all(), (tag, float(err.max()))


@pytest.mark.parametrize("G,dtype,D", [(1, torch.float16, 128), (1, torch.bfloat16, 64),
                                       (4, torch.bfloat16, 128), (8, torch.float16, 128)])
def test_two_calls_in_a_row_second_one_smaller(dev, G, dtype, D):
    rng = np.random.default_rng(100 + G + D)
    big = [64, 3008, 576, 1344, 4160, 192, 2112, 9000]      # several chunks per head at every chunk length
    small = [640, 64, 1100]
    first = _inputs(rng, 5, big, G, D, dtype, dev, partial=False)
    second = _inputs(rng, 2, small, G, D, dtype, dev, partial=True)
    _check(*first, G, dev, ("first", G, dtype, D))
    _check(*second, G, dev, ("second", G, dtype, D))
    # and the first again: the smaller call's leftovers must not matter either
    _check(*first, G, dev, ("first again", G, dtype, D))


def test_sizes_beyond_the_scratch_are_rejected(dev):
    from moa_amd import _lib
    lib = _lib.load()
    B, H, D = 64, 32, 128
    sumC = 400_000           # needs more than the 32 MiB the library holds
    assert lib.moa_decode_workspace_bytes(B, H, H, D, sumC) > _lib.MOA_DECODE_NOALLOC_MAX_BYTES
    x = torch.zeros(16, dtype=torch.float16, device=dev)    # never touched: the call is refused before any launch
    i = torch.zeros(B * H, dtype=torch.int64, device=dev)
    rc = lib.moa_decode_fwd_noalloc(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), i.data_ptr(),
                                    i.data_ptr(), B, H, H, D, sumC, 1.0, 0, None)
    assert rc == _lib.MOA_ERR_WORKSPACE
    assert "scratch" in _lib.last_error()


def test_headline_shape_fits(dev):
    """Batch 64, 32 heads, about 1.8e5 cache rows per batch row (the benchmark's decode launch) fits."""
    from moa_amd import _lib
    lib = _lib.load()
    assert lib.moa_decode_workspace_bytes(64, 32, 32, 128, 190_000) <= _lib.MOA_DECODE_NOALLOC_MAX_BYTES


def test_recorded_into_a_hip_graph(dev):
    """After one ordinary call (which does the per-device and per-kernel set-up), the entry point can be
    recorded into a HIP graph: it allocates nothing and its scratch sits at a fixed address.  Every replay,
    with eager work between the replays, gives the bits of the eager call."""
    from moa_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(7)
    q, kc, vc, hs, hv = _inputs(rng, 3, [64, 3008, 576, 1344], 4, 128, torch.bfloat16, dev, partial=True)
    B, Hq, D = q.shape
    Hkv, sumC = hs.shape[1], kc.shape[1]
    hs_d, hv_d = torch.from_numpy(hs).to(dev), torch.from_numpy(hv).to(dev)
    code = _lib.dtype_code(q.dtype)

    def call(o):
        rc = lib.moa_decode_fwd_noalloc(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), o.data_ptr(), hs_d.data_ptr(),
                                        hv_d.data_ptr(), B, Hq, Hkv, D, sumC, D ** -0.5, code, _lib.current_stream_ptr(dev))
        assert rc == 0, _lib.last_error()

    eager = torch.empty_like(q)
    call(eager)                       # the ordinary call that comes first
    torch.cuda.synchronize()
    o_graph = torch.full_like(q, float("nan"))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(o_graph)
    for i in range(3):
        o_graph.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o_graph, eager), i
        # eager work between the replays: new queries through the same scratch
        q2 = torch.randn_like(q)
        o2 = torch.empty_like(q)
        rc = lib.moa_decode_fwd_noalloc(q2.data_ptr(), kc.data_ptr(), vc.data_ptr(), o2.data_ptr(), hs_d.data_ptr(),
                                        hv_d.data_ptr(), B, Hq, Hkv, D, sumC, D ** -0.5, code, _lib.current_stream_ptr(dev))
        assert rc == 0
        torch.cuda.synchronize()
