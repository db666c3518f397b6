"""The ctypes stub that replaces ``from flashinfer import moa_prefill, moa_decode`` in the reference
(MoA/kernels/mixture_of_attention.py:22-30), run as a maintainer would run it: the reference's argument
order and layouts, results against the package's own operator (bit for bit) and the oracle."""
import numpy as np
import pytest
import torch

from oracle.moa_oracle import decode_segments, prefill_masked_dense
from prefill_checks import close_stated

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def test_prefill_through_the_stub(dev):
    from moa_amd import mixture_of_sparse_attention
    from moa_amd.kernels import minimal_binding as mb
    assert mb.CUDA_KERNEL_AVAILABLE
    B, H, N, D = 2, 4, 500, 128
    g = torch.Generator().manual_seed(3)
    q = torch.randn(B, N, H, D, generator=g).to(dev, torch.float16)            # the layout the reference passes (:437)
    k, v = (torch.randn(B, H, N, D, generator=g).to(dev, torch.float16) for _ in range(2))
    ns, nl = [1, 0, 2, 1], [2, 8, 1, 3]
    gb = torch.tensor(ns, dtype=torch.int64, device=dev)
    bb = torch.tensor(nl, dtype=torch.int64, device=dev)
    out = mb.moa_prefill(q, k, v, causal=True, num_global_blocks=gb, num_band_blocks=bb, kv_layout="HND",
                         sm_scale=D ** -0.5)
    assert out.shape == (B, N, H, D)
    want = mixture_of_sparse_attention(q.transpose(1, 2), k, v, D ** -0.5, sink_size=gb * 64, local_size=bb * 64)
    assert torch.equal(out, want)
    close_stated(out.transpose(1, 2), prefill_masked_dense(q.transpose(1, 2), k, v, D ** -0.5, ns, nl), "stub prefill")


def test_decode_through_the_stub(dev):
    from moa_amd import mixture_of_sparse_attention
    from moa_amd.kernels import minimal_binding as mb
    B, H, D = 3, 5, 128
    sizes = [128, 640, 64, 1100, 256]
    starts = np.concatenate([[0], np.cumsum(sizes)[:-1]])
    sumC = int(sum(sizes))
    g = torch.Generator().manual_seed(4)
    q = torch.randn(B, 1, H, D, generator=g).to(dev, torch.float16)
    k, v = (torch.randn(B, sumC, D, generator=g).to(dev, torch.float16) for _ in range(2))
    hs = torch.tensor(starts, dtype=torch.int64).expand(B, H).contiguous().to(dev)
    valid = torch.tensor([[128, 300, 0, 1100, 17], sizes, [1, 640, 64, 5, 256]], dtype=torch.int64).to(dev)
    out = mb.moa_decode(q, k, v, hs, valid, D ** -0.5)
    assert out.shape == (B, 1, H, D)
    want = mixture_of_sparse_attention(q.transpose(1, 2), k, v, D ** -0.5, head_start_index=hs,
                                       head_valid_length=valid)
    assert torch.equal(out, want)
    ref = decode_segments(q[:, 0].float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(),
                          hs.cpu().numpy(), valid.cpu().numpy(), D ** -0.5)
    close_stated(out[:, 0], torch.from_numpy(ref), "stub decode")
