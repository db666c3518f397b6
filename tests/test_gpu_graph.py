"""The decode step (fused rotary + append, then ring decode) captured in a HIP graph and replayed:
every replay must equal the same step run eagerly.  The library enqueues kernels only (no
allocation, no synchronisation, no memset), which is what capture needs; the one host value it
takes, kv_len, only decides "still inside the sink part?" and is constant once the prompt is longer
than the sinks."""
import pytest
import torch

from oracle.moa_oracle import rope_cos_sin

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _make(dev, seed, G):
    """A cache of 4 rings that holds a 200-token prompt; G query heads per ring."""
    from moa_amd import StaticCircularCache
    B, H, D, S = 2, 4, 128, 200
    cache_size, static = [128, 192, 256, 128], [64] * 4
    cache = StaticCircularCache([cache_size], static_size=[static], batch_size=B, head_dim=D, device=dev,
                                dtype=torch.float16)
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H * G, S, D, generator=g).to(dev, torch.float16)
    k, v = (torch.randn(B, H, S, D, generator=g).to(dev, torch.float16) for _ in range(2))
    cos, sin = rope_cos_sin(torch.arange(S)[None, :], D, dtype=torch.float16)
    cache.rope_update(q, k, v, cos.to(dev), sin.to(dev), 0)
    return cache, (B, H, D, S)


def _step(cache, q, k, v, cos, sin, D):
    from moa_amd import mixture_of_sparse_attention
    qe, kc, vc = cache.rope_update(q, k, v, cos, sin, 0)
    return mixture_of_sparse_attention(qe, kc, vc, D ** -0.5, head_start_index=cache.cache_head_start_index[0],
                                       head_valid_length=cache.cache_valid_length[0])


@pytest.mark.parametrize("G", [1, 4])   # 1: vector-ALU decode kernel; 4: grouped-query kernel on the matrix cores
def test_decode_step_replays_like_eager(dev, G):
    cache_g, (B, H, D, S) = _make(dev, 0, G)   # driven by graph replays
    cache_e, _ = _make(dev, 0, G)              # driven eagerly, same prompt
    g = torch.Generator().manual_seed(1)
    steps = []
    for t in range(5):
        q = torch.randn(B, H * G, 1, D, generator=g).to(dev, torch.float16)
        k, v = (torch.randn(B, H, 1, D, generator=g).to(dev, torch.float16) for _ in range(2))
        cos, sin = rope_cos_sin(torch.full((1, 1), S + t), D, dtype=torch.float16)
        steps.append((q, k, v, cos.to(dev), sin.to(dev)))
    # static input buffers of the graph; step 0 runs eagerly on a side stream (warm-up: workspaces)
    sq, sk, sv, sc, ss = (x.clone() for x in steps[0])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        out0 = _step(cache_g, sq, sk, sv, sc, ss, D)
    torch.cuda.current_stream().wait_stream(side)
    ref0 = _step(cache_e, *steps[0], D)
    assert torch.equal(out0, ref0)
    graph = torch.cuda.CUDAGraph()
    for dst, src in zip((sq, sk, sv, sc, ss), steps[1]):
        dst.copy_(src)
    with torch.cuda.graph(graph):
        out_static = _step(cache_g, sq, sk, sv, sc, ss, D)
    # capture records, it does not run: step 1 happens at the first replay
    for t in range(1, 5):
        for dst, src in zip((sq, sk, sv, sc, ss), steps[t]):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        ref = _step(cache_e, *steps[t], D)          # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(out_static, ref), t
        assert torch.equal(cache_g.key_cache[0], cache_e.key_cache[0]), t
        assert torch.equal(cache_g.value_cache[0], cache_e.value_cache[0]), t
        assert torch.equal(cache_g.cache_update_index[0], cache_e.cache_update_index[0]), t
        assert torch.equal(cache_g.cache_valid_length[0], cache_e.cache_valid_length[0]), t
