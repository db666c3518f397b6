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


def test_prompt_pass_replays_like_eager(dev):
    """The prompt side recorded into a HIP graph: rotary embedding, block-sparse prefill (its work queue is
    a slot of a device array chosen at record time: every replay of the graph reuses that slot, one after
    the other on a stream), bulk insert into the rings.  One ordinary call comes first, as the header asks
    (the first call on a device looks up device addresses, which a capture cannot contain).  Every replay
    runs on new inputs and must equal the same calls run eagerly, bit for bit, rings and indices included."""
    import copy

    from moa_amd import StaticCircularCache, mixture_of_sparse_attention
    from moa_amd.kernels.rotary import apply_rotary_pos_emb
    B, Hq, Hkv, N, D = 2, 8, 4, 1000, 128
    dtype = torch.bfloat16
    sink = torch.tensor([64, 64, 128, 0], device=dev)
    local = torch.tensor([128, 512, 256, 1024], device=dev)
    cache_size = [int(s + l) for s, l in zip(sink.tolist(), local.tolist())]
    cos, sin = rope_cos_sin(torch.arange(N)[None, :].expand(B, N), D, dtype=dtype)
    cos, sin = cos.to(dev), sin.to(dev)

    def fresh_cache():
        return StaticCircularCache([cache_size], static_size=[sink.tolist()], batch_size=B, head_dim=D, device=dev,
                                   dtype=dtype)

    def prompt(cache, q, k, v):
        qe, ke = apply_rotary_pos_emb(q, k, cos, sin)
        out = mixture_of_sparse_attention(qe, ke, v, D ** -0.5, sink_size=sink, local_size=local)
        cache.update(ke, v, 0)
        return out

    g = torch.Generator().manual_seed(5)
    def draw():
        q = torch.randn(B, N, Hq, D, generator=g).to(dev, dtype).transpose(1, 2)
        k, v = (torch.randn(B, N, Hkv, D, generator=g).to(dev, dtype).transpose(1, 2) for _ in range(2))
        return q, k, v

    q0, k0, v0 = draw()
    prompt(fresh_cache(), q0, k0, v0)            # set-up calls outside any capture
    torch.cuda.synchronize()

    sq, sk, sv = (t.clone() for t in (q0, k0, v0))   # static inputs of the graph
    cache_g = fresh_cache()
    cache_g._to_device(0, dev)                       # rings and index arrays allocated before the state is saved
    pristine = copy.deepcopy(cache_g)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        prompt(copy.deepcopy(pristine), sq, sk, sv)  # allocator warm-up on the capture stream
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            out_g = prompt(cache_g, sq, sk, sv)
    torch.cuda.current_stream().wait_stream(stream)

    index_names = ("cache_update_index", "cache_valid_length", "mask_cache")
    for rep in range(3):
        q, k, v = draw()
        # the rings and indices go back to their state at record time, with fill kernels (copy_)
        cache_g.key_cache[0].copy_(pristine.key_cache[0]); cache_g.value_cache[0].copy_(pristine.value_cache[0])
        for name in index_names:
            getattr(cache_g, name)[0].copy_(getattr(pristine, name)[0])
        sq.copy_(q); sk.copy_(k); sv.copy_(v)
        graph.replay()
        torch.cuda.synchronize()
        cache_e = copy.deepcopy(pristine)
        out_e = prompt(cache_e, q, k, v)
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e), rep
        assert torch.equal(cache_g.key_cache[0], cache_e.key_cache[0]) and torch.equal(cache_g.value_cache[0], cache_e.value_cache[0]), rep
        for name in index_names:
            assert torch.equal(getattr(cache_g, name)[0], getattr(cache_e, name)[0]), (rep, name)
