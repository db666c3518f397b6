"""GPU parity of the circular-cache kernels (through StaticCircularCache ->
ctypes -> libmoa_hip.so) against the reference's vectors, the CPU oracle and an
independent torch restatement.  Everything here is integer/byte work: the bar
is bit-exact."""
import json
import os

import numpy as np
import pytest
import torch

from oracle.moa_oracle import StaticCircularCacheOracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from moa_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _payload(B, H, S, D, base):
    t = np.arange(S, dtype=np.float32)[None, None, :, None]
    h = np.arange(H, dtype=np.float32)[None, :, None, None] * 1000.0
    b = np.arange(B, dtype=np.float32)[:, None, None, None] * 100000.0
    return np.broadcast_to(base + b + h + t, (B, H, S, D)).copy()


def _assert_state(cache, o, tag):
    assert cache.cache_update_index[0].cpu().numpy().tolist() == o.cache_update_index.tolist(), tag
    assert cache.cache_valid_length[0].cpu().numpy().tolist() == o.cache_valid_length.tolist(), tag
    mc = cache.mask_cache[0].cpu().numpy()
    assert np.array_equal(mc, o.mask_cache), tag
    assert cache._kv_len[0] == o.kv_len, tag
    m = o.mask_cache == 1
    kc = cache.key_cache[0].float().cpu().numpy()
    vc = cache.value_cache[0].float().cpu().numpy()
    assert np.array_equal(kc[m], o.key_cache[m]), tag
    assert np.array_equal(vc[m], o.value_cache[m]), tag
    # rows never written stay zero
    assert not kc[~m].any() and not vc[~m].any(), tag


def test_reference_vectors_on_gpu(dev, golden_dir):
    """Replays the cases written by the reference's own cache and checks every
    recorded step (fp32 payload, head_dim 8)."""
    from moa_amd import StaticCircularCache
    golden = json.load(open(os.path.join(golden_dir, "cache_update_vectors.json")))
    D = 8
    for case in golden["cases"]:
        B, S = case["B"], case["S"]
        H = len(case["cache_size"])
        cache = StaticCircularCache([case["cache_size"]], static_size=[case["static_size"]], batch_size=B,
                                    head_dim=D, device=dev, dtype=torch.float32)
        ctor = case["ctor"]   # what the reference's constructor builds (cache_utils.py:698-769)
        assert cache.cache_head_start_index[0].tolist() == ctor["head_start"], case["name"]
        assert cache.head_index[0].tolist() == ctor["head_index"], case["name"]
        assert cache.circular_cache_head_index[0].tolist() == ctor["circular_head"], case["name"]
        assert cache.circular_cache_size[0].tolist() == ctor["circular_size"], case["name"]
        assert cache.cache_update_index[0].tolist() == ctor["update_index"], case["name"]
        am = None
        if case["use_mask"]:
            am = torch.zeros(B, S, dtype=torch.int64, device=dev)
            for i, n in enumerate(case["prefill_lens"]):
                am[i, S - n:] = 1
        snaps = {s["step"]: s for s in case["steps"]}

        def check(step):
            if step not in snaps:
                return
            g = snaps[step]
            tag = (case["name"], step)
            assert cache.cache_update_index[0].tolist() == g["update_index"], tag
            assert cache.cache_valid_length[0].tolist() == g["valid_length"], tag
            assert cache.mask_cache[0].tolist() == g["mask_cache"], tag
            assert cache._kv_len[0] == g["kv_len"], tag
            m = cache.mask_cache[0].cpu().numpy() == 1
            gk = np.asarray(g["key_col0"], dtype=np.float32)
            kc = cache.key_cache[0].cpu().numpy()
            vc = cache.value_cache[0].cpu().numpy()
            for d in (0, D - 1):
                assert np.array_equal(kc[:, :, d][m], gk[m]), tag
                assert np.array_equal(vc[:, :, d][m], gk[m] + 0.5), tag

        if S > 0:
            k = torch.from_numpy(_payload(B, H, S, D, 0.0)).to(dev)
            rk, rv = cache.update(k, k + 0.5, 0, am)
            assert rk is k
            check(0)
        pos = S
        for i in range(case["n_decode"]):
            k = torch.from_numpy(_payload(B, H, 1, D, float(pos))).to(dev)
            if am is not None:
                am = torch.cat([am, torch.ones(B, 1, dtype=torch.int64, device=dev)], dim=-1)
            rk, rv = cache.update(k, k + 0.5, 0, am)
            assert rk is cache.key_cache[0] and rv is cache.value_cache[0]
            check(i + 1)
            pos += 1


@pytest.mark.parametrize("seed", range(12))
def test_random_against_oracle(dev, seed):
    """Random ring sizes, prompts (with and without left padding), decode runs;
    fp16 payload at head_dim 128/64 with integer values."""
    from moa_amd import StaticCircularCache
    rng = np.random.default_rng(100 + seed)
    H = int(rng.integers(1, 7))
    s = rng.integers(0, 5, size=H)
    c = rng.integers(1, 12, size=H)
    cache_size = (s + c).tolist()
    B = int(rng.integers(1, 4))
    D = 128 if seed % 2 == 0 else 64
    S = int(rng.integers(2, 50))
    steps = int(rng.integers(0, 40))
    use_mask = seed % 3 == 0
    dtype = torch.float16 if seed % 4 < 2 else torch.bfloat16
    cache = StaticCircularCache([cache_size], static_size=[s.tolist()], batch_size=B, head_dim=D,
                                device=dev, dtype=dtype)
    o = StaticCircularCacheOracle(cache_size, s.tolist(), B, D)
    am_np = None
    if use_mask:
        am_np = np.zeros((B, S), dtype=np.int64)
        for b in range(B):
            n = int(rng.integers(1, S + 1))
            am_np[b, S - n:] = 1
    # small integers are exact in fp16 and bf16
    k = rng.integers(-120, 120, size=(B, H, S, D)).astype(np.float32)
    v = rng.integers(-120, 120, size=(B, H, S, D)).astype(np.float32)
    # pass k as the transposed view the model hands over: [B,S,H,D] -> [B,H,S,D]
    kt = torch.from_numpy(k).to(dev, dtype).transpose(1, 2).contiguous().transpose(1, 2)
    vt = torch.from_numpy(v).to(dev, dtype)
    am = torch.from_numpy(am_np).to(dev) if use_mask else None
    cache.update(kt, vt, 0, am)
    o.update(k, v, am_np)
    _assert_state(cache, o, (seed, "prefill"))
    for i in range(steps):
        k1 = rng.integers(-120, 120, size=(B, H, 1, D)).astype(np.float32)
        v1 = rng.integers(-120, 120, size=(B, H, 1, D)).astype(np.float32)
        if i % 2 == 0:
            k1t = torch.from_numpy(k1).to(dev, dtype)
        else:  # [B,1,H,D] viewed as [B,H,1,D]
            k1t = torch.from_numpy(k1).to(dev, dtype).transpose(1, 2).contiguous().transpose(1, 2)
        cache.update(k1t, torch.from_numpy(v1).to(dev, dtype), 0)
        o.update(k1, v1)
        if i % 7 == 0 or i == steps - 1:
            _assert_state(cache, o, (seed, i))


def test_bookkeeping_only(dev):
    """update_cache_content=False: indices move, no payload is touched."""
    from moa_amd import StaticCircularCache
    cache = StaticCircularCache([[6, 9]], static_size=[[2, 3]], batch_size=2, head_dim=8, device=dev,
                                dtype=torch.float16, update_cache_content=False)
    o = StaticCircularCacheOracle([6, 9], [2, 3], 2, 8)
    k = np.zeros((2, 2, 11, 8), dtype=np.float32)
    cache.update(torch.from_numpy(k).to(dev, torch.float16), torch.from_numpy(k).to(dev, torch.float16), 0)
    o.update(k, k)
    for _ in range(9):
        cache.update(None, None, 0)
        o.update(k[:, :, :1], k[:, :, :1])
    assert cache.cache_update_index[0].tolist() == o.cache_update_index.tolist()
    assert cache.cache_valid_length[0].tolist() == o.cache_valid_length.tolist()
    assert np.array_equal(cache.mask_cache[0].cpu().numpy(), o.mask_cache)
    assert cache.key_cache[0] is None


def test_decode_config_scale_append(dev):
    """Benchmark-size decode config (B=64, H=32, D=128, fp16, ring = 64 + elastic
    window at N=16384): random ring positions incl. the last slot, several
    appends; checked against torch index ops on the GPU (the reference's own
    formulation, cache_utils.py:1031-1054) and the closed-form pointer."""
    from moa_amd import StaticCircularCache
    from moa_amd.workloads import elastic_spans, ring_cache_sizes
    B, H, D = 64, 32, 128
    spans = elastic_spans(H, 16384, seed=0)
    cache_size, static_size = ring_cache_sizes(spans)
    cache = StaticCircularCache([cache_size], static_size=[static_size], batch_size=B, head_dim=D,
                                device=dev, dtype=torch.float16)
    g = torch.Generator(device="cpu").manual_seed(0)
    # state as after a 16384-token prompt: rings full, pointers anywhere in the ring
    circ = cache.circular_cache_size[0].cpu()
    off = (torch.rand(B, H, generator=g) * circ[None, :].float()).long()
    off = torch.minimum(off, circ[None, :] - 1)
    off[0, :] = circ - 1          # wrap on the next step
    off[1, :] = 0
    cache.cache_update_index[0] = (cache.circular_cache_head_index[0].cpu()[None, :] + off).to(dev)
    cache.cache_valid_length[0] = cache.cache_max_length[0][None, :].expand(B, -1).contiguous().to(dev)
    cache._kv_len[0] = 16384
    k0 = torch.zeros(B, 1, H, D, dtype=torch.float16, device=dev).transpose(1, 2)
    cache.update(k0, k0, 0)   # materialise K/V on the device and make one step
    kc_ref = cache.key_cache[0].clone()
    vc_ref = cache.value_cache[0].clone()
    mask_ref = cache.mask_cache[0].clone()
    upd_ref = cache.cache_update_index[0].clone()
    ch = cache.circular_cache_head_index[0].to(dev)
    csz = cache.circular_cache_size[0].to(dev)
    bidx = torch.arange(B, device=dev)[:, None]
    gd = torch.Generator(device=dev).manual_seed(1)
    for step in range(4):
        kn = torch.randn(B, 1, H, D, generator=gd, device=dev, dtype=torch.float16).transpose(1, 2)
        vn = torch.randn(B, 1, H, D, generator=gd, device=dev, dtype=torch.float16).transpose(1, 2)
        cache.update(kn, vn, 0)
        kc_ref[bidx, upd_ref] = kn[:, :, -1, :]
        vc_ref[bidx, upd_ref] = vn[:, :, -1, :]
        mask_ref[bidx, upd_ref] = 1
        upd_ref = (upd_ref + 1 - ch[None, :]) % csz[None, :] + ch[None, :]
        assert torch.equal(cache.cache_update_index[0], upd_ref), step
        assert torch.equal(cache.key_cache[0], kc_ref), step
        assert torch.equal(cache.value_cache[0], vc_ref), step
        assert torch.equal(cache.mask_cache[0], mask_ref), step
        assert torch.equal(cache.cache_valid_length[0], cache.cache_max_length[0][None, :].expand(B, -1))
    # the wrapped row came back to the ring head + steps
    assert torch.equal(cache.cache_update_index[0][0], ch + 4)


def test_long_prompt_insert_properties(dev):
    """Prompt of 16384 tokens into production-size rings (B=2): every ring holds
    exactly the sinks and the last c tokens, at the closed-form slots."""
    from moa_amd import StaticCircularCache
    from moa_amd.workloads import elastic_spans, ring_cache_sizes
    B, H, D, N = 2, 32, 128, 16384
    spans = elastic_spans(H, N, seed=3)
    cache_size, static_size = ring_cache_sizes(spans)
    cache = StaticCircularCache([cache_size], static_size=[static_size], batch_size=B, head_dim=D,
                                device=dev, dtype=torch.float16)
    # payload: token index split over two exact fp16 numbers (t // 128, t % 128)
    t = torch.arange(N, device=dev)
    k = torch.zeros(B, H, N, D, dtype=torch.float16, device=dev)
    k[..., 0] = (t // 128).to(torch.float16)
    k[..., 1] = (t % 128).to(torch.float16)
    k[..., 2] = torch.arange(H, device=dev, dtype=torch.float16)[None, :, None]
    v = -k
    cache.update(k, v, 0)
    kc = cache.key_cache[0]
    tok = (kc[..., 0].long() * 128 + kc[..., 1].long())          # [B, sumC]
    for h in range(H):
        s, c = static_size[h], cache_size[h] - static_size[h]
        st = int(cache.head_index[0][h])
        expect = torch.empty(s + c, dtype=torch.long, device=dev)
        expect[:s] = torch.arange(s, device=dev)
        ring_tok = torch.arange(N - c, N, device=dev)
        expect[s + (ring_tok - s) % c] = ring_tok
        for b in range(B):
            assert torch.equal(tok[b, st:st + s + c], expect), (b, h)
            assert (kc[b, st:st + s + c, 2] == h).all()
        assert int(cache.cache_update_index[0][0, h]) == st + s + (N - s) % c
    assert torch.equal(cache.value_cache[0], -kc)
    assert torch.equal(cache.cache_valid_length[0].cpu(), torch.tensor(cache_size)[None, :].expand(B, -1))
    assert (cache.mask_cache[0] == 1).all()


def test_errors(dev):
    from moa_amd import StaticCircularCache, _lib
    cache = StaticCircularCache([[8]], static_size=[[2]], batch_size=1, head_dim=8, device="cpu",
                                dtype=torch.float16)
    k = torch.zeros(1, 1, 3, 8, dtype=torch.float16)
    with pytest.raises(_lib.MoaKernelError):
        cache.update(k, k, 0)          # CPU tensors: there is no CPU path
    cache = StaticCircularCache([[8]], static_size=[[2]], batch_size=1, head_dim=4, device=dev,
                                dtype=torch.float16)
    k = torch.zeros(1, 1, 3, 4, dtype=torch.float16, device=dev)
    with pytest.raises(NotImplementedError):
        cache.update(k, k, 0)          # 8-byte rows are not covered
    with pytest.raises(AssertionError):
        cache.update(torch.zeros(1, 2, 3, 4, dtype=torch.float16, device=dev), k, 0)   # head count
