"""Pins the floating-point side of the oracle by what mathematics fixes:
independent formulations against each other, special cases that reduce to a
library routine, brute force on tiny inputs, and invariants."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle.moa_oracle import (count_live_pairs, decode_grouped_sdpa, decode_segments,
                               live_kv_blocks, moa_token_mask, moa_token_mask_from_blocks,
                               prefill_blockwise, prefill_bruteforce, prefill_masked_dense,
                               prefill_p_rounded, round_to_storage, head_start_valid_to_head_index)


def test_mask_two_formulations_agree_exhaustively():
    for block in (4, 8):
        for n in (1, 7, 8, 9, 24, 29, 40):
            nb = (n + block - 1) // block
            for ns in range(0, nb + 2):
                for nl in range(0, nb + 2):
                    a = moa_token_mask(n, ns, nl, block)
                    b = moa_token_mask_from_blocks(n, ns, nl, block)
                    assert np.array_equal(a, b), (block, n, ns, nl)


def test_mask_special_cases():
    n = 320
    causal = np.tril(np.ones((n, n), dtype=bool))
    assert np.array_equal(moa_token_mask(n, 0, 5), causal)      # nl >= nb
    assert np.array_equal(moa_token_mask(n, 5, 0), causal)      # ns >= nb
    assert np.array_equal(moa_token_mask(n, 1, 99), causal)
    bd = moa_token_mask(n, 0, 1)                                  # block-diagonal causal
    i, j = np.nonzero(bd)
    assert ((i // 64) == (j // 64)).all() and (j <= i).all()
    assert bd.sum() == 5 * (64 * 65 // 2)
    assert not moa_token_mask(n, 0, 0).any()
    # query in block 4 with ns=1, nl=2 sees block 0, 3 and 4 only
    assert live_kv_blocks(4, 1, 2) == [0, 3, 4]
    assert live_kv_blocks(0, 1, 2) == [0]
    assert live_kv_blocks(1, 3, 1) == [0, 1]
    assert live_kv_blocks(5, 0, 0) == []
    # window seen by a query: between (nl-1)*64+1 and nl*64 most recent tokens
    m = moa_token_mask(640, 0, 3)
    assert m[639].sum() == 3 * 64 and m[576].sum() == 2 * 64 + 1


def test_count_live_pairs_matches_mask():
    for (n, ns, nl) in [(320, 1, 2), (333, 1, 3), (64, 1, 1), (200, 0, 1), (512, 2, 8), (130, 1, 0)]:
        pairs, tiles = count_live_pairs(n, ns, nl)
        assert pairs == int(moa_token_mask(n, ns, nl).sum())
        nb = (n + 63) // 64
        assert tiles == sum(len(live_kv_blocks(m, ns, nl)) for m in range(nb))


def _rand(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g)


def test_prefill_reduces_to_causal_sdpa():
    """The reference's own test case (tests/attention_kernel_test.py:35-76):
    sink 64 + local 64 on N=128 is dense causal; tolerance 1e-3."""
    B, H, N, D = 2, 4, 128, 128
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.rand(B, H, N, D, generator=g) for _ in range(3))
    o = prefill_masked_dense(q, k, v, 0.1, [1] * H, [1] * H)
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.1)
    torch.testing.assert_close(o, ref, rtol=1e-3, atol=1e-3)
    # wide windows on a longer ragged sequence
    q, k, v = (_rand((1, 2, 300, 32), s) for s in (1, 2, 3))
    o = prefill_masked_dense(q, k, v, 32 ** -0.5, [0, 7], [9, 1])
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=32 ** -0.5)
    torch.testing.assert_close(o, ref, rtol=1e-5, atol=1e-5)


def test_prefill_three_formulations_agree():
    N, D = 200, 16
    rng = np.random.default_rng(5)
    q, k, v = (rng.standard_normal((N, D)) for _ in range(3))
    for ns, nl in [(1, 1), (1, 2), (0, 2), (2, 1), (1, 0), (0, 0), (0, 1)]:
        bf = prefill_bruteforce(q, k, v, 0.3, ns, nl)
        bw = prefill_blockwise(q, k, v, 0.3, ns, nl)
        md = prefill_masked_dense(torch.from_numpy(q)[None, None], torch.from_numpy(k)[None, None],
                                  torch.from_numpy(v)[None, None], 0.3, [ns], [nl])[0, 0].numpy()
        assert np.abs(bf - bw).max() < 1e-12, (ns, nl)
        assert np.abs(bf - md).max() < 2e-5, (ns, nl)


def test_prefill_invariants():
    B, H, N, D = 2, 3, 192, 16
    q, k, v = (_rand((B, H, N, D), s) for s in (10, 11, 12))
    ns, nl = [1, 0, 2], [1, 2, 1]
    o = prefill_masked_dense(q, k, v, 0.25, ns, nl)
    # V == 1 => O == 1
    o1 = prefill_masked_dense(q, k, torch.ones_like(v), 0.25, ns, nl)
    torch.testing.assert_close(o1, torch.ones_like(o1), rtol=1e-6, atol=1e-6)
    # head-permutation equivariance
    perm = [2, 0, 1]
    op = prefill_masked_dense(q[:, perm], k[:, perm], v[:, perm], 0.25, [ns[i] for i in perm], [nl[i] for i in perm])
    torch.testing.assert_close(op, o[:, perm])
    # batch independence
    ob = prefill_masked_dense(q[1:], k[1:], v[1:], 0.25, ns, nl)
    torch.testing.assert_close(ob, o[1:])
    # shifting all keys by a vector orthogonal... simpler: scaling q by a and sm_scale by 1/a
    o2 = prefill_masked_dense(q * 4.0, k, v, 0.25 / 4.0, ns, nl)
    torch.testing.assert_close(o2, o, rtol=1e-4, atol=1e-5)


def test_round_to_storage_against_torch_casts():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000) * 10.0 ** rng.integers(-8, 3, 20000),
                        [0.0, 1.0, 1.00390625, 1.01171875, 256.0, 2.0 ** -20, 3.0 * 2.0 ** -26]]).astype(np.float32)
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        mine = round_to_storage(x, name)
        theirs = torch.from_numpy(x).to(dt).float().numpy()
        assert np.array_equal(mine, theirs), name
    # ties go to the even neighbour: 1 + 2^-8 -> 1, 1 + 3 * 2^-8 -> 1 + 2^-6 (bf16 spacing at 1 is 2^-7)
    assert round_to_storage(np.float32([1.00390625, 1.01171875]), "bf16").tolist() == [1.0, 1.015625]
    assert round_to_storage(x, None) is not None and np.array_equal(round_to_storage(x, None), x)


def test_p_rounded_prefill_is_pinned():
    """(1) without rounding it is the masked dense attention; (2) with rounding it equals a
    pure-Python evaluation of its defining formula that rounds through torch's scalar casts;
    (3) integer shifts of the reference exponent change nothing (bit for bit in the weights,
    to fp64 rounding in the output); (4) the rounding moves the result by no more than
    u * (attention of |V| + ...) with u = 2^-8 (bf16) / 2^-11 (f16)."""
    B, H, N, D = 1, 3, 192, 16
    q, k, v = (_rand((B, H, N, D), s) for s in (20, 21, 22))
    ns, nl = [1, 0, 2], [1, 2, 1]
    sm = 0.3
    exact = prefill_masked_dense(q, k, v, sm, ns, nl).numpy()
    none = prefill_p_rounded(q, k, v, sm, ns, nl, None)
    assert np.abs(none - exact).max() < 2e-6
    absv = prefill_p_rounded(q, k, v.abs(), sm, ns, nl, None)
    for name, dt, u in (("bf16", torch.bfloat16, 2.0 ** -8), ("f16", torch.float16, 2.0 ** -11)):
        got = prefill_p_rounded(q, k, v, sm, ns, nl, name, rows_per_step=80)
        # (2) brute force, head 0 and 2, a few rows incl. the first of a block
        c = sm * 1.4426950408889634
        for h in (0, 2):
            for i in (0, 1, 63, 64, 65, 130, 191):
                js = [j for j in range(i + 1) if (j // 64) < ns[h] or (j // 64) >= (i // 64) + 1 - nl[h]]
                t = [c * float(np.dot(q[0, h, i].double().numpy(), k[0, h, j].double().numpy())) for j in js]
                M = float(np.ceil(max(t)))
                p32 = [np.float32(2.0 ** (x - M)) for x in t]
                den = sum(float(x) for x in p32)
                o = np.zeros(D)
                for pj, j in zip(p32, js):
                    w = float(torch.tensor(float(pj), dtype=torch.float32).to(dt).float())
                    o += w * v[0, h, j].double().numpy()
                assert np.abs(o / den - got[0, h, i]).max() < 1e-12, (name, h, i)
        # (3) shift invariance: exact in bf16 up to the fp32 evaluation of 2^x (1e-8 relative per weight);
        # f16 rounds weights below 2^-14 on its subnormal grid (spacing 2^-24), which a shift moves:
        # up to 2^-25 * 2^shift per key, relative to a weight sum of about 1
        for shift in (-3, 5):
            shifted = prefill_p_rounded(q, k, v, sm, ns, nl, name, shift=shift)
            assert np.abs(shifted - got).max() < (1e-8 if name == "bf16" else 1e-4), (name, shift)
        # (4) the a-priori bound of the weight rounding
        assert (np.abs(got - none) <= u * absv + 1e-9).all(), name
        assert np.abs(got - none).max() > 0.05 * u, name     # and the rounding is really there


def _packed_case(seed, B=2, sizes=(64, 64, 128, 192, 192), D=16, full=True):
    rng = np.random.default_rng(seed)
    sizes = np.asarray(sizes)
    H = len(sizes)
    start = np.concatenate([[0], np.cumsum(sizes)[:-1]])
    sumc = int(sizes.sum())
    kc = rng.standard_normal((B, sumc, D)).astype(np.float32)
    vc = rng.standard_normal((B, sumc, D)).astype(np.float32)
    q = rng.standard_normal((B, H, D)).astype(np.float32)
    hs = np.broadcast_to(start, (B, H)).astype(np.int64).copy()
    if full:
        hv = np.broadcast_to(sizes, (B, H)).astype(np.int64).copy()
    else:
        hv = rng.integers(1, sizes + 1, size=(B, H)).astype(np.int64)
    return q, kc, vc, hs, hv, sizes


def test_decode_matches_grouped_sdpa():
    q, kc, vc, hs, hv, sizes = _packed_case(0)
    o = decode_segments(q, kc, vc, hs, hv, 0.25)
    hi = head_start_valid_to_head_index(hs, hv)
    assert hi.tolist() == [0, 64, 128, 256, 448, 640]
    ref = decode_grouped_sdpa(torch.from_numpy(q)[:, :, None, :], torch.from_numpy(kc),
                              torch.from_numpy(vc), hi, 0.25)          # [B,1,H,D]
    assert ref.shape == (2, 1, 5, 16)
    assert np.abs(o - ref[:, 0].numpy()).max() < 1e-5


def test_decode_ring_order_invariance_and_partial_fill():
    q, kc, vc, hs, hv, sizes = _packed_case(1, full=False)
    o = decode_segments(q, kc, vc, hs, hv, 0.3)
    rng = np.random.default_rng(2)
    kc2, vc2 = kc.copy(), vc.copy()
    for b in range(kc.shape[0]):
        for h in range(len(sizes)):
            s0, n = int(hs[b, h]), int(hv[b, h])
            p = rng.permutation(n)
            kc2[b, s0:s0 + n] = kc[b, s0:s0 + n][p]
            vc2[b, s0:s0 + n] = vc[b, s0:s0 + n][p]
            # garbage beyond the valid part must be ignored
            kc2[b, s0 + n:s0 + sizes[h]] = 1e4
            vc2[b, s0 + n:s0 + sizes[h]] = -1e4
    o2 = decode_segments(q, kc2, vc2, hs, hv, 0.3)
    assert np.abs(o - o2).max() < 1e-12
    # V == 1 => O == 1 ; valid == 0 => 0
    o3 = decode_segments(q, kc, np.ones_like(vc), hs, hv, 0.3)
    assert np.abs(o3 - 1).max() < 1e-12
    hv0 = hv.copy(); hv0[0, 1] = 0
    assert np.all(decode_segments(q, kc, vc, hs, hv0, 0.3)[0, 1] == 0)


def test_decode_equals_token_granular_prefill_row():
    """Decode at position p over {sinks} U {last c tokens} equals row p of dense
    attention with the token-granular mask j < s or p - j < c."""
    rng = np.random.default_rng(3)
    N, D, s, c = 150, 8, 4, 20
    k = rng.standard_normal((N, D)); v = rng.standard_normal((N, D)); qv = rng.standard_normal(D)
    p = N - 1
    keys = list(range(s)) + list(range(p - c + 1, p + 1))
    kc = k[keys][None]; vc = v[keys][None]
    o = decode_segments(qv[None, None], kc, vc, np.array([[0]]), np.array([[s + c]]), 0.35)[0, 0]
    sc = (k @ qv) * 0.35
    m = np.array([(j < s) or (p - j < c) for j in range(N)])
    sc = np.where(m, sc, -np.inf)
    w = np.exp(sc - sc.max()); w /= w.sum()
    assert np.abs(o - w @ v).max() < 1e-12


def test_decode_rounded_weights_match_the_prefill_formulation():
    """decode_segments(p_dtype=...) is prefill_p_rounded's formula on one query row: the row of a
    prompt that sees every key (a wide window) gives the same numbers."""
    rng = np.random.default_rng(12)
    N, D = 150, 16
    q, k, v = (rng.standard_normal((1, 1, N, D)).astype(np.float32) for _ in range(3))
    for name in ("bf16", "f16", None):
        full = prefill_p_rounded(q, k, v, 0.3, [0], [99], name)[0, 0, N - 1]
        dec = decode_segments(q[:, :, N - 1], k[0], v[0], np.array([[0]]), np.array([[N]]), 0.3, p_dtype=name)[0, 0]
        # (without rounding the prefill function still carries its weights in fp32, the decode one in fp64)
        assert np.abs(full - dec).max() < (1e-12 if name else 1e-7), name
    # and the weight rounding moves the result by no more than u * attention(|V|)
    exact = decode_segments(q[:, :, N - 1], k[0], v[0], np.array([[0]]), np.array([[N]]), 0.3)
    absv = decode_segments(q[:, :, N - 1], k[0], v[0], np.array([[0]]), np.array([[N]]), 0.3, abs_v=True)
    for name, u in (("bf16", 2.0 ** -8), ("f16", 2.0 ** -11)):
        dec = decode_segments(q[:, :, N - 1], k[0], v[0], np.array([[0]]), np.array([[N]]), 0.3, p_dtype=name)
        assert (np.abs(dec - exact) <= u * absv + 1e-9).all() and np.abs(dec - exact).max() > 0


def test_decode_gqa_group():
    q, kc, vc, hs, hv, sizes = _packed_case(4, sizes=(64, 128), D=8)
    rng = np.random.default_rng(9)
    q4 = rng.standard_normal((2, 4, 8)).astype(np.float32)   # 4 q heads on 2 kv heads
    o = decode_segments(q4, kc, vc, hs, hv, 0.2, group=2)
    for h in range(4):
        oh = decode_segments(q4[:, h:h + 1], kc, vc, hs[:, h // 2:h // 2 + 1], hv[:, h // 2:h // 2 + 1], 0.2)
        assert np.array_equal(o[:, h], oh[:, 0])
