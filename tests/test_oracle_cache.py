"""Pins the integer side of the oracle: the formula restatement of the
reference cache (StaticCircularCacheOracle) against (1) vectors written by the
reference's own StaticCircularCache (tests/golden/cache_update_vectors.json),
(2) an independent list+deque ring model, (3) hand-derived values of the
reference's demo (MoA/attention/cache_utils.py:1301-1371), and the plan->cache
helper against known answers and the reference's outputs on shipped plans."""
import json
import os

import numpy as np
import pytest

from oracle.moa_oracle import (RingModel, StaticCircularCacheOracle,
                               moa_config_to_cache_config)


def _payload(B, H, S, D, base):
    t = np.arange(S, dtype=np.float32)[None, None, :, None]
    h = np.arange(H, dtype=np.float32)[None, :, None, None] * 1000.0
    b = np.arange(B, dtype=np.float32)[:, None, None, None] * 100000.0
    return np.broadcast_to(base + b + h + t, (B, H, S, D)).copy()


@pytest.fixture(scope="module")
def golden(golden_dir):
    return json.load(open(os.path.join(golden_dir, "cache_update_vectors.json")))


def test_golden_cases_present(golden):
    names = [c["name"] for c in golden["cases"]]
    assert "reference_demo" in names and len(names) >= 8


def test_oracle_matches_reference_vectors(golden):
    for case in golden["cases"]:
        B, D, S = case["B"], case["D"], case["S"]
        H = len(case["cache_size"])
        o = StaticCircularCacheOracle(case["cache_size"], case["static_size"], B, D)
        ctor = case["ctor"]
        assert o.cache_head_start_index.tolist() == ctor["head_start"], case["name"]
        assert o.head_index.tolist() == ctor["head_index"]
        assert o.circular_cache_head_index.tolist() == ctor["circular_head"]
        assert o.circular_cache_size.tolist() == ctor["circular_size"]
        assert o.cache_update_index.tolist() == ctor["update_index"]
        am = None
        if case["use_mask"]:
            am = np.zeros((B, S), dtype=np.int64)
            for i, n in enumerate(case["prefill_lens"]):
                am[i, S - n:] = 1
        snaps = {s["step"]: s for s in case["steps"]}

        def check(step):
            if step not in snaps:
                return
            g = snaps[step]
            tag = (case["name"], step)
            assert o.cache_update_index.tolist() == g["update_index"], tag
            assert o.cache_valid_length.tolist() == g["valid_length"], tag
            assert o.mask_cache.tolist() == g["mask_cache"], tag
            assert o.kv_len == g["kv_len"], tag
            m = o.mask_cache == 1
            gk = np.asarray(g["key_col0"], dtype=np.float32)
            assert np.array_equal(o.key_cache[:, :, 0][m], gk[m]), tag
            assert np.array_equal(o.value_cache[:, :, 0][m], gk[m] + 0.5), tag

        if S > 0:
            k = _payload(B, H, S, D, 0.0)
            o.update(k, k + 0.5, am)
            check(0)
        pos = S
        for i in range(case["n_decode"]):
            k = _payload(B, H, 1, D, float(pos))
            if am is not None:
                am = np.concatenate([am, np.ones((B, 1), dtype=np.int64)], axis=-1)
            o.update(k, k + 0.5, am)
            check(i + 1)
            pos += 1


def test_reference_demo_hand_values():
    """Row 0 of the reference demo, derived by hand from the ring definition:
    head 0 (s=2,c=3) keeps t0,t1 | t11,t12,t13 ; head 1 (s=3,c=7) keeps
    t0..t2 | ring slots hold t10..t13,t7,t8,t9."""
    o = StaticCircularCacheOracle([5, 10], [2, 3], 1, 1)
    S = 14
    k = (np.arange(2)[:, None] * S + np.arange(S)[None, :]).astype(np.float32)[None, :, :, None]
    o.update(k, k)
    assert o.key_cache[0, :, 0].tolist() == [0, 1, 11, 12, 13, 14, 15, 16, 24, 25, 26, 27, 21, 22, 23]
    assert o.cache_update_index.tolist() == [[2, 12]]
    assert o.cache_valid_length.tolist() == [[5, 10]]
    # pointer sequences over decode steps
    seq0, seq1 = [], []
    for step in range(7):
        seq0.append(int(o.cache_update_index[0, 0]))
        seq1.append(int(o.cache_update_index[0, 1]))
        kn = np.full((1, 2, 1, 1), 100.0 + step, dtype=np.float32)
        o.update(kn, kn)
    assert seq0 == [2, 3, 4, 2, 3, 4, 2]
    assert seq1 == [12, 13, 14, 8, 9, 10, 11]


@pytest.mark.parametrize("seed", range(40))
def test_oracle_matches_ring_model(seed):
    """Random sizes / prompt lengths / decode counts: formula restatement vs the
    list+deque model: slot->token map, valid length, next pointer, evicted set."""
    rng = np.random.default_rng(seed)
    H = int(rng.integers(1, 5))
    s = rng.integers(0, 6, size=H)
    c = rng.integers(1, 9, size=H)
    cache = (s + c).tolist()
    B = 2
    N = int(rng.integers(0, 40))
    steps = int(rng.integers(0, 30))
    if N == 1:
        N = 2  # a 1-token "prefill" is a decode step by the reference's rule
    o = StaticCircularCacheOracle(cache, s.tolist(), B, 1)
    models = [[RingModel(int(o.head_index[h]), int(s[h]), int(c[h])) for h in range(H)] for _ in range(B)]
    tok = 0
    if N > 0:
        ids = (np.arange(N, dtype=np.float32) + 1)[None, None, :, None]
        k = np.broadcast_to(ids, (B, H, N, 1)).copy()
        o.update(k, -k)
        for b in range(B):
            for h in range(H):
                for t in range(N):
                    models[b][h].push(t + 1)
        tok = N
    for _ in range(steps):
        k = np.full((B, H, 1, 1), float(tok + 1), dtype=np.float32)
        o.update(k, -k)
        for b in range(B):
            for h in range(H):
                models[b][h].push(tok + 1)
        tok += 1
    for b in range(B):
        for h in range(H):
            m = models[b][h]
            sm = m.slot_map()
            seg = slice(int(o.head_index[h]), int(o.head_index[h + 1]))
            got = {int(o.head_index[h]) + i: int(x) for i, x in enumerate(o.key_cache[b, seg, 0])
                   if o.mask_cache[b, int(o.head_index[h]) + i] == 1}
            assert got == sm, (seed, b, h)
            assert int(o.cache_valid_length[b, h]) == m.valid_length
            assert int(o.cache_update_index[b, h]) == m.next_slot
            # evicted = everything seen that is neither static nor in the ring
            kept = set(sm.values())
            assert set(range(1, tok + 1)) - kept == set(m.evicted)
            assert np.array_equal(o.value_cache[b, seg, 0], -o.key_cache[b, seg, 0])


def test_closed_form_no_padding():
    """token t -> start+t if t<s else start+s+((t-s) mod c); kept iff t<s or t>=N-c;
    pointer = start+s+((N-s) mod c)."""
    for (s, c, N) in [(2, 3, 14), (3, 7, 14), (64, 64, 300), (64, 192, 100), (0, 5, 23), (4, 4, 4), (4, 4, 5)]:
        o = StaticCircularCacheOracle([s + c], [s], 1, 1)
        k = np.arange(N, dtype=np.float32)[None, None, :, None]
        keep = o.update_prefill(k, k)
        exp_keep = [(t < s) or (t >= N - c) for t in range(N)]
        assert keep[0, 0].tolist() == exp_keep
        for t in range(N):
            if exp_keep[t]:
                slot = t if t < s else s + ((t - s) % c)
                assert o.key_cache[0, slot, 0] == t
        if N > s:
            assert int(o.cache_update_index[0, 0]) == s + ((N - s) % c)
        else:
            assert int(o.cache_update_index[0, 0]) == N
        assert int(o.cache_valid_length[0, 0]) == min(N, s) + min(max(N - s, 0), c)


def test_plan_known_answers():
    f = lambda a, b, n, mn: moa_config_to_cache_config({"alphas": [[a]], "betas": [[b]]}, n, mn)
    r = f(0, 0.5, 1024, 1024); assert (r["cache_size"], r["static_size"]) == ([[1024]], [[64]])
    r = f(-1024, 0.125, 1024, 1024); assert r["cache_size"] == [[128]]
    r = f(1024, 1.0, 1024, 1024); assert r["cache_size"] == [[2048]]
    r = f(100.7, 0.3, 900, 100); assert r["cache_size"] == [[448]]
    r = f(0, 0, 10, 10); assert (r["cache_size"], r["static_size"]) == ([[128]], [[64]])


def test_plan_matches_reference_vectors(golden):
    single = [p for p in golden["plans"] if "alpha" in p]
    assert len(single) >= 7
    for p in single:
        r = moa_config_to_cache_config({"alphas": [[p["alpha"]]], "betas": [[p["beta"]]]},
                                       p["seq_len"], p["max_new_token"])
        assert r["cache_size"][0][0] == p["cache_size"], p
        assert r["static_size"][0][0] == p["static_size"], p


def test_plan_shipped_vicuna7b(golden, golden_dir):
    """tests/golden/plan_vicuna-7b-v1.5-16k_moa_alpha_beta.json is the data file
    examples/lmsys--vicuna-7b-v1.5-16k/moa_alpha_beta.json of the reference; the
    expected sizes were written by the reference's moa_config_to_cache_config."""
    plan = json.load(open(os.path.join(golden_dir, "plan_vicuna-7b-v1.5-16k_moa_alpha_beta.json")))
    rows = [p for p in golden["plans"] if p.get("plan_file", "").startswith("examples/lmsys--vicuna-7b")]
    assert len(rows) == 2
    for p in rows:
        r = moa_config_to_cache_config(plan, p["seq_len"], p["max_new_token"])
        assert r["cache_size"][0] == p["cache_size_layer0"]
        assert r["cache_size"][-1] == p["cache_size_last"]
        assert int(np.sum(r["cache_size"])) == p["cache_size_sum"]
        assert int(np.sum(r["static_size"])) == p["static_size_sum"]
