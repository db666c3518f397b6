"""Head permutation utilities (CPU): known answers and the invariance they exist for."""
import json
import os

import torch
from torch import nn

from moa_amd.attention.permutation_utils import (moa_config_to_permutation, permute_attention_projection,
                                                 permute_output_projection)


def test_permutation_known_answer():
    perms, clusters = moa_config_to_permutation(
        {"alphas": [[3, 1, 3, 1, 2], [5, 5, 5]], "betas": [[0.5, 0.2, 0.5, 0.1, 0.0], [0.1, 0.1, 0.1]]})
    # sort by (alpha, beta), ties keep the original order: (1,.1)->3, (1,.2)->1, (2,0)->4, (3,.5)->0,2
    assert perms[0].tolist() == [3, 1, 4, 0, 2] and perms[0].dtype == torch.int64
    assert clusters[0] == {0: (0, 0), 1: (1, 1), 2: (2, 2), 3: (3, 4)}
    assert perms[1].tolist() == [0, 1, 2] and clusters[1] == {0: (0, 2)}


def test_permutation_of_the_shipped_plan(golden_dir):
    """On the reference's vicuna-7b plan: a permutation of 0..H-1 per layer, (alpha, beta) sorted
    after it, clusters tile the heads and are constant inside."""
    plan = json.load(open(os.path.join(golden_dir, "plan_vicuna-7b-v1.5-16k_moa_alpha_beta.json")))
    perms, clusters = moa_config_to_permutation(plan)
    assert len(perms) == len(plan["alphas"])
    for l, (p, c) in enumerate(zip(perms, clusters)):
        H = len(plan["alphas"][l])
        assert sorted(p.tolist()) == list(range(H))
        pairs = [(plan["alphas"][l][i], plan["betas"][l][i]) for i in p.tolist()]
        assert pairs == sorted(pairs)
        covered = []
        for k in range(len(c)):
            a, b = c[k]
            assert len(set(pairs[a:b + 1])) == 1
            if k:
                assert pairs[a] != pairs[a - 1]
            covered += list(range(a, b + 1))
        assert covered == list(range(H))


def test_projection_permutation_keeps_the_layer_function():
    """y = o_proj(per-head f(q_proj x)) is unchanged when q and o are permuted together."""
    torch.manual_seed(0)
    H, D, hid = 6, 8, 32
    q, o = nn.Linear(hid, H * D, bias=True), nn.Linear(H * D, hid, bias=False)
    x = torch.randn(5, hid)
    scale = torch.arange(1, H + 1).float()          # a per-head function that depends on the head's plan

    def run(qp, op, head_scale):
        h = qp(x).view(5, H, D) * head_scale[None, :, None]
        return op(h.reshape(5, H * D))

    want = run(q, o, scale)
    perm = torch.tensor([4, 0, 5, 2, 1, 3])
    w_before = q.weight.data.clone()
    permute_attention_projection(q, perm, H)
    permute_output_projection(o, perm, H)
    assert torch.equal(q.weight.data.view(H, D, hid)[1], w_before.view(H, D, hid)[0])   # new head 1 = old head 0
    got = run(q, o, scale[perm])
    assert torch.allclose(got, want, atol=1e-5)
    # grouped-query: a permutation of 3 kv heads moves their 2 query heads each
    q2 = nn.Linear(hid, H * D, bias=False)
    w0 = q2.weight.data.clone().view(H, D, hid)
    permute_attention_projection(q2, torch.tensor([2, 0, 1]), 3, 2)
    w1 = q2.weight.data.view(H, D, hid)
    assert torch.equal(w1[0], w0[4]) and torch.equal(w1[1], w0[5]) and torch.equal(w1[2], w0[0])
    permute_attention_projection(q2, None, 3, 2)   # no permutation: untouched
    assert torch.equal(q2.weight.data.view(H, D, hid), w1)
