"""Pins oracle.rope_reference (CPU): the installed transformers' own function, a
hand-computed known answer and what the mathematics of a rotation fixes."""
import math

import pytest
import torch

from oracle.moa_oracle import rope_reference, rope_cos_sin


def _rand(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_equals_transformers_function(dtype):
    """Bit for bit against apply_rotary_pos_emb of the installed transformers (the formula has not
    changed since the 4.44.2 the reference pins)."""
    m = pytest.importorskip("transformers.models.llama.modeling_llama")
    B, H, N, D = 2, 3, 17, 64
    q, k = _rand((B, H, N, D), dtype, 1), _rand((B, 2, N, D), dtype, 2)
    pos = torch.arange(N)[None, :].repeat(B, 1) + torch.tensor([[0], [5]])
    cos, sin = rope_cos_sin(pos, D, dtype=dtype)
    fn = getattr(m.apply_rotary_pos_emb, "__wrapped__", m.apply_rotary_pos_emb)
    qe, ke = fn(q, k, cos, sin)
    assert torch.equal(rope_reference(q, cos, sin), qe)
    assert torch.equal(rope_reference(k, cos, sin), ke)


def test_hand_computed_known_answer():
    """D=4: pairs are (x0,x2) and (x1,x3); angle theta0 for the first, theta1 for the second."""
    x = torch.tensor([[[[1.0, 2.0, 3.0, 4.0]]]], dtype=torch.float64)
    t0, t1 = 0.5, -1.25
    cos = torch.tensor([[[math.cos(t0), math.cos(t1), math.cos(t0), math.cos(t1)]]], dtype=torch.float64)
    sin = torch.tensor([[[math.sin(t0), math.sin(t1), math.sin(t0), math.sin(t1)]]], dtype=torch.float64)
    want = [1 * math.cos(t0) - 3 * math.sin(t0), 2 * math.cos(t1) - 4 * math.sin(t1),
            3 * math.cos(t0) + 1 * math.sin(t0), 4 * math.cos(t1) + 2 * math.sin(t1)]
    got = rope_reference(x, cos, sin)[0, 0, 0].tolist()
    assert got == pytest.approx(want, abs=1e-15)


def test_position_zero_is_identity_and_norms_are_kept():
    B, H, N, D = 1, 2, 9, 32
    x = _rand((B, H, N, D), torch.float64, 3)
    cos, sin = rope_cos_sin(torch.arange(N)[None, :], D, dtype=torch.float64)
    y = rope_reference(x, cos, sin)
    assert torch.equal(y[:, :, 0], x[:, :, 0])
    # each (i, i+D/2) pair is rotated: its norm is unchanged
    n_in = x[..., : D // 2] ** 2 + x[..., D // 2:] ** 2
    n_out = y[..., : D // 2] ** 2 + y[..., D // 2:] ** 2
    assert torch.allclose(n_in, n_out, rtol=0, atol=1e-6)


def test_scores_depend_on_relative_position_only():
    D = 64
    q, k = _rand((1, 1, 1, D), torch.float64, 4), _rand((1, 1, 1, D), torch.float64, 5)

    def score(m, n):
        cq, sq = rope_cos_sin(torch.tensor([[m]]), D, dtype=torch.float64)
        ck, sk = rope_cos_sin(torch.tensor([[n]]), D, dtype=torch.float64)
        return float((rope_reference(q, cq, sq) * rope_reference(k, ck, sk)).sum())

    assert score(7, 3) == pytest.approx(score(104, 100), abs=1e-4)   # tables are fp32-accurate
    assert score(7, 3) != pytest.approx(score(7, 4), abs=1e-3)


def test_cos_sin_tables():
    cos, sin = rope_cos_sin(torch.tensor([[0, 1, 2]]), 8)
    assert cos.shape == (1, 3, 8) and torch.equal(cos[..., :4], cos[..., 4:])
    assert float(cos[0, 1, 0]) == pytest.approx(math.cos(1.0), abs=1e-6)
    assert float(sin[0, 2, 1]) == pytest.approx(math.sin(2.0 * 10000 ** (-2 / 8)), abs=1e-6)
