"""How the parity tests of the matrix-core kernels compare a GPU result with the CPU oracle.

The path is specified with |out - ref| <= 2e-3 + 1e-2 |ref| against an fp32 reference.

fp16: that bound, against the oracle's exact attention, every element.

bf16: the kernels round the softmax weights to bf16 in front of P.V, as the reference's kernel rounds
them to fp16 (MoA/kernels/block_sparse_attention_prefill.py:608-610).  With 8 significant bits that
rounding alone moves an output by up to 2^-8 * sum_j w_j |v_j|, which exceeds 2e-3 + 1e-2 |ref| in
rows whose weight sits on a few keys (rows that see few keys, peaked scores) where the sum cancels.
So there are two comparisons:
  (1) against the oracle that rounds the weights at the same place (prefill_p_rounded /
      decode_segments(p_dtype=...); the kernels keep their reference exponent integral, which makes
      the rounded weights independent of the order the keys are met in): the stated bound, every element;
  (2) against the exact oracle: every element inside the a-priori bound of the weight rounding plus
      the output rounding, 2^-8 * (attention of |V| + |ref|) + 2e-3; the elements outside the STATED
      bound are counted, recorded, and held to a rate in EVERY comparison: at most MAX_FRACTION of the
      elements (with three standard deviations of counting noise on top, so that a comparison of a few
      thousand elements is not failed by one element), 1e-5 at the benchmark's size where the callers say so.
      Measured on the MI355X: 1.2e-4 at worst over the random plans (N = 65), 2.0e-4 with peaked scores,
      6e-7 at the benchmark's size.  Normalising a row by the sum of the ROUNDED weights instead of the
      exact sum does not change these counts (3 against 3, 25 against 24, 267 against 261 elements in a CPU
      experiment over N = 65 .. 1024): the elements outside belong to rows in which two to six keys carry
      the weight and their values cancel, and there the relative error 2^-9 of each weight stays what it is.
`stats` collects what was measured (tag, elements, outside, max error) for the test report.
"""
import numpy as np
import torch

from oracle.moa_oracle import prefill_masked_dense, prefill_p_rounded

ATOL, RTOL = 2e-3, 1e-2
U_BF16 = 2.0 ** -8
MAX_FRACTION = 2.5e-4   # of the elements of a bf16 result may lie outside the stated bound against the exact oracle

stats = []


def p_dtype_name(dtype):
    return {torch.float16: "f16", torch.bfloat16: "bf16"}[dtype]


def close_stated(out, ref, tag):
    """Every element inside the stated bound."""
    out = out.float().cpu().double()
    ref = torch.as_tensor(np.asarray(ref.cpu() if hasattr(ref, "cpu") else ref)).double()
    assert torch.isfinite(out).all(), tag
    err = (out - ref).abs()
    bound = ATOL + RTOL * ref.abs()
    bad = err > bound
    assert not bad.any(), (tag, float(err.max()), int(bad.sum()), [int(x) for x in bad.nonzero()[0]])
    return float(err.max())


def allowed_outside(elements, max_fraction):
    """The count a rate of max_fraction allows among `elements`, with three standard deviations of
    counting noise and one element on top."""
    mean = max_fraction * elements
    return int(mean + 3.0 * mean ** 0.5 + 1.0)


def close_counted(out, ref, ref_absv, tag, max_fraction=MAX_FRACTION, u=U_BF16):
    """Rounded weights against the exact oracle: comparison (2) of the module docstring."""
    out = out.float().cpu().double()
    ref = torch.as_tensor(np.asarray(ref.cpu() if hasattr(ref, "cpu") else ref)).double()
    ref_absv = torch.as_tensor(np.asarray(ref_absv.cpu() if hasattr(ref_absv, "cpu") else ref_absv)).double()
    assert torch.isfinite(out).all(), tag
    err = (out - ref).abs()
    outside = int((err > ATOL + RTOL * ref.abs()).sum())
    stats.append({"tag": str(tag), "elements": out.numel(), "outside_stated_bound": outside,
                  "max_abs_err": float(err.max())})
    apriori = u * (ref_absv + ref.abs()) + ATOL
    bad = err > apriori
    assert not bad.any(), (tag, float(err.max()), int(bad.sum()), [int(x) for x in bad.nonzero()[0]])
    assert outside <= allowed_outside(out.numel(), max_fraction), (tag, outside, out.numel(), float(err.max()))
    return outside


def check_prefill(out, q, k, v, sm, ns, nl, tag, max_fraction=MAX_FRACTION):
    """out, q: [B, Hq, N, D]; k, v: [B, Hkv, N, D] with Hq a multiple of Hkv; ns, nl per kv head."""
    G = q.shape[1] // k.shape[1]
    if G > 1:
        k, v = k.repeat_interleave(G, dim=1), v.repeat_interleave(G, dim=1)
        ns = [x for x in ns for _ in range(G)]
        nl = [x for x in nl for _ in range(G)]
    ref = prefill_masked_dense(q, k, v, sm, ns, nl)
    if out.dtype == torch.float16:
        close_stated(out, ref, tag)
        return
    ref_p = prefill_p_rounded(q, k, v, sm, ns, nl, "bf16")
    close_stated(out, torch.from_numpy(ref_p), (tag, "weights rounded"))
    ref_absv = prefill_masked_dense(q, k, v.abs(), sm, ns, nl)
    close_counted(out, ref, ref_absv, tag, max_fraction)


def masked_attention_gpu(q, k, v, mask, sm, p_dtype=None):
    """torch restatement of the oracle's prefill_p_rounded on the GPU in fp32, for sizes the CPU oracle
    takes too long for (checked against it on a small case in test_gpu_prefill.py).
    q, k, v [B, H, N, D]; mask bool [H, N, N].  p_dtype None: plain masked softmax attention."""
    t = torch.matmul(q.float(), k.float().transpose(-1, -2)) * (sm * 1.4426950408889634)
    t = t.masked_fill(~mask[None], float("-inf"))
    alive = mask.any(-1)[None, :, :, None]
    M = torch.ceil(t.amax(dim=-1, keepdim=True))
    M = torch.where(alive, M, torch.zeros_like(M))
    p = torch.exp2(t - M)
    del t
    l = p.sum(-1, keepdim=True)
    if p_dtype is not None:
        p = p.to(p_dtype).float()
    o = torch.matmul(p, v.float()) / torch.where(alive, l, torch.ones_like(l))
    return torch.where(alive, o, torch.zeros_like(o))
