"""Shared helpers of the GPU parity tests (the oracle is the checker, the HIP path is what is checked)."""
import torch

from oracle import dsa_ref as R

MAX_ABS = 2e-2      # tolerance stated for the bf16 path against the fp32 oracle
MIN_COS = 0.9995
# The stated bound is absolute.  The results themselves are stored in bf16, whose spacing at |x| in [2^e, 2^(e+1)) is
# 2^(e-7): from |x| = 4 on that spacing (0.031, 0.0625 at 8, ...) exceeds 2e-2, and no bf16 kernel can promise less
# than one step there.  So: |got - want| <= max(MAX_ABS, one bf16 step at |want|).


def bf16_step(x):
    """Spacing of bf16 values at magnitude |x| (8 significant bits): 2^(floor(log2|x|) - 7)."""
    x = x.abs().clamp(min=2.0 ** -126)
    return torch.exp2(torch.floor(torch.log2(x)) - 7)


def cosine(a, b):
    a, b = a.double().flatten(), b.double().flatten()
    den = a.norm() * b.norm()
    return 1.0 if den == 0 else float(torch.dot(a, b) / den)


def assert_close_bf16(got, want, name, max_abs=MAX_ABS, min_cos=MIN_COS, steps=1):
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    assert got.shape == want.shape, (name, got.shape, want.shape)
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    diff = (got - want).abs()
    err = diff.max().item()
    # a direction needs a vector: where the reference is zero up to fp32 rounding (dq of a one-token segment) the
    # cosine compares noise with noise, and only the absolute bound says anything
    cos = cosine(got, want) if want.abs().max().item() > 1e-4 else 1.0
    limit = torch.maximum(torch.full_like(want, max_abs), steps * bf16_step(want))
    excess = diff - limit
    worst = int(excess.argmax())
    assert excess.max().item() <= 0 and cos > min_cos, (
        f"{name}: |err| {diff.flatten()[worst].item():.4g} at |want| {want.abs().flatten()[worst].item():.4g} "
        f"(limit max({max_abs}, {steps} bf16 step(s) of |want|) = {limit.flatten()[worst].item():.4g}), max-abs {err:.4g}, "
        f"cosine {cos:.6f} (limit {min_cos})")
    return err, cos


def oracle_topk_from_gpu_scores(scores_cpu, cu, K):
    """Oracle top-k over the valid part of every row of a (T, ld) score matrix."""
    T = scores_cpu.shape[0]
    idx = torch.full((T, K), -1, dtype=torch.int32)
    n = torch.zeros(T, dtype=torch.int32)
    for a, b in R.segments(cu):
        L = b - a
        if L == 0:
            continue
        sc = scores_cpu[a:b, :L].clone()
        if L <= K:
            sc = torch.zeros(L, L)
        else:
            sc[:K] = 0.0            # dense rows: scores are not consulted (and were never written)
        sc = sc.masked_fill(torch.triu(torch.ones(L, L, dtype=torch.bool), 1), float("-inf"))
        idx[a:b], n[a:b] = R.topk_select_segment(sc, K, base=a)
    return idx, n


def oracle_grads_by_segment(t, idx, n, cu):
    """(out, dq, dk, dv) of the fp32 oracle, one segment at a time (segments are independent; the autograd graph of
    the longest one is what has to fit in host memory).  ``t``: dict of CPU tensors q, k, v, dout; ``idx``/``n``: the
    selection with global packed row ids."""
    outs, dqs, dks, dvs = [], [], [], []
    for a, b in R.segments(cu):
        if b == a:
            continue
        loc = torch.where(idx[a:b] >= 0, idx[a:b] - a, idx[a:b])
        o, dq, dk, dv = R.sparse_attention_grads(t["q"][a:b], t["k"][a:b], t["v"][a:b], loc, n[a:b], [0, b - a], t["dout"][a:b])
        outs.append(o); dqs.append(dq); dks.append(dk); dvs.append(dv)
    return torch.cat(outs), torch.cat(dqs), torch.cat(dks), torch.cat(dvs)
