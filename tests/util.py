"""Shared helpers of the GPU parity tests (the oracle is the checker, the HIP path is what is checked)."""
import torch

from oracle import dsa_ref as R

MAX_ABS = 2e-2      # tolerance stated for the bf16 path against the fp32 oracle
MIN_COS = 0.9995


def cosine(a, b):
    a, b = a.double().flatten(), b.double().flatten()
    den = a.norm() * b.norm()
    return 1.0 if den == 0 else float(torch.dot(a, b) / den)


def assert_close_bf16(got, want, name, max_abs=MAX_ABS, min_cos=MIN_COS):
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    assert got.shape == want.shape, (name, got.shape, want.shape)
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    err = (got - want).abs().max().item()
    cos = cosine(got, want)
    assert err <= max_abs and cos > min_cos, f"{name}: max-abs {err:.4g} (limit {max_abs}), cosine {cos:.6f} (limit {min_cos})"
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
