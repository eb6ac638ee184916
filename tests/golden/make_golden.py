"""Writes the golden fixtures of tests/golden/ (run from the repo root: python tests/golden/make_golden.py).

Two kinds of vectors, both small enough to commit:

* ``topk_ties.npz`` - adversarial score rows (ties, -inf, signed zeros, short rows) with the selection
  worked out here by brute force in plain Python (sort the (−score, key) pairs), independently of the
  oracle's torch code.  They pin the tie-break rule "score descending, then key index ascending".
* ``c1_toy.npz`` - the whole toy configuration C1 (2048 packed tokens, fp32 inputs regenerated from
  its seed): every selected key, and the outputs and gradients at every 16th token, computed by a
  loop-level numpy restatement of softmax attention over the selected keys in float64.

The reference repository holds no vectors for this path (its tests compare end-to-end logits with
real checkpoints), so these are the fixed points that both the oracle (CPU tests) and the HIP kernels
(GPU tests) are compared with.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from vlm_training_amd import workloads as W  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def brute_topk(row, K):
    """row: python floats of the causal window (key 0..len-1).  Returns ascending key list."""
    order = sorted(range(len(row)), key=lambda j: (-row[j], j))
    return sorted(order[:K])


def tie_cases():
    rng = np.random.default_rng(7)
    cases = []
    inf = float("inf")
    cases.append(("all_equal", [[1.0] * (i + 1) for i in range(12)], 4))
    cases.append(("descending_then_ties", [[float(5 - min(j, 5)) for j in range(i + 1)] for i in range(16)], 5))
    cases.append(("neg_inf_and_zeros", [[(-inf if (j % 3 == 0) else (0.0 if j % 2 else -0.0)) for j in range(i + 1)] for i in range(14)], 6))
    cases.append(("two_levels", [[(2.0 if (j * 7 + i) % 5 < 2 else 1.0) for j in range(i + 1)] for i in range(40)], 9))
    cases.append(("k_one", [[float((j * 13) % 7) for j in range(i + 1)] for i in range(20)], 1))
    cases.append(("k_exceeds_rows", [[float((j * 5) % 3) for j in range(i + 1)] for i in range(6)], 16))
    q = rng.integers(-3, 4, size=(70, 70)).astype(np.float32)
    cases.append(("random_small_ints", [[float(q[i, j]) for j in range(i + 1)] for i in range(70)], 8))
    big = rng.standard_normal((300, 300)).astype(np.float32)
    big[:, ::7] = big[:, :1]                      # every 7th key ties with key 0
    cases.append(("gaussian_with_tied_columns", [[float(big[i, j]) for j in range(i + 1)] for i in range(300)], 33))
    return cases


def write_ties():
    out = {}
    names = []
    for name, rows, K in tie_cases():
        L = len(rows)
        sc = np.full((L, L), -np.inf, dtype=np.float32)
        idx = np.full((L, K), -1, dtype=np.int32)
        n = np.zeros(L, dtype=np.int32)
        for i, row in enumerate(rows):
            sc[i, :len(row)] = np.asarray(row, dtype=np.float32)
            sel = brute_topk([float(np.float32(x)) for x in row], K)
            idx[i, :len(sel)] = sel
            n[i] = len(sel)
        out[name + "/scores"], out[name + "/idx"], out[name + "/n"], out[name + "/K"] = sc, idx, n, np.int32(K)
        names.append(name)
    out["names"] = np.array(names)
    np.savez_compressed(os.path.join(HERE, "topk_ties.npz"), **out)
    print("topk_ties.npz:", len(names), "cases")


def write_c1():
    w = W.C1
    t = W.make_inputs(w, device="cpu")
    q, k, v = (t[x].double().numpy() for x in ("q", "k", "v"))
    qi, ki, wi = (t[x].double().numpy() for x in ("q_idx", "k_idx", "w_idx"))
    dout = t["dout"].double().numpy()
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    K = w.top_k
    index_scale = w.Di ** -0.5 * w.Hi ** -0.5
    scale = D ** -0.5
    idx = np.full((T, K), -1, dtype=np.int32)
    n = np.zeros(T, dtype=np.int32)
    out = np.zeros((T, Hq, D))
    dq, dk, dv = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
    cu = list(w.cu)
    for a, b in zip(cu[:-1], cu[1:]):
        for tq in range(a, b):
            keys = np.arange(a, tq + 1)
            # indexer score in float32 arithmetic order-insensitively close to the operator: sum_h w_h relu(q_h . k) * scale
            dots = np.maximum(qi[tq] @ ki[keys].T, 0.0)            # (Hi, nk)
            sc = (wi[tq][:, None] * dots).sum(0) * index_scale
            sel = brute_topk([float(x) for x in sc], K)
            sel = np.asarray(sel, dtype=np.int64) + a
            idx[tq, :len(sel)] = sel
            n[tq] = len(sel)
            for hq in range(Hq):
                hk = hq // G
                s = (k[sel, hk] @ q[tq, hq]) * scale
                p = np.exp(s - s.max())
                p /= p.sum()
                o = p @ v[sel, hk]
                out[tq, hq] = o
                g = dout[tq, hq]
                dp = v[sel, hk] @ g
                ds = p * (dp - (p * dp).sum())
                dq[tq, hq] = (ds @ k[sel, hk]) * scale
                np.add.at(dk[:, hk], sel, np.outer(ds, q[tq, hq]) * scale)
                np.add.at(dv[:, hk], sel, np.outer(p, g))
    rows = np.arange(0, T, 16)
    np.savez_compressed(os.path.join(HERE, "c1_toy.npz"), idx=idx.astype(np.int16), n=n.astype(np.int16), rows=rows.astype(np.int32),
                        out=out[rows].astype(np.float32), dq=dq[rows].astype(np.float32),
                        dk=dk[rows].astype(np.float32), dv=dv[rows].astype(np.float32))
    print("c1_toy.npz: T", T, "rows kept", len(rows))


if __name__ == "__main__":
    write_ties()
    write_c1()
