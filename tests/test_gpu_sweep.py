"""Randomised geometries (fixed seeds) against the oracle: head_dim 64-256 with the padded sizes between, 1-4 kv heads,
group sizes 1-16 incl. 3 and 5, segments of 1-513 tokens, top-k 1-256, dense causal, dense non-causal and sparse; and the
indexer-training kernels (attention mass, selected scores, indexer backward) on their own set.  The hand-picked cases of
test_gpu_parity.py cover the known borders; this walks between them."""
import random

import pytest
import torch

from oracle import dsa_ref as R
from tests.util import assert_close_bf16, oracle_topk_from_gpu_scores
from vlm_training_amd import ops, workloads as W

pytestmark = pytest.mark.gpu
DEV = "cuda"
SEG_CHOICES = [1, 2, 5, 31, 32, 33, 64, 100, 127, 128, 129, 200, 257, 300, 513]


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_attention_on_random_geometries(seed):
    rng = random.Random(seed)
    for case in range(12):
        D = rng.choice([64, 72, 80, 96, 128, 256])
        Hkv = rng.choice([1, 2, 3, 4])
        Hq = Hkv * rng.choice([1, 2, 3, 4, 5, 8, 16])
        segs = tuple(rng.choice(SEG_CHOICES) for _ in range(rng.randint(1, 6)))
        K = rng.choice([1, 4, 16, 32, 64, 100, 256])
        sparse = rng.random() < 0.7
        causal = True if sparse else rng.random() < 0.7
        w = W.Workload(f"sweep{seed}_{case}", torch.bfloat16, segs, Hq, Hkv, D, rng.choice([8, 32, 64]), rng.choice([32, 64, 128]),
                       K, 0.5, 100 * seed + case)
        what = f"seed {seed} case {case}: D={D} Hq={Hq} Hkv={Hkv} segs={segs} K={K} sparse={sparse} causal={causal}"
        print(what, flush=True)
        t = W.make_inputs(w, device="cpu")
        d = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in t.items()}
        q, k, v = (d[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
        if sparse:
            out, idx, n = ops.dsa_varlen_attn(q, k, v, d["cu_seqlens"], w.max_seqlen, indexer_q=d["q_idx"], indexer_k=d["k_idx"],
                                              indexer_w=d["w_idx"], top_k=K, return_indices=True)
            sc = ops.indexer_scores(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen).cpu()
            wi, wn = oracle_topk_from_gpu_scores(sc, list(w.cu), K)
            assert torch.equal(idx.cpu(), wi) and torch.equal(n.cpu(), wn), what + ": selection"
            out.backward(d["dout"])
            ro, rq, rk, rv = R.sparse_attention_grads(t["q"], t["k"], t["v"], wi, wn, t["cu_seqlens"], t["dout"])
        else:
            out = ops.dsa_varlen_attn(q, k, v, d["cu_seqlens"], w.max_seqlen, causal=causal)
            out.backward(d["dout"])
            qf, kf, vf = (t[x].float().requires_grad_(True) for x in ("q", "k", "v"))
            ro = R.dense_varlen_causal(qf, kf, vf, t["cu_seqlens"], causal=causal)
            ro.backward(t["dout"].float())
            rq, rk, rv, ro = qf.grad, kf.grad, vf.grad, ro.detach()
        for name, got, want in (("out", out, ro), ("dq", q.grad, rq), ("dk", k.grad, rk), ("dv", v.grad, rv)):
            assert_close_bf16(got, want, what + ": " + name)


@pytest.mark.parametrize("seed", [0, 1])
def test_indexer_training_kernels_on_random_geometries(seed):
    rng = random.Random(1000 + seed)
    for case in range(10):
        D = rng.choice([64, 128, 256])
        Hkv = rng.choice([1, 2, 3, 4, 8])
        Hq = Hkv * rng.choice([1, 2, 3, 4, 5, 8, 16])
        Hi, Di = rng.choice([4, 8, 16, 32, 40, 64]), rng.choice([32, 64, 128])
        segs = tuple(rng.choice([1, 2, 5, 31, 33, 64, 100, 129, 257, 513, 700]) for _ in range(rng.randint(1, 5)))
        K = rng.choice([1, 4, 16, 64, 100, 256])
        w = W.Workload(f"n3_{seed}_{case}", torch.bfloat16, segs, Hq, Hkv, D, Hi, Di, K, 0.5, 500 + 100 * seed + case)
        what = f"seed {seed} case {case}: D={D} Hq={Hq} Hkv={Hkv} Hi={Hi} Di={Di} segs={segs} K={K}"
        print(what, flush=True)
        t = W.make_inputs(w, device="cpu")
        d = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in t.items()}
        scale = D ** -0.5
        idx, n = ops.index_topk(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen, K)
        out, lse = ops.attn_fwd(d["q"], d["k"], d["v"], idx, n, d["cu_seqlens"], w.max_seqlen, scale)
        mass = ops.attn_mass(d["q"], d["k"], lse, idx, n, d["cu_seqlens"], w.max_seqlen, scale)
        want = R.attention_mass(t["q"].float(), t["k"].float(), idx.cpu(), n.cpu(), list(w.cu), scale)
        assert (mass.cpu() - want).abs().max().item() <= 2e-3, what + ": mass"
        assert (mass.sum(1).cpu() - 1.0).abs().max().item() <= 2e-3, what + ": mass rows sum to one"
        live = torch.arange(K)[None] < n.cpu()[:, None]
        assert bool((mass.cpu()[~live] == 0).all()), what + ": slots past n[t]"
        g = torch.Generator().manual_seed(case)
        # the gradient the KL loss hands down is softmax - mass, small and of mixed sign: scaled to that size here
        dscore = torch.where(live, torch.randn(w.T, K, generator=g) * 0.05, torch.zeros(()))
        dq, dk, dw = ops.indexer_bwd(d["q_idx"], d["k_idx"], d["w_idx"], idx, n, dscore.to(DEV), d["cu_seqlens"], w.max_seqlen)
        qi, ki, wi = (t[x].float().requires_grad_(True) for x in ("q_idx", "k_idx", "w_idx"))
        sel = R.selected_scores(qi, ki, wi, idx.cpu(), n.cpu(), list(w.cu))
        (sel * dscore).sum().backward()
        assert_close_bf16(dq, qi.grad, what + ": dq_idx")
        assert_close_bf16(dk, ki.grad, what + ": dk_idx")
        assert_close_bf16(dw, wi.grad, what + ": dw")
        i2, n2, s2 = ops.index_topk(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen, K, return_scores=True)
        assert torch.equal(i2, idx) and torch.equal(n2, n), what + ": selection with scores"
        serr = ((s2.cpu() - sel.detach()).abs() * live).max().item()
        assert serr <= 2e-2 * max(1.0, sel.detach().abs().max().item()), what + f": selected scores {serr}"
