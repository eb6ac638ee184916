"""GPU parity at the full sizes of the measurement configurations, and the paths only large inputs reach.

C2, C3 and C5 in full against the fp32 oracle (selection bit-exact on the GPU's own scores; out, dq, dk, dv within the
stated tolerance); C4 (one 131 072-token sequence) by size-independent statements plus the oracle on sampled query
rows; the chunked score/select loop forced onto a small input."""
import ctypes

import pytest
import torch

from oracle import dsa_ref as R
from tests.util import assert_close_bf16, oracle_grads_by_segment, oracle_topk_from_gpu_scores
from vlm_training_amd import _lib, ops, workloads as W

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _log(msg):
    print(msg, flush=True)


def _ptr(x):
    return ctypes.c_void_p(x.data_ptr())


# ------------------------------------------------------------------------------------------ C2, C3, C5 in full
@pytest.mark.timeout(900)
@pytest.mark.parametrize("name", ["C2", "C5", "C3"])
def test_measurement_configuration_in_full_against_the_oracle(name):
    w = W.WORKLOADS[name]
    _log(f"{w.name} in full: T={w.T}")
    t = W.make_inputs(w, device="cpu")
    d = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in t.items()}
    q, k, v = (d[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
    out, idx, n = ops.dsa_varlen_attn(q, k, v, d["cu_seqlens"], w.max_seqlen, indexer_q=d["q_idx"], indexer_k=d["k_idx"],
                                      indexer_w=d["w_idx"], top_k=w.top_k, return_indices=True)
    out.backward(d["dout"])
    sc = ops.indexer_scores(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen).cpu()
    torch.cuda.synchronize()
    want_idx, want_n = oracle_topk_from_gpu_scores(sc, list(w.cu), w.top_k)
    del sc
    assert torch.equal(n.cpu(), want_n)
    assert torch.equal(idx.cpu(), want_idx), "top-k index sets differ from the oracle on identical scores"
    ref = oracle_grads_by_segment(t, want_idx, want_n, list(w.cu))
    res = [assert_close_bf16(got, want, nm) for nm, got, want in zip(("out", "dq", "dk", "dv"), (out, q.grad, k.grad, v.grad), ref)]
    _log(f"  {w.name}: " + " ".join(f"({e:.2e},{c:.6f})" for e, c in res))


# ------------------------------------------------------------------------------------------ chunked score/select loop
@pytest.mark.parametrize("rows_per_chunk", [64, 100, 4])
def test_index_topk_in_several_chunks_equals_one_chunk_and_the_oracle(rows_per_chunk):
    """dsa_index_topk works through the query rows in chunks that fit its workspace; a workspace of a few rows forces
    the loop that otherwise only a 131 072-token sequence reaches (second and later chunks, row_begin > 0)."""
    _log(f"index_topk chunks of {rows_per_chunk} rows")
    lib = _lib.load()
    w = W.scaled(W.C3, (700, 33, 0, 420, 1), top_k=64, name="chunks")
    t = W.make_inputs(w, device=DEV, with_dout=False)
    T, N, K = w.T, len(w.seg_lens), w.top_k
    scale = (w.Di ** -0.5) * (w.Hi ** -0.5)
    ld = (w.max_seqlen + 31) // 32 * 32
    st = torch.cuda.current_stream().cuda_stream
    one_idx, one_n = ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], t["cu_seqlens"], w.max_seqlen, K)
    nbytes = rows_per_chunk * ld * 4
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=DEV)
    idx = torch.full((T, K), -7, dtype=torch.int32, device=DEV)
    n = torch.full((T,), -7, dtype=torch.int32, device=DEV)
    rc = lib.dsa_index_topk(_ptr(t["q_idx"]), _ptr(t["k_idx"]), _ptr(t["w_idx"]), _ptr(t["cu_seqlens"]), T, N, w.Hi, w.Di, K,
                            scale, 0, w.max_seqlen, _ptr(idx), _ptr(n), _ptr(ws), nbytes, st)
    assert rc == 0, lib.dsa_last_error().decode()
    torch.cuda.synchronize()
    assert torch.equal(idx, one_idx) and torch.equal(n, one_n)
    sc = ops.indexer_scores(t["q_idx"], t["k_idx"], t["w_idx"], t["cu_seqlens"], w.max_seqlen).cpu()
    want_idx, want_n = oracle_topk_from_gpu_scores(sc, list(w.cu), K)
    assert torch.equal(idx.cpu(), want_idx) and torch.equal(n.cpu(), want_n)
    # the variant that keeps the selected scores walks the same chunks
    sel = torch.empty((T, K), dtype=torch.float32, device=DEV)
    rc = lib.dsa_index_topk_scores(_ptr(t["q_idx"]), _ptr(t["k_idx"]), _ptr(t["w_idx"]), _ptr(t["cu_seqlens"]), T, N, w.Hi, w.Di,
                                   K, scale, 0, w.max_seqlen, _ptr(idx), _ptr(n), _ptr(sel), _ptr(ws), nbytes, st)
    assert rc == 0, lib.dsa_last_error().decode()
    _, _, one_sel = ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], t["cu_seqlens"], w.max_seqlen, K, return_scores=True)
    assert torch.equal(idx, one_idx) and torch.equal(sel, one_sel)
    # a workspace below four rows is refused, not overrun
    rc = lib.dsa_index_topk(_ptr(t["q_idx"]), _ptr(t["k_idx"]), _ptr(t["w_idx"]), _ptr(t["cu_seqlens"]), T, N, w.Hi, w.Di, K,
                            scale, 0, w.max_seqlen, _ptr(idx), _ptr(n), _ptr(ws), 3 * ld * 4, st)
    assert rc == -3


def test_bound_above_the_lds_cache_keeps_short_rows_on_the_cached_select():
    """max_seqlen = None stands for the packed length; when that exceeds the select kernel's LDS cache (8192 keys)
    while every segment is shorter, the rows must still come out identical (they are served by the cached kernel, the
    rows longer than the cache by the one that re-reads memory)."""
    _log("top-k with a bound above the cache")
    w = W.scaled(W.C2, (4100, 3000, 900, 1300), top_k=256, name="bound")          # T = 9300 > 8192, longest row 4100
    t = W.make_inputs(w, device=DEV, with_dout=False)
    a = ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], t["cu_seqlens"], w.max_seqlen, w.top_k)
    b = ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], t["cu_seqlens"], w.T, w.top_k)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    # and with rows on both sides of the cache size in one launch
    w2 = W.scaled(W.C2, (9000, 500), top_k=300, name="bound2")
    t2 = W.make_inputs(w2, device=DEV, with_dout=False)
    idx, n = ops.index_topk(t2["q_idx"], t2["k_idx"], t2["w_idx"], t2["cu_seqlens"], w2.max_seqlen, w2.top_k)
    sc = ops.indexer_scores(t2["q_idx"], t2["k_idx"], t2["w_idx"], t2["cu_seqlens"], w2.max_seqlen)
    for r in (299, 300, 301, 4000, 8191, 8192, 8193, 8999, 9000 + 499):
        a0 = 0 if r < 9000 else 9000
        want = R.topk_from_score_rows([sc[r, : r - a0 + 1].cpu()], w2.top_k)[0]
        assert idx[r, : int(n[r])].cpu().tolist() == [a0 + c for c in want], r


# ------------------------------------------------------------------------------------------ C4
@pytest.mark.timeout(900)
def test_long_single_sequence_by_invariants_and_sampled_rows():
    """C4 as benchmarked (one causal sequence of 131 072 tokens, top-k 2048): the chunked score/select loop over 64
    chunks, the gather kernels at long range, bitmap rows of 4096 words.  Checked by statements that hold at any size
    (as for the headline configuration), and on sampled query rows against the oracle: selection bit-exact on the
    GPU's own scores of that row, out and dq of sampled query rows and dk, dv of sampled key rows within tolerance."""
    _log("C4 full size")
    w = W.C4
    lib = _lib.load()
    t = W.make_inputs(w, device=DEV)
    cu = t["cu_seqlens"]
    G, K, T = w.Hq // w.Hkv, w.top_k, w.T
    q, k, v = (t[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
    out, idx, n = ops.dsa_varlen_attn(q, k, v, cu, w.max_seqlen, indexer_q=t["q_idx"], indexer_k=t["k_idx"],
                                      indexer_w=t["w_idx"], top_k=K, return_indices=True)
    out.backward(t["dout"])
    torch.cuda.synchronize()
    out, dq, dk, dv = out.detach(), q.grad, k.grad, v.grad
    # selection: counts, range, order
    pos = torch.arange(T, device=DEV)
    assert torch.equal(n.long(), torch.clamp(pos + 1, max=K))
    col = torch.arange(K, device=DEV)[None, :]
    valid = col < n[:, None]
    assert bool(((idx == -1) | valid).all()) and bool((idx[valid] >= 0).all())
    assert bool((idx <= pos[:, None])[valid].all())
    assert bool(((idx[:, 1:] > idx[:, :-1]) | ~valid[:, 1:]).all())
    del valid, col
    for x in (out, dq, dk, dv):
        assert bool(torch.isfinite(x).all())
    # <dq, q> = <dk, k> per kv head (both are sum dS * S), and rows of P sum to one (sum_s dV[s] = sum_t dO[t])
    a = (dq.float() * t["q"].float()).sum(dim=(0, 2)).view(w.Hkv, G).sum(1)
    b = (dk.float() * t["k"].float()).sum(dim=(0, 2))
    assert torch.allclose(a, b, rtol=2e-2, atol=2e-2 * float(a.abs().max())), (a, b)
    want = t["dout"].float().sum(0).view(w.Hkv, G, w.D).sum(1)
    assert torch.allclose(dv.float().sum(0), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    # sampled rows: around top_k, around the select kernel's LDS cache, around the tile/gather crossover, the end
    X = lib.dsa_get_tile_crossover() * K                 # first row of the gather kernels (a multiple of 256 here)
    assert K < X < T and X % 256 == 0
    rows = [0, 1, K - 1, K, K + 1, 8191, 8192, 8193, X - 1, X, X + 1, 65535, 100003, T - 2, T - 1]
    scale = (w.Di ** -0.5) * (w.Hi ** -0.5)
    st = torch.cuda.current_stream().cuda_stream
    row_sc = torch.empty((1, T), dtype=torch.float32, device=DEV)
    idx_c, n_c = idx.cpu(), n.cpu()
    for r in rows:
        if r + 1 > K:
            rc = lib.dsa_indexer_scores(_ptr(t["q_idx"]), _ptr(t["k_idx"]), _ptr(t["w_idx"]), _ptr(cu), T, 1, w.Hi, w.Di, scale, 0,
                                        r, r + 1, 0, _ptr(row_sc), T, st)
            assert rc == 0, lib.dsa_last_error().decode()
            torch.cuda.synchronize()
            want_sel = R.topk_from_score_rows([row_sc[0, : r + 1].cpu()], K)[0]
        else:
            want_sel = list(range(r + 1))
        assert idx_c[r, : int(n_c[r])].tolist() == want_sel, f"row {r}: selection differs from the oracle"
        assert bool((idx_c[r, int(n_c[r]):] == -1).all())
    # out and dq of the sampled rows against the oracle's gather form (dq[t] depends on row t's own keys only)
    qc = t["q"].cpu().float().requires_grad_(True)
    kc, vc = t["k"].cpu().float(), t["v"].cpu().float()
    ref = R.sparse_attention_rows(qc, kc, vc, idx_c, n_c, rows)
    (ref * t["dout"].cpu().float()[rows]).sum().backward()
    e1 = assert_close_bf16(out[rows], ref.detach(), "out (sampled rows)")
    e2 = assert_close_bf16(dq[rows], qc.grad[rows], "dq (sampled rows)")
    _log(f"  C4 sampled rows: out ({e1[0]:.2e},{e1[1]:.6f}) dq ({e2[0]:.2e},{e2[1]:.6f})")
    # dk and dv of sampled key rows (first key tile, around top_k, around the select cache and the tile/gather crossover,
    # the last tile): every query that selected the key is looked up in idx and attended over its own keys by the oracle
    keys = [17, K, 8192, X, 100003, T - 70, T - 1]
    want_dk, want_dv = R.sparse_attention_key_rows(t["q"].cpu(), t["k"].cpu(), t["v"].cpu(), t["dout"].cpu(), idx_c, n_c, keys)
    e3 = assert_close_bf16(dk[keys], want_dk, "dk (sampled key rows)")
    e4 = assert_close_bf16(dv[keys], want_dv, "dv (sampled key rows)")
    _log(f"  C4 sampled key rows: dk ({e3[0]:.2e},{e3[1]:.6f}) dv ({e4[0]:.2e},{e4[1]:.6f})")
    # a second run is bit-identical
    q2, k2, v2 = (t[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
    out2, idx2, _ = ops.dsa_varlen_attn(q2, k2, v2, cu, w.max_seqlen, indexer_q=t["q_idx"], indexer_k=t["k_idx"],
                                        indexer_w=t["w_idx"], top_k=K, return_indices=True)
    out2.backward(t["dout"])
    torch.cuda.synchronize()
    assert torch.equal(out2, out) and torch.equal(idx2, idx)
    assert torch.equal(q2.grad, dq) and torch.equal(k2.grad, dk) and torch.equal(v2.grad, dv)
