"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs.

Bars: top-k index sets bit-exact given identical fp32 scores; outputs and gradients within
max-abs 2e-2 and cosine > 0.9995 of the fp32 oracle."""
import ctypes
import math

import pytest
import torch

from oracle import dsa_ref as R
from tests.util import assert_close_bf16, cosine, oracle_topk_from_gpu_scores
from vlm_training_amd import ops, workloads as W

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _log(msg):
    print(msg, flush=True)


# ------------------------------------------------------------------------------------------ D2
def _topk_case(scores, cu, K):
    T = scores.shape[0]
    idx, n = ops.topk_from_scores(scores.to(DEV).contiguous(), torch.tensor(cu, dtype=torch.int32, device=DEV), K)
    torch.cuda.synchronize()
    want_idx, want_n = oracle_topk_from_gpu_scores(scores, cu, K)
    assert torch.equal(n.cpu(), want_n)
    bad = (idx.cpu() != want_idx).any(dim=1).nonzero().flatten()
    assert bad.numel() == 0, f"rows differ: {bad[:8].tolist()} got {idx[bad[0]].tolist()[:16]} want {want_idx[bad[0]].tolist()[:16]}"


@pytest.mark.parametrize("K", [1, 7, 64, 300])
def test_topk_bit_exact_random_and_ties(K):
    _log(f"topk K={K}")
    g = torch.Generator().manual_seed(K)
    cu = [0, 130, 130, 700, 1000]
    T, ld = cu[-1], 576
    for kind in ("normal", "quantised", "all_equal", "signed_zero", "relu_like"):
        sc = torch.randn(T, ld, generator=g)
        if kind == "quantised":
            sc = torch.round(sc * 4) / 4
        elif kind == "all_equal":
            sc = torch.full((T, ld), 0.125)
        elif kind == "signed_zero":
            sc = torch.zeros(T, ld)
            sc[:, 1::2] = -0.0
            sc[:, ::7] = torch.randn(T, len(range(0, ld, 7)), generator=g).clamp(min=0) * 0.0
        elif kind == "relu_like":
            sc = torch.relu(sc) * torch.randn(T, 1, generator=g)
        _topk_case(sc, cu, K)


def test_topk_long_rows_uncached_path():
    _log("topk long rows")
    g = torch.Generator().manual_seed(3)
    L = 9000                                    # longer than the LDS key cache
    rows = [8191, 8192, 8193, L - 1]
    cu = [0, L]
    sc = torch.full((L, L), float("nan"))       # only a few rows are filled and checked
    K = 2048
    scd = torch.zeros(L, L)
    for r in rows:
        scd[r] = torch.round(torch.randn(L, generator=g) * 64) / 64
    idx, n = ops.topk_from_scores(scd.to(DEV), torch.tensor(cu, dtype=torch.int32, device=DEV), K)
    for r in rows:
        want = R.topk_from_score_rows([scd[r, :r + 1]], K)[0]
        assert idx[r].cpu().tolist() == want, r
        assert int(n[r]) == K


# ------------------------------------------------------------------------------------------ D1
@pytest.mark.parametrize("Hi,Di", [(4, 32), (32, 64), (64, 128), (32, 128), (20, 64)])
def test_indexer_scores_match_oracle(Hi, Di):
    _log(f"indexer Hi={Hi} Di={Di}")
    g = torch.Generator().manual_seed(Hi * 1000 + Di)
    cu = [0, 70, 70, 333, 520]
    T = cu[-1]
    qi = (torch.randn(T, Hi, Di, generator=g) * 0.5).bfloat16()
    ki = (torch.randn(T, Di, generator=g) * 0.5).bfloat16()
    w = (torch.randn(T, Hi, generator=g) * 0.5).bfloat16()
    sc = ops.indexer_scores(qi.to(DEV), ki.to(DEV), w.to(DEV), torch.tensor(cu, dtype=torch.int32, device=DEV), 263).cpu()
    for a, b in R.segments(cu):
        L = b - a
        if L == 0:
            continue
        want = R.indexer_scores_segment(qi[a:b], ki[a:b], w[a:b])
        low = torch.tril(torch.ones(L, L, dtype=torch.bool))
        got = sc[a:b, :L]
        err = (got[low] - want[low]).abs().max().item()
        assert err < 2e-5 * max(1.0, want[low].abs().max().item()), err
        assert torch.isneginf(sc[a:b, :L][~low]).all()      # untouched above the diagonal


# ------------------------------------------------------------------------------------------ whole operator
@pytest.fixture
def crossover():
    """Lets a test drive the tile kernels, the gather kernels, or a mix; restores the default afterwards."""
    old = ops.set_tile_crossover(16)
    ops.set_tile_crossover(old)
    yield ops.set_tile_crossover
    ops.set_tile_crossover(old)


def _run_case(w, check_bwd=True):
    t = W.make_inputs(w, device="cpu")
    cu = t["cu_seqlens"]
    d = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in t.items()}
    q = d["q"].clone().requires_grad_(True)
    k = d["k"].clone().requires_grad_(True)
    v = d["v"].clone().requires_grad_(True)
    out, idx, n = ops.dsa_varlen_attn(q, k, v, d["cu_seqlens"], w.max_seqlen, indexer_q=d["q_idx"], indexer_k=d["k_idx"],
                                      indexer_w=d["w_idx"], top_k=w.top_k, return_indices=True)
    # (1) top-k bit-exact given the GPU's own fp32 scores
    sc = ops.indexer_scores(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen).cpu()
    want_idx, want_n = oracle_topk_from_gpu_scores(sc, cu.tolist(), w.top_k)
    assert torch.equal(n.cpu(), want_n)
    assert torch.equal(idx.cpu(), want_idx), "top-k index sets differ from the oracle on identical scores"
    # (2) outputs / gradients against the fp32 oracle on the same selection
    if check_bwd:
        ref_out, rdq, rdk, rdv = R.sparse_attention_grads(t["q"], t["k"], t["v"], want_idx, want_n, cu, t["dout"])
        out.backward(d["dout"])
        torch.cuda.synchronize()
        res = [assert_close_bf16(out, ref_out, "out"), assert_close_bf16(q.grad, rdq, "dq"),
               assert_close_bf16(k.grad, rdk, "dk"), assert_close_bf16(v.grad, rdv, "dv")]
    else:
        ref_out = R.sparse_attention(t["q"], t["k"], t["v"], want_idx, want_n, cu)
        res = [assert_close_bf16(out, ref_out, "out")]
    _log(f"  {w.name}: " + " ".join(f"({e:.2e},{c:.6f})" for e, c in res))
    return out


def test_c1_toy_fp32_full():
    _log("C1 full")
    _run_case(W.C1)


def test_fp32_carrier_of_three_operands_equals_the_single_operand_launches():
    """q, k, v split into stacked bf16 parts by one launch, and the three gradients combined by one: bit-identical to
    the launches that take one operand each, and hi + lo gives the fp32 value back to 2^-16 relative."""
    _log("fp32 carrier, three operands")
    g = torch.Generator(device=DEV).manual_seed(5)
    T, Hq, Hkv, D = 333, 6, 2, 20
    q = torch.randn(T, Hq, D, device=DEV, generator=g)
    k = torch.randn(T, Hkv, D, device=DEV, generator=g)
    v = torch.randn(T, Hkv, D, device=DEV, generator=g)
    yq, yk, yv = ops._split_stack_qkv(q, k, v)
    assert torch.equal(yq, ops._split_stack(q, 0)) and torch.equal(yk, ops._split_stack(k, 1))
    assert torch.equal(yv, ops._split_stack(v, 0))
    back = yq[..., :D].float() + yq[..., D:2 * D].float()
    assert (back - q).abs().max() <= 2.0 ** -16 * q.abs().max()
    gq, gk, gv = (torch.randn(y.shape, device=DEV, generator=g).bfloat16() for y in (yq, yk, yv))
    dq, dk, dv = ops._split_combine_qkv(gq, gk, gv)
    assert torch.equal(dq, ops._split_combine(gq, 2)) and torch.equal(dk, ops._split_combine(gk, 1))
    assert torch.equal(dv, ops._split_combine(gv, 2))
    assert torch.equal(dq, gq[..., :D].float() + gq[..., 2 * D:3 * D].float())
    e = ops._split_stack_qkv(q[:0], k[:0], v[:0])
    assert [x.shape[0] for x in e] == [0, 0, 0]


def test_three_fp32_arrays_rounded_to_bf16_by_one_launch_equal_torch_casts():
    """The indexer's inputs of an fp32 caller: same bits as tensor.to(torch.bfloat16) (round to nearest even, infinities,
    signed zeros, subnormals, values that round up to the next power of two), NaN stays NaN; odd element counts."""
    _log("fp32 -> bf16 x3")
    g = torch.Generator(device=DEV).manual_seed(9)
    a = torch.randn(333, 5, 32, device=DEV, generator=g)
    b = torch.randn(333, 32, device=DEV, generator=g) * 1e-3
    c = torch.randn(333, 5, device=DEV, generator=g) * 1e4
    special = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), 1.0 + 2.0 ** -8, 1.0 + 2.0 ** -9, 1.0 + 3 * 2.0 ** -9,
                            1.99999988, 3.3895314e38, 1e-40, -1e-45, 65504.0], device=DEV)
    c.view(-1)[:special.numel()] = special
    c.view(-1)[-1] = float("nan")
    ya, yb, yc = ops._as_bf16_x3(a, b, c)
    for y, x in ((ya, a), (yb, b), (yc, c)):
        want = x.to(torch.bfloat16)
        assert y.shape == x.shape and y.dtype == torch.bfloat16 and y.is_contiguous()
        assert torch.equal(torch.isnan(y), torch.isnan(want))
        ok = ~torch.isnan(want)
        assert torch.equal(y.view(torch.int16)[ok], want.view(torch.int16)[ok])
    # anything but three fp32 tensors goes through the plain casts
    h = ops._as_bf16_x3(a.half(), b, c)
    assert torch.equal(h[0], a.half().to(torch.bfloat16)) and torch.equal(h[1], b.to(torch.bfloat16))


@pytest.mark.parametrize("name,segs,K", [
    ("C2", (700, 333, 40, 0, 515, 204), 256),
    ("C3", (1100, 64, 600, 284), 512),
    ("C5", (300, 65, 73, 107, 500, 33, 74), 128),
])
def test_scaled_configs(name, segs, K):
    _log(f"scaled {name}")
    _run_case(W.scaled(W.WORKLOADS[name], segs, top_k=K, name=name + "-scaled"))


@pytest.mark.parametrize("name,segs,K", [
    ("C3", (900, 70, 333), 64),
    ("C5", (420, 65, 300), 32),
    ("C1", (300, 200), 16),
])
def test_tile_and_gather_paths_agree_with_the_oracle(crossover, name, segs, K):
    """crossover 0 = gather kernels only, 1<<20 = tile kernels only, 2 = rows split at pos 2K (rounded to 256)."""
    _log(f"paths {name}")
    w = W.scaled(W.WORKLOADS[name], segs, top_k=K, name=name + "-paths")
    outs = {}
    for c in (0, 1 << 20, 2):
        crossover(c)
        outs[c] = _run_case(w).detach().float()
    assert (outs[0] - outs[1 << 20]).abs().max().item() < 2e-2
    split = (2 * K + 255) // 256 * 256            # mixed run: tile rows before the split, gather rows after
    a = 0
    for L in segs:
        assert torch.equal(outs[2][a:a + min(L, split)], outs[1 << 20][a:a + min(L, split)])
        assert torch.equal(outs[2][a + min(L, split):a + L], outs[0][a + min(L, split):a + L])
        a += L


def test_headline_geometry_with_full_top_k():
    """C3 head geometry with its real top_k = 2048 on segments long enough to have sparse rows spanning
    many bitmap words, plus an image-patch run (clustered selections)."""
    _log("C3 K=2048")
    _run_case(W.scaled(W.C3, (3000, 2304), top_k=2048, name="C3-k2048"))


@pytest.mark.parametrize("Hq,Hkv,D", [(6, 2, 128), (4, 4, 64), (16, 1, 128), (2, 1, 256)])
def test_sparse_path_odd_head_groups(Hq, Hkv, D):
    """Group sizes that are not the configs': G = 3 (padded to 4), 1, 16 and 2, through tiles and gather."""
    _log(f"odd groups {Hq}/{Hkv}/{D}")
    base = W.Workload("odd", torch.bfloat16, (333, 140, 515), Hq, Hkv, D, 8, 32, 48, 0.5, 77)
    old = ops.set_tile_crossover(3)                      # rows before pos 256 on tiles, the rest gathered
    try:
        _run_case(base)
    finally:
        ops.set_tile_crossover(old)


@pytest.mark.parametrize("n_short", [63, 64, 65, 300, 4500])
def test_many_segments_in_every_launch_order_of_the_key_tiles(n_short):
    """dK/dV lists its key tiles longest walk first; 300 segments go through the order table, 4500 are more than
    it holds (plain order).  The query-side kernels hand their blocks out heaviest first over the whole batch for up to
    64 segments (a wave holds the lengths in its lanes) and segment by segment beyond: 63, 64 and 65 segments sit on
    both sides of that.  Lengths 0-3 with two long segments between them."""
    _log(f"many segments {n_short}")
    g = torch.Generator().manual_seed(23 + n_short)
    lens = torch.randint(0, 4, (n_short,), generator=g).tolist()
    lens[n_short // 3] = 333
    lens[2 * n_short // 3] = 130
    cu = [0]
    for L in lens:
        cu.append(cu[-1] + L)
    T, Hq, Hkv, D = cu[-1], 4, 2, 64
    q = (torch.randn(T, Hq, D, generator=g) * 0.7).bfloat16()
    k = (torch.randn(T, Hkv, D, generator=g) * 0.7).bfloat16()
    v = (torch.randn(T, Hkv, D, generator=g) * 0.7).bfloat16()
    do = torch.randn(T, Hq, D, generator=g).bfloat16()
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    out = ops.dsa_varlen_attn(qd, kd, vd, torch.tensor(cu, dtype=torch.int32, device=DEV), 333)
    out.backward(do.to(DEV))
    qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
    ref = R.dense_varlen_causal(qr, kr, vr, cu)
    ref.backward(do.float())
    assert_close_bf16(out, ref, "out")
    assert_close_bf16(qd.grad, qr.grad, "dq")
    assert_close_bf16(kd.grad, kr.grad, "dk")
    assert_close_bf16(vd.grad, vr.grad, "dv")


@pytest.mark.parametrize("D,Hq,Hkv,segs,K", [
    (128, 4, 1, (3000, 700, 1), 256),                      # one GPU's share of an 8-way head-sharded layer: 31 workgroups
    (256, 8, 1, (1669, 300), 128),                         # head_dim 256, both halves of head_dim write one partial slot
    (64, 2, 2, (2500,), 0),                                # dense, a single segment, one head per kv head
    (128, 12, 3, (1100, 1300, 90), 64),                    # three heads per kv head (padded to four)
])
def test_key_tile_walks_cut_into_pieces_match_the_oracle(D, Hq, Hkv, segs, K):
    """A dK/dV launch of few workgroups cuts long key-tile walks into pieces (fp32 partial sums added in piece order by a
    second kernel).  The launch-order table in the workspace must say that walks were cut here; out, dq, dk, dv against
    the oracle as everywhere; a second run is bit-identical."""
    _log(f"pieces D={D} {Hq}/{Hkv} segs={segs} K={K}")
    w = W.Workload("pieces", torch.bfloat16, segs, Hq, Hkv, D, 8, 32, max(K, 1), 0.5, 901)
    t = W.make_inputs(w, device="cpu")
    d = {k_: (v_.to(DEV) if torch.is_tensor(v_) else v_) for k_, v_ in t.items()}
    scale = D ** -0.5
    if K:
        idx, n = ops.index_topk(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen, K)
    else:
        idx, n = None, None
    out, lse = ops.attn_fwd(d["q"], d["k"], d["v"], idx, n, d["cu_seqlens"], w.max_seqlen, scale)
    lib = ops._lib.load()
    ws_bytes = lib.dsa_attn_bwd_workspace_bytes(w.T, Hq, w.max_seqlen, 1 if K else 0)
    ws = torch.zeros((ws_bytes,), dtype=torch.uint8, device=DEV)
    bufs = (torch.empty_like(d["q"]), torch.empty_like(d["k"]), torch.empty_like(d["v"]), ws)
    dq, dk, dv, _ = ops.attn_bwd(d["dout"], d["q"], d["k"], d["v"], out, lse, idx, n, d["cu_seqlens"], w.max_seqlen, scale, 15, bufs)
    torch.cuda.synchronize()
    lib.dsa_tile_order_bytes.restype = ctypes.c_size_t
    order_bytes = (lib.dsa_tile_order_bytes(w.T) + 255) // 256 * 256
    header = ws[ws_bytes - order_bytes: ws_bytes - order_bytes + 16].view(torch.int32).cpu().tolist()
    assert header[0] > 0 and header[1] >= 32 and header[2] > 0, header      # entries, steps per piece, tiles that were cut
    if K:
        wi, wn = idx.cpu(), n.cpu()
        ro, rq, rk, rv = R.sparse_attention_grads(t["q"], t["k"], t["v"], wi, wn, t["cu_seqlens"], t["dout"])
    else:
        qf, kf, vf = (t[x].float().requires_grad_(True) for x in ("q", "k", "v"))
        ro = R.dense_varlen_causal(qf, kf, vf, t["cu_seqlens"])
        ro.backward(t["dout"].float())
        rq, rk, rv, ro = qf.grad, kf.grad, vf.grad, ro.detach()
    for name, got, want in (("out", out, ro), ("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        assert_close_bf16(got, want, name)
    dk1, dv1 = dk.clone(), dv.clone()
    ops.attn_bwd(d["dout"], d["q"], d["k"], d["v"], out, lse, idx, n, d["cu_seqlens"], w.max_seqlen, scale, 15, bufs)
    assert torch.equal(dk, dk1) and torch.equal(dv, dv1)


@pytest.mark.parametrize("D,Hq,Hkv,segs,K,sparse", [
    (64, 16, 1, (128, 64), 4, True),                       # sixteen heads and a few hundred queries on the same four keys
    (256, 16, 2, (716, 65, 73, 512, 300), 4, True),        # the head geometry of C5 (group of 8, head_dim 256)
    (256, 64, 4, (2, 2, 257, 2, 31, 200), 4, True),
    (128, 48, 3, (64, 257, 64, 1), 4, True),
    (128, 12, 3, (257, 128, 200, 129), 4, True),
    (64, 64, 4, (127, 257, 5, 127, 257, 127), 4, True),
    (128, 64, 4, (31, 2, 200, 1, 2), 4, True),
    (256, 64, 4, (127, 32, 127, 257, 31, 300), 0, False),  # dense causal, group of 16
    (128, 16, 1, (2, 2, 300, 1, 100, 1), 0, False),
])
def test_large_head_groups_with_few_keys_keep_dv_within_the_bound(D, Hq, Hkv, segs, K, sparse):
    """dV[s] sums P * dO over every (query, head) that attends s.  With few keys per query the probabilities are
    large, and with a large head group many rows meet in one key row: the bf16 rounding of P then piles up.  The
    key-side kernel carries the rounding remainder of P for such blocks; these are the geometries where it matters."""
    _log(f"few keys D={D} {Hq}/{Hkv} segs={segs} K={K}")
    w = W.Workload("fewkeys", torch.bfloat16, segs, Hq, Hkv, D, 8, 32, max(K, 1), 0.5, 100 + D + Hq)
    if sparse:
        _run_case(w)
        return
    t = W.make_inputs(w, device="cpu")
    qd, kd, vd = (t[x].to(DEV).requires_grad_(True) for x in ("q", "k", "v"))
    out = ops.dsa_varlen_attn(qd, kd, vd, t["cu_seqlens"].to(DEV), w.max_seqlen)
    out.backward(t["dout"].to(DEV))
    qr, kr, vr = (t[x].float().requires_grad_(True) for x in ("q", "k", "v"))
    ref = R.dense_varlen_causal(qr, kr, vr, t["cu_seqlens"])
    ref.backward(t["dout"].float())
    for name, got, want in (("out", out, ref), ("dq", qd.grad, qr.grad), ("dk", kd.grad, kr.grad), ("dv", vd.grad, vr.grad)):
        assert_close_bf16(got, want, name)


def test_dense_path_equals_reference_semantics():
    _log("dense path")
    g = torch.Generator().manual_seed(11)
    cu = [0, 190, 190, 400, 431]
    T = cu[-1]
    for Hq, Hkv, D in ((8, 2, 64), (4, 4, 128), (16, 2, 256), (6, 2, 128)):
        q = (torch.randn(T, Hq, D, generator=g) * 0.7).bfloat16()
        k = (torch.randn(T, Hkv, D, generator=g) * 0.7).bfloat16()
        v = (torch.randn(T, Hkv, D, generator=g) * 0.7).bfloat16()
        do = torch.randn(T, Hq, D, generator=g).bfloat16()
        qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
        out = ops.dsa_varlen_attn(qd, kd, vd, torch.tensor(cu, dtype=torch.int32, device=DEV), 210)
        out.backward(do.to(DEV))
        qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
        ref = R.dense_varlen_causal(qr, kr, vr, cu)
        ref.backward(do.float())
        assert_close_bf16(out, ref, f"out {Hq}/{Hkv}/{D}")
        assert_close_bf16(qd.grad, qr.grad, "dq")
        assert_close_bf16(kd.grad, kr.grad, "dk")
        assert_close_bf16(vd.grad, vr.grad, "dv")


@pytest.mark.parametrize("profile", ["rising", "falling", "all_low", "spikes", "all_high"])
@pytest.mark.parametrize("D", [128, 256])
def test_forward_reference_point_follows_logits_of_any_scale(profile, D):
    """The forward forms P against a running reference and looks for a tile's maximum only when a sum says it must:
    logits that rise by hundreds along the keys (the reference has to move again and again), fall (it never moves
    after the first tile), sit far below zero (nothing may underflow as a whole), far above (nothing may overflow),
    or spike in single keys - out, lse and dv against fp32 softmax of the same bf16 inputs."""
    _log(f"reference point {profile} D={D}")
    g = torch.Generator().manual_seed(3)
    T, Hq, Hkv = 700, 4, 2
    cu = [0, 450, 700]
    u = torch.nn.functional.normalize(torch.randn(D, generator=g), dim=0)
    pos = torch.arange(T, dtype=torch.float32)
    level = {"rising": pos * 0.6 - 100, "falling": 150 - pos * 0.6, "all_low": -300 + torch.randn(T, generator=g),
             "all_high": 300 + torch.randn(T, generator=g),
             "spikes": torch.where((pos.long() % 97) == 13, torch.tensor(120.0), torch.tensor(-20.0))}[profile]
    # logit(t, s) = scale * q[t].k[s] = level[s] + noise: q = sqrt(D) u (+ noise), k[s] = level[s] u (+ noise)
    q = (D ** 0.5 * u + 0.05 * torch.randn(T, Hq, D, generator=g)).bfloat16()
    k = (level[:, None, None] * u + 0.05 * torch.randn(T, Hkv, D, generator=g)).bfloat16()
    v = torch.randn(T, Hkv, D, generator=g).bfloat16()
    do = torch.randn(T, Hq, D, generator=g).bfloat16()
    cu_d = torch.tensor(cu, dtype=torch.int32, device=DEV)
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    out = ops.dsa_varlen_attn(qd, kd, vd, cu_d, 450)
    out.backward(do.to(DEV))
    _, lse = ops.attn_fwd(q.to(DEV), k.to(DEV), v.to(DEV), None, None, cu_d, 450, D ** -0.5)
    qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
    ref = R.dense_varlen_causal(qr, kr, vr, cu)
    ref.backward(do.float())
    want_lse = torch.empty(Hq, T)
    for a, b in zip(cu[:-1], cu[1:]):
        logit = torch.einsum("thd,shd->hts", q[a:b].float(), k[a:b].float().repeat_interleave(Hq // Hkv, dim=1)) * D ** -0.5
        logit = logit.masked_fill(torch.ones(b - a, b - a, dtype=torch.bool).triu(1), float("-inf"))
        want_lse[:, a:b] = torch.logsumexp(logit, dim=-1)
    assert torch.isfinite(lse).all()
    assert (lse.cpu() - want_lse).abs().max() <= 2e-3 * max(1.0, want_lse.abs().max().item())
    assert_close_bf16(out, ref, f"out {profile}")
    # (keys of norm 300 multiply the bf16 rounding of dS into dq far beyond the bound of ordinary inputs: the backward
    # is checked for the finite results and for dv, which no key scales)
    assert all(torch.isfinite(x.grad).all() for x in (qd, kd, vd))
    assert_close_bf16(vd.grad, vr.grad, "dv", steps=2)


@pytest.mark.parametrize("Hq,Hkv,D,causal,segs", [
    (16, 16, 72, False, (1024, 300, 77)),                  # the 1152 / 16 vision tower: padded to the head_dim-96 kernels
    (8, 2, 96, True, (700, 1, 333, 1500)),                 # head_dim 96 itself, causal, four heads per kv head
    (6, 2, 80, True, (513, 129)),                          # three heads per kv head (padded to four)
    (4, 1, 96, True, (3000, 700)),                         # few workgroups: dK/dV walks in pieces at head_dim 96
    (2, 2, 88, False, (2, 31, 64, 5)),                     # tiny segments
])
def test_head_dim_96_kernels_without_a_selection(Hq, Hkv, D, causal, segs):
    """Head dims between 64 and 96 run on head_dim-96 instantiations of the three tile kernels when no keys are selected
    (rows padded with zero columns by the operator; the 72-wide heads of the vision towers wasted 44 % of the matrix
    work at 128).  out, dq, dk, dv against the oracle; the kernels refuse head_dim 96 with a selection."""
    _log(f"head_dim 96 path: {Hq}/{Hkv}/{D} causal={causal} segs={segs}")
    g = torch.Generator().manual_seed(D * 7 + Hq)
    cu = [0]
    for L in segs:
        cu.append(cu[-1] + L)
    T = cu[-1]
    q = (torch.randn(T, Hq, D, generator=g) * 0.6).bfloat16()
    k = (torch.randn(T, Hkv, D, generator=g) * 0.6).bfloat16()
    v = (torch.randn(T, Hkv, D, generator=g) * 0.6).bfloat16()
    do = torch.randn(T, Hq, D, generator=g).bfloat16()
    qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
    cud = torch.tensor(cu, dtype=torch.int32, device=DEV)
    out = ops.dsa_varlen_attn(qd, kd, vd, cud, max(segs), causal=causal)
    assert out.shape == (T, Hq, D)
    out.backward(do.to(DEV))
    qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
    ref = R.dense_varlen_causal(qr, kr, vr, cu, causal=causal)
    ref.backward(do.float())
    assert_close_bf16(out, ref, "out")
    assert_close_bf16(qd.grad, qr.grad, "dq")
    assert_close_bf16(kd.grad, kr.grad, "dk")
    assert_close_bf16(vd.grad, vr.grad, "dv")
    if D == 96:                                             # the C ABI takes head_dim 96 as it is, and only without idx
        q96, k96, v96 = qd.detach(), kd.detach(), vd.detach()
        o2, lse2 = ops.attn_fwd(q96, k96, v96, None, None, cud, max(segs), D ** -0.5, causal=causal)
        assert torch.equal(o2, out.detach())
        idx = torch.zeros(T, 4, dtype=torch.int32, device=DEV)
        nn = torch.ones(T, dtype=torch.int32, device=DEV)
        with pytest.raises(RuntimeError):
            ops.attn_fwd(q96, k96, v96, idx, nn, cud, max(segs), D ** -0.5)


def test_non_causal_packed_attention_for_the_vision_towers():
    """causal=False: every key of the own segment (models/qwen3_vl/model.py:423-428 calls
    dispatch_varlen_attention(..., causal=False) with cu_seqlens built from grid_thw)."""
    _log("non-causal")
    import vlm_training_amd as M
    g = torch.Generator().manual_seed(21)
    cu = [0, 64, 64, 320, 401, 977]
    T = cu[-1]
    # 16 x 72 is the 1152-wide vision tower of the 8B models (head_dim between the kernels' sizes), 16 x 64 the 1024-wide one
    for Hq, Hkv, D in ((16, 16, 64), (16, 16, 72), (4, 2, 128), (2, 1, 256)):
        q = (torch.randn(T, Hq, D, generator=g) * 0.6).bfloat16()
        k = (torch.randn(T, Hkv, D, generator=g) * 0.6).bfloat16()
        v = (torch.randn(T, Hkv, D, generator=g) * 0.6).bfloat16()
        do = torch.randn(T, Hq, D, generator=g).bfloat16()
        qd, kd, vd = (x.to(DEV).requires_grad_(True) for x in (q, k, v))
        out = M.dispatch_varlen_attention(qd, kd, vd, torch.tensor(cu, dtype=torch.int32, device=DEV), 576, causal=False)
        assert out.shape == (T, Hq, D)
        out.backward(do.to(DEV))
        qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
        ref = R.dense_varlen_causal(qr, kr, vr, cu, causal=False)
        ref.backward(do.float())
        assert_close_bf16(out, ref, f"out {Hq}/{Hkv}/{D}")
        assert_close_bf16(qd.grad, qr.grad, "dq")
        assert_close_bf16(kd.grad, kr.grad, "dk")
        assert_close_bf16(vd.grad, vr.grad, "dv")
    with pytest.raises(ValueError):
        ops.dsa_varlen_attn(qd, kd, vd, torch.tensor(cu, dtype=torch.int32, device=DEV), 576, causal=False,
                            indexer_q=torch.zeros(T, 2, 32, device=DEV), indexer_k=torch.zeros(T, 32, device=DEV),
                            indexer_w=torch.zeros(T, 2, device=DEV), top_k=8)


def test_call_from_a_compiled_block():
    """The reference compiles every decoder block (train/infra.py:236-248); the operator must then run as an
    opaque call inside the compiled function (the reference wraps its own in @torch.compiler.disable,
    models/qwen3_5/model.py:90-91)."""
    _log("compiled caller")
    import vlm_training_amd as M
    g = torch.Generator().manual_seed(33)
    cu = torch.tensor([0, 100, 356], dtype=torch.int32, device=DEV)
    q = (torch.randn(356, 4, 128, generator=g) * 0.5).bfloat16().to(DEV)
    k = (torch.randn(356, 2, 128, generator=g) * 0.5).bfloat16().to(DEV)
    v = (torch.randn(356, 2, 128, generator=g) * 0.5).bfloat16().to(DEV)

    def block(q, k, v):
        return M.dispatch_varlen_attention(q * 1.0, k, v, cu, 256) + 1.0

    want = block(q, k, v)
    got = torch.compile(block, backend="eager")(q, k, v)
    assert torch.equal(got, want)


def test_topk_at_least_longest_segment_is_dense():
    _log("K >= L")
    w = W.scaled(W.C2, (300, 120, 77), top_k=512, name="C2-dense")
    t = W.make_inputs(w, device=DEV)
    out, idx, n = ops.dsa_varlen_attn(t["q"], t["k"], t["v"], t["cu_seqlens"], w.max_seqlen, indexer_q=t["q_idx"],
                                      indexer_k=t["k_idx"], indexer_w=t["w_idx"], top_k=512, return_indices=True)
    dense = ops.dsa_varlen_attn(t["q"], t["k"], t["v"], t["cu_seqlens"], w.max_seqlen)
    assert torch.equal(out, dense)                       # same kernel, same key order -> bit-identical
    cu = w.cu
    for a, b in zip(cu[:-1], cu[1:]):
        for r in (a, (a + b) // 2, b - 1):
            assert idx[r, : r - a + 1].cpu().tolist() == list(range(a, r + 1)) and int(n[r]) == r - a + 1
            assert (idx[r, r - a + 1:] == -1).all()


def test_packing_equivalence_pad_independence_determinism():
    _log("invariants")
    w = W.scaled(W.C2, (400, 150, 290), top_k=96, name="C2-inv")
    t = W.make_inputs(w, device=DEV)
    kw = dict(indexer_q=t["q_idx"], indexer_k=t["k_idx"], indexer_w=t["w_idx"], top_k=96, return_indices=True)
    out, idx, n = ops.dsa_varlen_attn(t["q"], t["k"], t["v"], t["cu_seqlens"], w.max_seqlen, **kw)
    out2, idx2, _ = ops.dsa_varlen_attn(t["q"], t["k"], t["v"], t["cu_seqlens"], w.max_seqlen, **kw)
    assert torch.equal(out, out2) and torch.equal(idx, idx2)            # I4 bitwise determinism
    cu = w.cu
    for a, b in zip(cu[:-1], cu[1:]):                                   # I2 packed == solo
        sl = slice(a, b)
        solo, sidx, _ = ops.dsa_varlen_attn(t["q"][sl], t["k"][sl], t["v"][sl], torch.tensor([0, b - a], dtype=torch.int32, device=DEV),
                                            b - a, indexer_q=t["q_idx"][sl], indexer_k=t["k_idx"][sl], indexer_w=t["w_idx"][sl],
                                            top_k=96, return_indices=True)
        assert torch.equal(torch.where(idx[sl] >= 0, idx[sl] - a, idx[sl]), sidx)
        assert torch.equal(out[sl], solo)
    pad = 100                                                           # I3 pad tail as one more segment
    ext = {name: torch.cat([t[name], torch.zeros(pad, *t[name].shape[1:], dtype=t[name].dtype, device=DEV)])
           for name in ("q", "k", "v", "q_idx", "k_idx", "w_idx")}
    cu_pad = torch.tensor(cu + [cu[-1] + pad], dtype=torch.int32, device=DEV)
    outp = ops.dsa_varlen_attn(ext["q"], ext["k"], ext["v"], cu_pad, w.max_seqlen, indexer_q=ext["q_idx"],
                               indexer_k=ext["k_idx"], indexer_w=ext["w_idx"], top_k=96)
    assert torch.equal(outp[: cu[-1]], out) and torch.isfinite(outp).all()


def test_backward_is_deterministic_and_unselected_keys_get_zero():
    _log("bwd determinism")
    w = W.scaled(W.C3, (500, 260), top_k=32, name="C3-det")
    t = W.make_inputs(w, device=DEV)
    grads = []
    for _ in range(2):
        q, k, v = (t[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
        out, idx, n = ops.dsa_varlen_attn(q, k, v, t["cu_seqlens"], w.max_seqlen, indexer_q=t["q_idx"], indexer_k=t["k_idx"],
                                          indexer_w=t["w_idx"], top_k=32, return_indices=True)
        out.backward(t["dout"])
        grads.append((q.grad.clone(), k.grad.clone(), v.grad.clone()))
    for a, b in zip(*grads):
        assert torch.equal(a, b)
    used = torch.zeros(w.T, dtype=torch.bool, device=DEV)
    used[idx[idx >= 0].long()] = True
    assert (grads[0][1][~used] == 0).all() and (grads[0][2][~used] == 0).all()


@pytest.mark.parametrize("segs,K", [
    ((700, 333, 40, 0, 515, 204), 256),       # rows inside and beyond top_k, an empty segment
    ((9000, 100), 512),                       # rows beyond the LDS cache of the selection kernel
    ((65,), 64), ((1100, 64, 600, 284), 2048),  # one key more than top_k; top_k above every row
])
def test_bitmap_left_by_the_selection_kernel_equals_the_one_built_from_the_list(segs, K):
    """index_topk(..., bitmap=) writes, from the ballots of its compaction, the words the forward builds from idx/n:
    every byte of the rows equal (also the zero words behind a row's window, over a buffer that held other bytes), same
    idx/n/scores as without it, and a forward and backward that read it give the bits of the ones that build their own;
    for the exact longest segment and for the bound T (odd word counts per row)."""
    _log(f"bitmap from top-k segs={segs} K={K}")
    w = W.scaled(W.C2, segs, top_k=K, name="bm")
    t = W.make_inputs(w, device=DEV)
    cu, scale, lib = t["cu_seqlens"], w.D ** -0.5, ops._lib.load()
    for ms in (w.max_seqlen, w.T):
        nbytes, used = lib.dsa_attn_fwd_workspace_bytes(w.T, ms, 1), w.T * ((ms + 31) // 32) * 4
        a = torch.full((nbytes,), 0xAB, dtype=torch.uint8, device=DEV)
        b = torch.full((nbytes,), 0xCD, dtype=torch.uint8, device=DEV)
        idx, n, sel = ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], cu, ms, K, return_scores=True, bitmap=a)
        idx2, n2, sel2 = ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], cu, ms, K, return_scores=True)
        assert torch.equal(idx, idx2) and torch.equal(n, n2) and torch.equal(sel, sel2)
        a2 = torch.full((nbytes,), 0x17, dtype=torch.uint8, device=DEV)
        idx3, n3 = ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], cu, ms, K, bitmap=a2)
        assert torch.equal(idx, idx3) and torch.equal(n, n3)
        out, lse = ops.attn_fwd(t["q"], t["k"], t["v"], idx, n, cu, ms, scale, ws=b)
        assert torch.equal(a[:used], b[:used]) and torch.equal(a2[:used], b[:used])
        out2, lse2 = ops.attn_fwd(t["q"], t["k"], t["v"], idx, n, cu, ms, scale, ws=a, bitmap_ready=True)
        assert torch.equal(out, out2) and torch.equal(lse, lse2) and torch.equal(a[:used], b[:used])
    with pytest.raises(RuntimeError, match="selection bitmap"):
        ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], cu, w.max_seqlen, K, bitmap=a[:8])


@pytest.mark.parametrize("sparse", [True, False])
def test_backward_passes_side_by_side_give_the_same_bits(sparse):
    """dQ on the library's second stream beside dK/dV (modes 1 and 2) against one pass after the other (mode 0), with
    eager work queued right behind the call on the caller's stream, which must wait for both passes."""
    _log(f"bwd overlap sparse={sparse}")
    w = W.scaled(W.C2, (900, 77, 410, 1300), top_k=128, name="overlap")
    t = W.make_inputs(w, device=DEV)
    cu, msl, scale = t["cu_seqlens"], w.max_seqlen, w.D ** -0.5
    idx, n = ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], cu, msl, w.top_k) if sparse else (None, None)
    out, lse = ops.attn_fwd(t["q"], t["k"], t["v"], idx, n, cu, msl, scale)
    old = ops.set_bwd_overlap(0)
    try:
        res = {}
        for mode in (0, 1, 2, 0, 2):
            ops.set_bwd_overlap(mode)
            for stream in (torch.cuda.current_stream(), torch.cuda.Stream()):
                stream.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(stream):
                    dq, dk, dv = ops.attn_bwd(t["dout"], t["q"], t["k"], t["v"], out, lse, idx, n, cu, msl, scale)
                    sums = dq.float().sum() + dk.float().sum() + dv.float().sum()     # queued behind the call
                torch.cuda.current_stream().wait_stream(stream)
                got = (dq, dk, dv, sums)
                if not res:
                    res = got
                for a, b in zip(res, got):
                    assert torch.equal(a, b), f"mode {mode}"
    finally:
        ops.set_bwd_overlap(old)
    assert old == 1


def test_reference_named_entry_points():
    _log("entry points")
    import vlm_training_amd as M
    g = torch.Generator().manual_seed(5)
    cu = torch.tensor([0, 100, 260], dtype=torch.int32, device=DEV)
    q = torch.randn(260, 8, 64, generator=g).bfloat16().to(DEV)
    k = torch.randn(260, 2, 64, generator=g).bfloat16().to(DEV)
    v = torch.randn(260, 2, 64, generator=g).bfloat16().to(DEV)
    a = M.dispatch_varlen_attention(q, k, v, cu, 160)
    b = M.run_varlen_attn(q, k, v, cu, 160)
    c = M.varlen_attn(q, k, v, cu, cu, 160, 160, is_causal=True)
    hf, none = M.varlen_attention_forward(q.transpose(0, 1).unsqueeze(0), k.transpose(0, 1).unsqueeze(0),
                                          v.transpose(0, 1).unsqueeze(0), cu.unsqueeze(0))
    assert none is None and hf.shape == (1, 260, 8, 64)
    assert torch.equal(a, b) and torch.equal(a, c) and torch.equal(a, hf[0])
    assert torch.equal(a, M.SelfAttention._run_varlen_attn(q, k, v, cu, 160))      # models/qwen3_5/model.py:90-98
    # two separately built offsets tensors with equal contents are accepted (torch's routine takes any two tensors);
    # different contents are not: this operator is self-attention
    assert torch.equal(a, M.varlen_attn(q, k, v, cu, cu.clone(), 160, 160, is_causal=True))
    with pytest.raises(ValueError):
        M.varlen_attn(q, k, v, cu, torch.tensor([0, 90, 260], dtype=torch.int32, device=DEV), 160, 160, is_causal=True)
    ref = R.dense_varlen_causal(q.cpu(), k.cpu(), v.cpu(), cu.cpu())
    assert_close_bf16(a, ref, "dispatch_varlen_attention")


def test_argument_errors_cross_the_boundary_as_exceptions(monkeypatch):
    q = torch.zeros(8, 4, 64, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(8, 3, 64, dtype=torch.bfloat16, device=DEV)
    cu = torch.tensor([0, 8], dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError):
        ops.dsa_varlen_attn(q, k, k, cu, 8)
    k = torch.zeros(8, 2, 96, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        ops.dsa_varlen_attn(q, k, k, cu, 8)
    q = torch.zeros(8, 4, 80, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(8, 2, 80, dtype=torch.bfloat16, device=DEV)
    assert ops.dsa_varlen_attn(q, k, k, cu, 8).shape == q.shape        # padded to head_dim 96 and cut back
    with pytest.raises(RuntimeError):
        ops.attn_fwd(q, k, k, None, None, cu, 8, 0.1)  # the C ABI itself covers head_dim 64 / 128 / 256 (and 96 without idx)
    big = torch.zeros(8, 2, 320, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        ops.dsa_varlen_attn(big, big, big, cu, 8)
    with pytest.raises(RuntimeError):
        ops.dsa_varlen_attn(q.cpu(), k.cpu(), k.cpu(), cu.cpu(), 8)
    monkeypatch.setenv("DSA_DEBUG_NAN", "1")
    qi = torch.zeros(8, 2, 32, dtype=torch.bfloat16, device=DEV)
    qi[3, 1, 5] = float("nan")
    with pytest.raises(ValueError):
        ops.index_topk(qi, torch.zeros(8, 32, dtype=torch.bfloat16, device=DEV),
                       torch.zeros(8, 2, dtype=torch.bfloat16, device=DEV), cu, 8, 2)


def test_debug_switch_checks_the_segment_table_before_any_launch(monkeypatch):
    """DSA_DEBUG_META=1 copies cu_seqlens to the host and refuses a table that does not end at T, that decreases, or
    whose longest segment exceeds max_seqlen (the kernels would clip such a segment without a word).  Without the
    switch nothing is copied and the same calls go through."""
    q = torch.zeros(64, 4, 64, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(64, 2, 64, dtype=torch.bfloat16, device=DEV)
    qi = torch.zeros(64, 2, 32, dtype=torch.bfloat16, device=DEV)
    ki = torch.zeros(64, 32, dtype=torch.bfloat16, device=DEV)
    wi = torch.zeros(64, 2, dtype=torch.bfloat16, device=DEV)
    good = torch.tensor([0, 40, 64], dtype=torch.int32, device=DEV)
    short = torch.tensor([0, 40, 60], dtype=torch.int32, device=DEV)
    back = torch.tensor([0, 50, 40, 64], dtype=torch.int32, device=DEV)
    monkeypatch.setenv("DSA_DEBUG_META", "1")
    launched = []
    real = ops._lib.load

    def counting():
        launched.append(1)
        return real()

    monkeypatch.setattr(ops._lib, "load", counting)
    for cu, bound, what in ((short, 64, "end at T"), (back, 64, "non-decreasing"), (good, 32, "below the longest segment")):
        with pytest.raises(ValueError, match=what):
            ops.dsa_varlen_attn(q, k, k, cu, bound)
        with pytest.raises(ValueError, match=what):
            ops.dsa_varlen_attn(q, k, k, cu, bound, indexer_q=qi, indexer_k=ki, indexer_w=wi, top_k=8)
    with pytest.raises(ValueError, match="below the longest segment"):
        ops.index_topk(qi, ki, wi, good, 39, 8)
    assert not launched                                          # every refusal came before the library was touched
    assert ops.dsa_varlen_attn(q, k, k, good, 40).shape == q.shape and launched
    monkeypatch.delenv("DSA_DEBUG_META")
    assert ops.dsa_varlen_attn(q, k, k, good, 64).shape == q.shape


# ------------------------------------------------------------------------------------------ golden fixtures
def _golden(name):
    import os

    import numpy as np
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name))


def test_golden_tie_cases_bit_exact():
    """Selections worked out by brute force in plain Python (tests/golden/make_golden.py)."""
    _log("golden ties")
    z = _golden("topk_ties.npz")
    for name in z["names"]:
        sc = torch.from_numpy(z[f"{name}/scores"])
        L, K = sc.shape[0], int(z[f"{name}/K"])
        idx, n = ops.topk_from_scores(sc.to(DEV).contiguous(), torch.tensor([0, L], dtype=torch.int32, device=DEV), K)
        torch.cuda.synchronize()
        assert torch.equal(n.cpu(), torch.from_numpy(z[f"{name}/n"])), name
        assert torch.equal(idx.cpu(), torch.from_numpy(z[f"{name}/idx"])), name


def test_golden_toy_configuration():
    """C1 against the float64 loop-level restatement: overlap of the selections, then outputs and
    gradients on the golden selection."""
    _log("golden C1")
    z = _golden("c1_toy.npz")
    w = W.C1
    t = W.make_inputs(w, device="cpu")
    d = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in t.items()}
    gidx = torch.from_numpy(z["idx"].astype("int32"))
    gn = torch.from_numpy(z["n"].astype("int32"))
    idx, n = ops.index_topk(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen, w.top_k)
    assert torch.equal(n.cpu(), gn)
    # the indexer rounds its fp32 inputs to bf16 once, so near-ties may be ordered differently from the
    # float64 scores: the selections must still share nearly all keys
    hit = sum(len(set(a[:m].tolist()) & set(b[:m].tolist())) for a, b, m in zip(idx.cpu(), gidx, gn.tolist()))
    overlap = hit / int(gn.sum())
    _log(f"  golden C1 selection overlap {overlap:.4f}")
    assert overlap > 0.97, overlap
    q, k, v = (d[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
    out = ops._DsaVarlenAttn.apply(q, k, v, d["cu_seqlens"], w.max_seqlen, gidx.to(DEV), gn.to(DEV), w.D ** -0.5, True)
    out.backward(d["dout"])
    torch.cuda.synchronize()
    rows = torch.from_numpy(z["rows"]).long()
    for name, got in (("out", out), ("dq", q.grad), ("dk", k.grad), ("dv", v.grad)):
        assert_close_bf16(got.detach().cpu()[rows], torch.from_numpy(z[name]), "golden " + name)


# ------------------------------------------------------------------------------------------ sync-free bound
def test_any_upper_bound_of_the_longest_segment_gives_the_same_result():
    """max_seqlen=None (bound = T, no device-to-host copy of the lengths) against the exact maximum:
    same selection, bit-identical outputs and gradients, sparse and dense, on a packed row built the
    way the reference's collate step builds it (padding tail as the last segment)."""
    _log("max_seqlen bound")
    w = W.random_packed_workload(W.scaled(W.C2, (1,), top_k=96), max_length=3072, seed=11, mean_len=500)
    assert w.T == 3072 and len(w.seg_lens) >= 3
    t = W.make_inputs(w, device=DEV)
    res = []
    for ms in (w.max_seqlen, None, 3000):
        q, k, v = (t[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
        out, idx, n = ops.dsa_varlen_attn(q, k, v, t["cu_seqlens"], ms, indexer_q=t["q_idx"], indexer_k=t["k_idx"],
                                          indexer_w=t["w_idx"], top_k=w.top_k, return_indices=True)
        out.backward(t["dout"])
        dense = ops.dsa_varlen_attn(t["q"], t["k"], t["v"], t["cu_seqlens"], ms)
        res.append((idx, n, out.detach(), q.grad, k.grad, v.grad, dense))
    for other in res[1:]:
        for a, b in zip(res[0], other):
            assert torch.equal(a, b)


# ------------------------------------------------------------------------------------------ full size
def test_headline_configuration_at_full_size_by_invariants():
    """C3 as benchmarked (32768 packed tokens), checked by statements that hold at any size:
    selections are ascending, causal, inside the query's segment and of size min(pos+1, K);
    softmax rows sum to one (V = 1 gives out = 1, and sum_s dV[s] = sum_t dO[t] per kv head);
    sum <dq, q> = sum <dk, k> per kv head (both equal sum dS.S); two runs are bit-identical."""
    _log("C3 full size")
    w = W.C3
    t = W.make_inputs(w, device=DEV)
    cu = t["cu_seqlens"]
    G = w.Hq // w.Hkv

    def run(vv):
        q, k, v = (x.clone().requires_grad_(True) for x in (t["q"], t["k"], vv))
        out, idx, n = ops.dsa_varlen_attn(q, k, v, cu, w.max_seqlen, indexer_q=t["q_idx"], indexer_k=t["k_idx"],
                                          indexer_w=t["w_idx"], top_k=w.top_k, return_indices=True)
        out.backward(t["dout"])
        return out.detach(), idx, n, q.grad, k.grad, v.grad

    out, idx, n, dq, dk, dv = run(t["v"])
    torch.cuda.synchronize()
    # selection
    pos = torch.cat([torch.arange(L, device=DEV) for L in w.seg_lens])
    seg0 = torch.cat([torch.full((L,), a, device=DEV) for a, L in zip(w.cu[:-1], w.seg_lens)])
    assert torch.equal(n.long(), torch.clamp(pos + 1, max=w.top_k))
    col = torch.arange(w.top_k, device=DEV)[None, :]
    valid = col < n[:, None]
    assert bool(((idx == -1) | valid).all()) and bool((idx[valid] >= 0).all())
    assert bool((idx >= seg0[:, None])[valid].all()) and bool((idx <= (seg0 + pos)[:, None])[valid].all())
    inc = (idx[:, 1:] > idx[:, :-1]) | ~valid[:, 1:]
    assert bool(inc.all())
    # finiteness and the <dq,q> = <dk,k> identity per kv head
    for x in (out, dq, dk, dv):
        assert bool(torch.isfinite(x).all())
    a = (dq.float() * t["q"].float()).sum(dim=(0, 2)).view(w.Hkv, G).sum(1)
    b = (dk.float() * t["k"].float()).sum(dim=(0, 2))
    assert torch.allclose(a, b, rtol=2e-2, atol=2e-2 * float(a.abs().max())), (a, b)
    # rows of P sum to one
    want = t["dout"].float().sum(0).view(w.Hkv, G, w.D).sum(1)
    got = dv.float().sum(0)
    assert torch.allclose(got, want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    out1 = run(torch.ones_like(t["v"]))[0]
    assert float((out1.float() - 1).abs().max()) <= 2 ** -7
    # determinism
    again = run(t["v"])
    for x, y in zip((out, idx, n, dq, dk, dv), again):
        assert torch.equal(x, y)


# ------------------------------------------------------------------------------------------ the torch routine itself
def test_dense_path_against_torch_varlen_attn_on_the_gpu():
    """The routine the reference calls (train/model_attention.py:123-132: torch.nn.attention.varlen.varlen_attn,
    here in the torch 2.10 ``is_causal`` form) runs on the GPU box; the dense path must agree with it on the
    packed layout the reference uses, forward and gradients, to the bar of two bf16 kernels."""
    _log("torch varlen_attn")
    try:
        from torch.nn.attention.varlen import varlen_attn as torch_varlen_attn
    except Exception as e:                               # older / differently built torch
        pytest.skip(f"torch.nn.attention.varlen not available: {e!r}")
    for w in (W.scaled(W.C3, (700, 64, 1300, 1), name="vs-torch-gqa4"), W.scaled(W.C5, (333, 512, 90), name="vs-torch-d256")):
        t = W.make_inputs(w, device=DEV)
        cu = t["cu_seqlens"]
        res = []
        for fn in ("torch", "ours"):
            q, k, v = (t[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
            if fn == "torch":
                try:
                    out = torch_varlen_attn(q, k, v, cu, cu, w.max_seqlen, w.max_seqlen, is_causal=True)
                except Exception as e:
                    pytest.skip(f"torch varlen_attn does not run on this build: {e!r}")
            else:
                out = ops.dsa_varlen_attn(q, k, v, cu, w.max_seqlen)
            out.backward(t["dout"])
            res.append((out.detach(), q.grad, k.grad, v.grad))
        torch.cuda.synchronize()
        for name, a, b in zip(("out", "dq", "dk", "dv"), res[1], res[0]):
            err, cos = assert_close_bf16(a, b, f"{w.name} {name} vs torch")
            _log(f"  {w.name} {name}: max-abs {err:.2e} cosine {cos:.6f}")


def test_dense_c_abi_entry_points_equal_the_general_ones():
    """dsa_dense_fwd / dsa_dense_bwd are the general entry points with no selection: same bits."""
    import ctypes
    from vlm_training_amd import _lib
    lib = _lib.load()
    w = W.scaled(W.C2, (300, 77, 500), name="dense-abi")
    t = W.make_inputs(w, device=DEV)
    q, k, v, cu = t["q"], t["k"], t["v"], t["cu_seqlens"]
    scale = w.D ** -0.5
    out0, lse0 = ops.attn_fwd(q, k, v, None, None, cu, w.max_seqlen, scale)
    dq0, dk0, dv0 = ops.attn_bwd(t["dout"], q, k, v, out0, lse0, None, None, cu, w.max_seqlen, scale)
    out, lse = torch.empty_like(out0), torch.empty_like(lse0)
    st = torch.cuda.current_stream().cuda_stream
    p = lambda x: ctypes.c_void_p(x.data_ptr())
    rc = lib.dsa_dense_fwd(p(q), p(k), p(v), p(cu), w.T, len(w.seg_lens), w.Hq, w.Hkv, w.D, scale, 0, w.max_seqlen, 1,
                           p(out), p(lse), st)
    assert rc == 0, lib.dsa_last_error()
    ws = torch.empty((lib.dsa_attn_bwd_workspace_bytes(w.T, w.Hq, w.max_seqlen, 0),), dtype=torch.uint8, device=DEV)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    rc = lib.dsa_dense_bwd(p(t["dout"]), p(q), p(k), p(v), p(out), p(lse), p(cu), w.T, len(w.seg_lens), w.Hq, w.Hkv, w.D,
                           scale, 0, w.max_seqlen, 1, p(dq), p(dk), p(dv), p(ws), ws.numel(), st)
    assert rc == 0, lib.dsa_last_error()
    torch.cuda.synchronize()
    for a, b in ((out, out0), (lse, lse0), (dq, dq0), (dk, dk0), (dv, dv0)):
        assert torch.equal(a, b)


# ------------------------------------------------------------------------------------------ indexer training target
@pytest.mark.parametrize("Hq,Hkv,D,K,segs", [(8, 2, 128, 64, (300, 1, 77, 513)), (32, 8, 128, 256, (1024, 700)),
                                              (6, 2, 64, 16, (130, 64, 5)), (16, 2, 256, 128, (600, 257)),
                                              (16, 1, 128, 32, (200, 90)), (5, 1, 128, 8, (97,)), (3, 3, 64, 100, (50, 400)),
                                              (2, 1, 64, 5, (40, 3)), (12, 4, 128, 2048, (2500,))])
def test_attention_mass_matches_the_oracle(Hq, Hkv, D, K, segs):
    """Target of the indexer's KL loss: head mean of the probabilities the forward gave the selected keys.
    Tolerance: |err| <= 2e-3 absolute on probabilities in [0,1] (bf16 inputs, fp32 exponentials against the
    forward's own lse) and rows summing to one within 2e-3."""
    _log(f"mass {Hq}/{Hkv}/{D} K={K}")
    w = W.Workload("mass", torch.bfloat16, segs, Hq, Hkv, D, 4, 32, K, 0.5, 77)
    t = W.make_inputs(w, device="cpu")
    d = {k_: (v_.to(DEV) if torch.is_tensor(v_) else v_) for k_, v_ in t.items()}
    scale = D ** -0.5
    idx, n = ops.index_topk(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen, K)
    out, lse = ops.attn_fwd(d["q"], d["k"], d["v"], idx, n, d["cu_seqlens"], w.max_seqlen, scale)
    mass = ops.attn_mass(d["q"], d["k"], lse, idx, n, d["cu_seqlens"], w.max_seqlen, scale)
    assert mass.shape == (w.T, K) and mass.dtype == torch.float32
    want = R.attention_mass(t["q"].float(), t["k"].float(), idx.cpu(), n.cpu(), list(w.cu), scale)
    err = (mass.cpu() - want).abs().max().item()
    assert err <= 2e-3, err
    assert (mass.sum(1).cpu() - 1.0).abs().max().item() <= 2e-3
    pad = torch.arange(K, device=DEV)[None, :] >= n[:, None]
    assert float(mass[pad].abs().sum()) == 0.0
    again = ops.attn_mass(d["q"], d["k"], lse, idx, n, d["cu_seqlens"], w.max_seqlen, scale)
    assert torch.equal(mass, again)                       # fixed summation order: bit-identical from run to run
    # with the bitmap the selection kernel left instead of one built here: the same bits
    bm = torch.empty((ops._lib.load().dsa_attn_fwd_workspace_bytes(w.T, w.max_seqlen, 1),), dtype=torch.uint8, device=DEV)
    idx2, n2 = ops.index_topk(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen, K, bitmap=bm)
    assert torch.equal(idx2, idx) and torch.equal(n2, n)
    assert torch.equal(ops.attn_mass(d["q"], d["k"], lse, idx, n, d["cu_seqlens"], w.max_seqlen, scale, bitmap=bm), mass)


def test_operator_returns_the_mass_beside_the_output_and_stays_differentiable():
    _log("return_mass")
    w = W.scaled(W.C2, (300, 120, 77), top_k=64, name="C2-mass")
    t = W.make_inputs(w, device=DEV)
    q, k, v = (t[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
    out, idx, n, mass = ops.dsa_varlen_attn(q, k, v, t["cu_seqlens"], w.max_seqlen, indexer_q=t["q_idx"],
                                            indexer_k=t["k_idx"], indexer_w=t["w_idx"], top_k=64,
                                            return_indices=True, return_mass=True)
    assert mass.shape == (w.T, 64) and not mass.requires_grad
    assert (mass.sum(1) - 1.0).abs().max().item() <= 2e-3
    want = R.attention_mass(t["q"].float().cpu(), t["k"].float().cpu(), idx.cpu(), n.cpu(), list(w.cu))
    assert (mass.cpu() - want).abs().max().item() <= 2e-3
    out.backward(t["dout"])
    ref = ops.dsa_varlen_attn(t["q"], t["k"], t["v"], t["cu_seqlens"], w.max_seqlen, indexer_q=t["q_idx"],
                              indexer_k=t["k_idx"], indexer_w=t["w_idx"], top_k=64)
    assert torch.equal(out, ref) and q.grad is not None and torch.isfinite(q.grad).all()
    with pytest.raises(ValueError):
        ops.dsa_varlen_attn(t["q"], t["k"], t["v"], t["cu_seqlens"], w.max_seqlen, return_mass=True)


@pytest.mark.parametrize("segs,K", [((300, 1, 77, 513), 64), ((40, 3), 5), ((900,), 1024)])
def test_selected_scores_and_indexer_kl(segs, K):
    """Scores of the selected keys (also for rows whose whole window is selected) and the KL loss of the indexer
    against the attention mass with its gradient.  Scores: same tolerance as the dense score rows (the same kernel
    wrote them); loss and gradient: 1e-4 absolute against torch's log_softmax / autograd on the same inputs."""
    _log(f"indexer kl {segs} K={K}")
    w = W.Workload("kl", torch.bfloat16, segs, 8, 2, 128, 8, 64, K, 0.5, 91)
    t = W.make_inputs(w, device="cpu")
    d = {k_: (v_.to(DEV) if torch.is_tensor(v_) else v_) for k_, v_ in t.items()}
    idx0, n0 = ops.index_topk(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen, K)
    idx, n, sel = ops.index_topk(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen, K, return_scores=True)
    assert torch.equal(idx, idx0) and torch.equal(n, n0)
    dense = ops.indexer_scores(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen)      # (T, ld)
    cu = list(w.cu)
    seg_start = torch.zeros(w.T, dtype=torch.long)
    for a, b in zip(cu[:-1], cu[1:]):
        seg_start[a:b] = a
    loc = (idx.cpu().long() - seg_start[:, None]).clamp(min=0)
    want_sel = torch.where(idx.cpu() >= 0, torch.gather(dense.cpu(), 1, loc), torch.zeros(()))
    assert torch.equal(sel.cpu(), want_sel)                 # the very values the selection was made from
    ref_sel = R.selected_scores(t["q_idx"].float(), t["k_idx"].float(), t["w_idx"].float(), idx.cpu(), n.cpu(), cu)
    assert (sel.cpu() - ref_sel).abs().max().item() <= 2e-2 * max(1.0, ref_sel.abs().max().item())
    scale = w.D ** -0.5
    out, lse = ops.attn_fwd(d["q"], d["k"], d["v"], idx, n, d["cu_seqlens"], w.max_seqlen, scale)
    mass = ops.attn_mass(d["q"], d["k"], lse, idx, n, d["cu_seqlens"], w.max_seqlen, scale)
    loss, dscore = ops.indexer_kl(sel, mass, n)
    s = sel.cpu().clone().requires_grad_(True)
    ref_loss = R.indexer_kl(s, mass.cpu(), n.cpu())
    (ref_loss.sum() / w.T).backward()
    assert (loss.cpu() - ref_loss.detach()).abs().max().item() <= 1e-4 * max(1.0, ref_loss.max().item())
    assert (dscore.cpu() - s.grad).abs().max().item() <= 1e-4 / w.T + 1e-7
    assert (loss >= -1e-6).all()                            # a KL divergence
    loss2, none = ops.indexer_kl(sel, mass, n, want_grad=False)
    assert none is None and torch.equal(loss2, loss)


@pytest.mark.parametrize("Hi,Di,K,segs", [(8, 64, 16, (130, 64, 5)), (64, 128, 64, (300, 1, 77, 513)), (32, 64, 100, (50, 400)),
                                           (40, 128, 8, (97, 200)), (64, 128, 512, (700,)), (8, 64, 16, (1700, 40, 600)),
                                           (4, 32, 128, (256, 512, 384))])
def test_indexer_backward_matches_autograd_of_the_oracle(Hi, Di, K, segs):
    """dq_idx, dk_idx, dw for an arbitrary gradient at the selected scores, against torch autograd through the
    oracle's score formula on the same bf16 inputs.  Tolerance as for the attention gradients (bf16 outputs)."""
    _log(f"indexer bwd Hi={Hi} Di={Di} K={K}")
    w = W.Workload("ibwd", torch.bfloat16, segs, 4, 2, 64, Hi, Di, K, 0.5, 123)
    t = W.make_inputs(w, device="cpu")
    d = {k_: (v_.to(DEV) if torch.is_tensor(v_) else v_) for k_, v_ in t.items()}
    idx, n = ops.index_topk(d["q_idx"], d["k_idx"], d["w_idx"], d["cu_seqlens"], w.max_seqlen, K)
    g = torch.Generator().manual_seed(5)
    dscore = torch.randn(w.T, K, generator=g)
    dscore = torch.where(torch.arange(K)[None] < n.cpu()[:, None], dscore, torch.zeros(()))
    dq, dk, dw = ops.indexer_bwd(d["q_idx"], d["k_idx"], d["w_idx"], idx, n, dscore.to(DEV), d["cu_seqlens"], w.max_seqlen)
    qi, ki, wi = (t[x].float().requires_grad_(True) for x in ("q_idx", "k_idx", "w_idx"))
    sel = R.selected_scores(qi, ki, wi, idx.cpu(), n.cpu(), list(w.cu))
    (sel * dscore).sum().backward()
    assert_close_bf16(dq, qi.grad, "dq_idx")
    assert_close_bf16(dk, ki.grad, "dk_idx")
    assert_close_bf16(dw, wi.grad, "dw")
    # run to run, and with the query side on the library's second stream beside the key side or behind it: the same bits
    old = ops.set_bwd_overlap(0)
    try:
        for mode in (0, 2, 1):
            ops.set_bwd_overlap(mode)
            dq2, dk2, dw2 = ops.indexer_bwd(d["q_idx"], d["k_idx"], d["w_idx"], idx, n, dscore.to(DEV), d["cu_seqlens"], w.max_seqlen)
            tail = dq2.float().sum() + dk2.float().sum() + dw2.sum()      # queued right behind the call
            assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dw, dw2), f"mode {mode}"
            assert torch.isfinite(tail)
    finally:
        ops.set_bwd_overlap(old)


def test_indexer_training_step_end_to_end():
    """Attention with return_mass, then the indexer's KL loss and its gradients, against the oracle: loss value
    and d loss / d (q_idx, k_idx, w) through torch autograd of the oracle's formulas."""
    _log("indexer training step")
    import vlm_training_amd as M
    w = W.Workload("itrain", torch.bfloat16, (300, 120, 77, 260), 8, 2, 128, 16, 64, 48, 0.5, 321)
    t = W.make_inputs(w, device="cpu")
    d = {k_: (v_.to(DEV) if torch.is_tensor(v_) else v_) for k_, v_ in t.items()}
    qi, ki, wi = (d[x].clone().requires_grad_(True) for x in ("q_idx", "k_idx", "w_idx"))
    out, idx, n, mass = M.dsa_varlen_attn(d["q"], d["k"], d["v"], d["cu_seqlens"], w.max_seqlen, indexer_q=qi, indexer_k=ki,
                                          indexer_w=wi, top_k=w.top_k, return_indices=True, return_mass=True)
    loss = M.indexer_kl_loss(qi, ki, wi, mass, d["cu_seqlens"], w.max_seqlen, w.top_k)
    (loss * 3.0).backward()
    # the same with the selection and its scores handed over by the operator (no second run of the indexer)
    o2, i2, n2, m2, s2 = M.dsa_varlen_attn(d["q"], d["k"], d["v"], d["cu_seqlens"], w.max_seqlen, indexer_q=qi, indexer_k=ki,
                                           indexer_w=wi, top_k=w.top_k, return_indices=True, return_mass=True,
                                           return_scores=True)
    assert torch.equal(o2, out) and torch.equal(i2, idx) and torch.equal(m2, mass)
    loss2 = M.indexer_kl_loss(qi, ki, wi, m2, d["cu_seqlens"], w.max_seqlen, w.top_k, selection=(i2, n2, s2))
    assert torch.equal(loss2, loss)
    rq, rk, rw = (t[x].float().requires_grad_(True) for x in ("q_idx", "k_idx", "w_idx"))
    sel = R.selected_scores(rq, rk, rw, idx.cpu(), n.cpu(), list(w.cu))
    ref = R.indexer_kl(sel, mass.cpu(), n.cpu()).mean()
    (ref * 3.0).backward()
    assert abs(loss.item() - ref.item()) <= 1e-3 * max(1.0, abs(ref.item()))
    for got, want, name in ((qi.grad, rq.grad, "dq_idx"), (ki.grad, rk.grad, "dk_idx"), (wi.grad, rw.grad, "dw")):
        assert got is not None and got.dtype == torch.bfloat16
        scale = want.abs().max().item()
        assert (got.float().cpu() - want).abs().max().item() <= 2e-2 * scale + 1e-6, name
        assert cosine(got.float().cpu(), want) > 0.9995, name
