#!/usr/bin/env python3
"""Benchmark of the DSA packed-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3] [--no-cpu-baseline]

A step is one forward + backward pass of the whole operator (indexer scores -> top-k -> sparse
attention forward -> sparse attention backward) over one synthetic packed batch that is already
resident in HBM.  Prints ONE JSON line: whole-operator tokens/s, the roofline figures of the
dominant kernel measured live with events on the launch stream, the per-stage times, and the CPU
oracle timed on a bounded sample of the same workload on this box's host cores.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0        # MI355X HBM3E, published
PEAK_MFMA_BF16_TFLOPS = 2500.0


def timed(fn, iters, warmup=1):
    """Average milliseconds of fn() measured with events on torch's current stream (the launch stream)."""
    for _ in range(warmup):
        fn()
    beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    beg.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return beg.elapsed_time(end) / iters


def cpu_baseline(w, threads, sample_only=False):
    """The CPU oracle (fp32 torch) fwd+bwd on this box's host cores: the whole workload, one segment at a time
    (segments are independent), or - ``sample_only`` - one long segment scaled by causal pairs.  Beside it the dense
    restatement of the operator the reference itself calls (per-segment causal attention with repeat_kv GQA,
    models/qwen3/model.py:125-129,166-169), fwd+bwd on the same tensors."""
    from oracle import dsa_ref as R
    from vlm_training_amd import workloads as W
    torch.set_num_threads(threads)
    P, _ = w.pair_counts()
    if sample_only or P > 2e8:                              # C4: 8.6e9 pairs do not finish in minutes
        cands = [L for L in w.seg_lens if L > w.top_k] or [max(w.seg_lens)]
        L = min(max(cands), 6144)
        sw = W.scaled(w, (L,), name=w.name + "-cpu-sample")
        what = f"one {L}-token segment of {w.name}"
    else:
        sw, what = w, f"the whole of {w.name}, segment by segment"
    t = W.make_inputs(sw, device="cpu")
    P_s, _ = sw.pair_counts()
    cu = sw.cu
    t0 = time.perf_counter()
    for a, b in zip(cu[:-1], cu[1:]):
        if b == a:
            continue
        idx, n = R.dsa_select(t["q_idx"][a:b], t["k_idx"][a:b], t["w_idx"][a:b], [0, b - a], sw.top_k)
        R.sparse_attention_grads(t["q"][a:b], t["k"][a:b], t["v"][a:b], idx, n, [0, b - a], t["dout"][a:b])
    dt = time.perf_counter() - t0
    t0 = time.perf_counter()
    for a, b in zip(cu[:-1], cu[1:]):
        if b == a:
            continue
        q, k, v = (t[x][a:b].float().requires_grad_(True) for x in ("q", "k", "v"))
        R.dense_varlen_causal(q, k, v, [0, b - a]).backward(t["dout"][a:b].float())
    dt_dense = time.perf_counter() - t0
    est, est_dense = dt * P / P_s, dt_dense * P / P_s       # the oracle's cost is proportional to causal pairs
    scaled = "" if sw is w else f"; scaled by causal pairs ({P_s} of {P}) to the whole batch"
    return {
        "value": w.T / est, "unit": "tokens/s", "cores": threads, "kind": "port",
        "sample": f"DSA oracle (indexer, top-k, sparse attention fwd+bwd) on {what}: {dt:.2f} s{scaled}",
        "dense_reference_operator": {"value": w.T / est_dense, "unit": "tokens/s", "seconds": dt_dense,
                                     "what": "dense causal packed attention fwd+bwd (what the reference calls), same tensors"},
    }


def _eager_qk_norm_rope(q, k, qw, kw, cos, sin, eps=1e-6):
    """The reference layer's own sequence of eager torch ops around the attention call, in bf16
    (models/qwen3_vl/model.py:256-269: per-head F.rms_norm, transpose to (1,H,T,D), apply_rope = x*cos +
    rotate_half(x)*sin, transpose back, .contiguous()) - timed beside the fused kernel, nothing else."""
    import torch.nn.functional as F

    def rope(x):                                         # x (1,H,T,D)
        half = x.shape[-1] // 2
        rot = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
        return x * cos[None, None] + rot * sin[None, None]

    qn = F.rms_norm(q, (q.shape[-1],), qw, eps).unsqueeze(0).transpose(1, 2)
    kn = F.rms_norm(k, (k.shape[-1],), kw, eps).unsqueeze(0).transpose(1, 2)
    qo, ko = rope(qn), rope(kn)
    return (qo.transpose(1, 2).reshape(q.shape).contiguous(), ko.transpose(1, 2).reshape(k.shape).contiguous())


def prologue_stage(w, dev, iters):
    """The fused element-wise kernels either side of the operator, at the workload's geometry: HBM-bound,
    so each is reported as algorithmic bytes / time against the 8 TB/s peak, beside the reference's own
    sequence of eager torch ops (F.rms_norm, transposes, apply_rope, contiguous copies) on the same GPU."""
    from vlm_training_amd import prologue
    T, Hq, Hkv, D = w.T, w.Hq, w.Hkv, w.D
    g = torch.Generator(device="cpu").manual_seed(w.seed)
    mk = lambda *s: torch.randn(*s, generator=g).bfloat16().to(dev)
    q, k, gq, gk = mk(T, Hq, D), mk(T, Hkv, D), mk(T, Hq, D), mk(T, Hkv, D)
    qw, kw = mk(D) * 0.1 + 1, mk(D) * 0.1 + 1
    ang = torch.arange(T, dtype=torch.float32, device=dev)[:, None] * (
        1.0 / 1e6 ** (torch.arange(0, D, 2, dtype=torch.float32, device=dev) / D))[None, :]
    cos, sin = torch.cat((ang.cos(), ang.cos()), -1).bfloat16(), torch.cat((ang.sin(), ang.sin()), -1).bfloat16()
    gate = mk(T, Hq, D)
    e = 2
    rows = (Hq + Hkv) * D * e
    res = {}

    def entry(ms, nbytes):
        gbs = nbytes / (ms * 1e-3) / 1e9
        return {"ms": ms, "algorithmic_bytes": nbytes, "GB/s": gbs, "frac_hbm_peak": gbs / PEAK_HBM_GBS}

    qr, kr = q.clone().requires_grad_(True), k.clone().requires_grad_(True)
    qwr, kwr = qw.clone().requires_grad_(True), kw.clone().requires_grad_(True)
    with torch.no_grad():
        ms = timed(lambda: prologue.qk_norm_rope(q, k, qw, kw, cos, sin), iters)
        res["qk_norm_rope_fwd"] = entry(ms, T * (2 * rows + 2 * D * e + (Hq + Hkv) * 4))
        eager = timed(lambda: _eager_qk_norm_rope(q, k, qw, kw, cos, sin), iters)
        res["qk_norm_rope_fwd"]["eager_torch_ms"] = eager
        ms = timed(lambda: prologue.sigmoid_gate(q, gate), iters)
        res["sigmoid_gate_fwd"] = entry(ms, T * Hq * D * e * 3)
    oq, ok = prologue.qk_norm_rope(qr, kr, qwr, kwr, cos, sin)
    ms = timed(lambda: torch.autograd.grad((oq, ok), (qr, kr, qwr, kwr), (gq, gk), retain_graph=True), iters)
    res["qk_norm_rope_bwd"] = entry(ms, T * (3 * rows + 2 * D * e + (Hq + Hkv) * 4))
    return res


def reference_operator(w, t, iters):
    """The reference's own operator on the same GPU and batch: torch.nn.attention.varlen.varlen_attn (dense
    causal, what train/model_attention.py:123-132 calls) against this library's dense path (no indexer)."""
    from vlm_training_amd import ops
    try:
        from torch.nn.attention.varlen import varlen_attn as torch_varlen_attn
    except Exception as e:
        return {"error": repr(e)[:200]}
    cu, msl = t["cu_seqlens"], w.max_seqlen

    def run(fn):
        q, k, v = (t[x].detach().requires_grad_(True) for x in ("q", "k", "v"))
        fn(q, k, v).backward(t["dout"])

    try:
        theirs = timed(lambda: run(lambda q, k, v: torch_varlen_attn(q, k, v, cu, cu, msl, msl, is_causal=True)), iters)
    except Exception as e:
        return {"error": repr(e)[:200]}
    ours = timed(lambda: run(lambda q, k, v: ops.dsa_varlen_attn(q, k, v, cu, msl)), iters)
    return {"what": "dense causal packed attention fwd+bwd on this workload (the operator the reference calls)",
            "torch_varlen_attn_ms": theirs, "this_library_dense_ms": ours, "speedup": theirs / ours}


def indexer_target_stage(w, t, iters):
    """The indexer's training path beside the operator: attention mass of the selected keys (one more pass over the
    forward's S = QK^T with the saved log-sum-exp: 2*Hq*D flop per selected pair, 2*Hkv*4 bytes of partial tables),
    index+top-k that also keeps the selected scores (every row scored), the KL loss with its gradient at the scores,
    and the indexer backward (query side 4*Hi*Di, key side 4*Hi*Di flop per causal pair of a visited tile)."""
    from vlm_training_amd import ops
    cu, msl, scale = t["cu_seqlens"], w.max_seqlen, w.D ** -0.5
    # as the operator runs them: the selection kernel leaves the bitmap (and the selected scores), forward and mass read it
    lib = ops._lib.load()
    bm = torch.empty((max(lib.dsa_attn_fwd_workspace_bytes(w.T, msl, 1), 4),), dtype=torch.uint8, device=t["q"].device) \
        if lib.dsa_get_tile_crossover() > 0 else None
    idx, n, sel = ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], cu, msl, w.top_k, return_scores=True, bitmap=bm)
    out, lse = ops.attn_fwd(t["q"], t["k"], t["v"], idx, n, cu, msl, scale, ws=bm, bitmap_ready=bm is not None)
    ms = timed(lambda: ops.attn_mass(t["q"], t["k"], lse, idx, n, cu, msl, scale, bitmap=bm), iters)
    P, S = w.pair_counts()
    res = {"attn_mass": {"ms": ms, "selected_pair_TFLOP/s": 2.0 * w.Hq * w.D * S / ms / 1e9,
                         "partial_table_GB/s": 2.0 * w.Hkv * 4 * S / ms / 1e6}}
    mass = ops.attn_mass(t["q"], t["k"], lse, idx, n, cu, msl, scale, bitmap=bm)
    res["index_topk_with_scores_ms"] = timed(
        lambda: ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], cu, msl, w.top_k, return_scores=True, bitmap=bm), iters)
    res["indexer_kl_ms"] = timed(lambda: ops.indexer_kl(sel, mass, n), iters)
    loss, dscore = ops.indexer_kl(sel, mass, n)
    res["mean_kl"] = float(loss.mean())
    if w.Di in (64, 128) and w.Hi <= 64:
        ms = timed(lambda: ops.indexer_bwd(t["q_idx"], t["k_idx"], t["w_idx"], idx, n, dscore, cu, msl), iters)
        res["indexer_bwd"] = {"ms": ms, "causal_pair_TFLOP/s": 8.0 * w.Hi * w.Di * P / ms / 1e9}
    return res


def vision_tower_operator(dev, iters):
    """The vision towers' form of the call (models/qwen3_vl/model.py:423-428): non-causal packed attention over the
    patches of each image, 16 heads of 72 (hidden 1152) or 64 (hidden 1024), six images of 768-4096 patches."""
    from vlm_training_amd import dispatch_varlen_attention
    try:
        from torch.nn.attention.varlen import varlen_attn as torch_varlen_attn
    except Exception:
        torch_varlen_attn = None
    lens = [4096, 4096, 2304, 1024, 4096, 768]
    T, H = sum(lens), 16
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=dev)
    g = torch.Generator(device=dev).manual_seed(5)
    res = {"what": f"non-causal packed attention fwd+bwd, {H} heads, images of {lens} patches"}
    for D in (72, 64):
        q, k, v = (torch.randn(T, H, D, device=dev, generator=g).mul_(0.5).bfloat16().requires_grad_(True) for _ in range(3))
        do = torch.randn(T, H, D, device=dev, generator=g).bfloat16()
        pairs = sum(n * n for n in lens)

        def run(fn):
            q.grad = k.grad = v.grad = None              # no accumulation kernels inside the timed region
            fn(q, k, v).backward(do)

        ms = timed(lambda: run(lambda a, b, c: dispatch_varlen_attention(a, b, c, cu, max(lens), causal=False)), iters)
        e = {"ms": ms, "TFLOP/s": 14.0 * H * D * pairs / ms / 1e9}          # 4 (forward) + 10 (backward) flop per pair, head and dim
        if torch_varlen_attn is not None:
            try:
                e["torch_varlen_attn_ms"] = timed(lambda: run(lambda a, b, c: torch_varlen_attn(
                    a, b, c, cu, cu, max(lens), max(lens), is_causal=False)), iters)
            except Exception as ex:
                e["torch_varlen_attn_error"] = repr(ex)[:200]
        res[f"head_dim_{D}"] = e
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)   # the first steps after start-up run a few percent slower
    ap.add_argument("--workload", default="C3")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample", action="store_true", help="time the CPU oracle on one segment only (about 10 s) instead of the whole workload")
    ap.add_argument("--crossover", type=int, default=None,
                    help="tile/gather split (rows with pos < top_k * crossover run on the tile kernels; 0 = gather kernels only)")
    ap.add_argument("--only-step", action="store_true", help="the timed steps and the roofline line only (for profiler runs)")
    ap.add_argument("--indexer-training", action="store_true",
                    help="with --only-step: also run the indexer's training path (mass, selected scores, KL, indexer backward)")
    ap.add_argument("--head-shard", type=int, default=1,
                    help="measure one GPU's share of the workload with the attention heads split this many ways (the "
                         "reference's tensor parallelism); implies --only-step")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy (a known-size kernel to scale rocprof's FETCH_SIZE/WRITE_SIZE by)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collectives, no sharding); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    from vlm_training_amd import ops, workloads as W
    w = W.WORKLOADS[args.workload]
    if args.head_shard > 1:
        w = W.head_shard(w, args.head_shard)
        args.only_step = True
    if args.crossover is not None:
        ops.set_tile_crossover(args.crossover)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    t = W.make_inputs(w, device=dev)
    cu, msl = t["cu_seqlens"], w.max_seqlen
    q = t["q"].requires_grad_(True)
    k = t["k"].requires_grad_(True)
    v = t["v"].requires_grad_(True)
    scale = w.D ** -0.5

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)          # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    def step():
        q.grad = k.grad = v.grad = None
        out = ops.dsa_varlen_attn(q, k, v, cu, msl, indexer_q=t["q_idx"], indexer_k=t["k_idx"], indexer_w=t["w_idx"],
                                  top_k=w.top_k)
        out.backward(t["dout"])

    # ---- the metric: whole-operator fwd+bwd --------------------------------------------------
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    wall0 = time.perf_counter()
    marks[0].record()
    for i in range(args.steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - wall0) * 1e3 / args.steps
    ms_per_step = max(marks[0].elapsed_time(marks[-1]) / args.steps, wall_ms)
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    pct = lambda f: per_step[min(len(per_step) - 1, int(f * len(per_step)))]
    tokens_per_s = w.T / (ms_per_step * 1e-3)

    # ---- per-stage times (each kernel alone, same stream) ------------------------------------
    it = max(2, min(args.steps, 20))
    with torch.no_grad():
        qd, kd, vd = q.detach(), k.detach(), v.detach()
        # as the operator runs them: the selection kernel leaves the bitmap, forward and backward read it, and the
        # query side of the backward forms delta itself where it owns every row (else the delta pass runs with it)
        lib = ops._lib.load()
        bm = torch.empty((max(lib.dsa_attn_fwd_workspace_bytes(w.T, msl, 1), 4),), dtype=torch.uint8, device=dev) \
            if lib.dsa_get_tile_crossover() > 0 else None
        idx, n = ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], cu, msl, w.top_k, bitmap=bm)
        out, lse = ops.attn_fwd(qd, kd, vd, idx, n, cu, msl, scale, ws=bm, bitmap_ready=bm is not None)
        bufs = ops.attn_bwd(t["dout"], qd, kd, vd, out, lse, idx, n, cu, msl, scale, 15,
                            (torch.empty_like(qd), torch.empty_like(kd), torch.empty_like(vd),
                             torch.empty((ops._lib.load().dsa_attn_bwd_workspace_bytes(w.T, w.Hq, msl, 1),),
                                         dtype=torch.uint8, device=dev)))
        stage_ms = {
            "index_topk": timed(lambda: ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], cu, msl, w.top_k, bitmap=bm), it),
            "attn_fwd": timed(lambda: ops.attn_fwd(qd, kd, vd, idx, n, cu, msl, scale, ws=bm, bitmap_ready=bm is not None), it),
        }
        # (part bits: 1 delta, 2 bitmap from the list, 4 query side, 8 key side)
        for name, part in (("bwd_dq", 1 | 4), ("bwd_dkv", 8)):
            stage_ms[name] = timed(lambda: ops.attn_bwd(t["dout"], qd, kd, vd, out, lse, idx, n, cu, msl, scale, part, bufs), it)
        # passes the step no longer runs at this workload, alone, for comparison
        passes_alone = {name: timed(lambda: ops.attn_bwd(t["dout"], qd, kd, vd, out, lse, idx, n, cu, msl, scale, part, bufs), it)
                        for name, part in (("delta_pass", 1), ("bitmap_from_list", 2), ("dq_reading_delta", 4))}

    # ---- roofline ----------------------------------------------------------------------------
    wk = w.work()
    S = wk["S"]
    unit = w.Hq * w.D * S                 # one flop-unit: a multiply-add pass over every selected (query, key, head, d)
    kern = {   # algorithmic flop per launch of the three attention kernels (selected pairs only)
        "attn_fwd": ("dsa_tile_fwd_kernel", 4 * unit),          # QK^T + PV
        "bwd_dq": ("dsa_tile_dq_kernel", 6 * unit),             # QK^T + dO V^T + dS K
        # QK^T + dO V^T + P^T dO + dS^T Q (head_dim 256 runs the producer/consumer form, twice)
        "bwd_dkv": ("dsa_tile_dkv2_kernel" if w.D <= 128 else "dsa_tile_dkvpc_kernel", 8 * unit),
    }
    dom = max(kern, key=lambda name: stage_ms[name])
    dom_kernel, dom_flop = kern[dom]
    achieved = dom_flop / (stage_ms[dom] * 1e-3) / 1e12
    # what the matrix cores actually execute: the tile kernels compute every causal pair of a visited tile and mask
    # the unselected ones, so their MFMA rate is the selected-pair rate times (executed pairs / selected pairs)
    xq, xk = w.executed_pairs(ops._lib.load().dsa_get_tile_crossover())
    executed_pairs = {"attn_fwd": xq, "bwd_dq": xq, "bwd_dkv": xk}
    executed = dom_flop / S * executed_pairs[dom] / (stage_ms[dom] * 1e-3) / 1e12
    executed_by_kernel = {kern[name][0]: kern[name][1] / S * executed_pairs[name] / (stage_ms[name] * 1e-3) / 1e12 / PEAK_MFMA_BF16_TFLOPS
                          for name in kern}
    t_roof_ms = {
        "index_topk": max(wk["F1"] / (PEAK_MFMA_BF16_TFLOPS * 1e12), wk["B2"] / (PEAK_HBM_GBS * 1e9)) * 1e3,
        "attn_fwd": max(wk["F3"] / (PEAK_MFMA_BF16_TFLOPS * 1e12), wk["B3"] / (PEAK_HBM_GBS * 1e9)) * 1e3,
        "attn_bwd": max(wk["F4"] / (PEAK_MFMA_BF16_TFLOPS * 1e12), wk["B4"] / (PEAK_HBM_GBS * 1e9)) * 1e3,
    }
    roof_total = sum(t_roof_ms.values())
    # per stage: measured time against the stage's nominal roofline (the larger of flop / MFMA peak and bytes / HBM
    # peak, the bytes being those a row gather of the selected keys would move) and against its flop alone
    stage_time = {"index_topk": stage_ms["index_topk"], "attn_fwd": stage_ms["attn_fwd"],
                  "attn_bwd": stage_ms["bwd_dq"] + stage_ms["bwd_dkv"]}
    stage_work = {"index_topk": (wk["F1"], wk["B2"]), "attn_fwd": (wk["F3"], wk["B3"]), "attn_bwd": (wk["F4"], wk["B4"])}
    stage_roofline = {}
    for name, (flop, nbytes) in stage_work.items():
        t_mfma, t_hbm = flop / (PEAK_MFMA_BF16_TFLOPS * 1e12) * 1e3, nbytes / (PEAK_HBM_GBS * 1e9) * 1e3
        stage_roofline[name] = {"ms": stage_time[name], "flop": flop, "bytes": nbytes, "t_mfma_ms": t_mfma, "t_hbm_ms": t_hbm,
                                "bound": "mfma" if t_mfma >= t_hbm else "hbm", "frac_nominal": max(t_mfma, t_hbm) / stage_time[name],
                                "frac_mfma": t_mfma / stage_time[name]}
    compute_bound_ms = (wk["F1"] + 3.5 * wk["F3"]) / (PEAK_MFMA_BF16_TFLOPS * 1e12) * 1e3
    traffic = None      # HBM bytes per launch as last measured with rocprofv3 --pmc (separate runs)
    try:
        if args.head_shard > 1:
            raise OSError("no counter run for head shards")
        with open(os.path.join(ROOT, "profiles", f"hbm_traffic_{args.workload}.json")) as fh:
            traffic = json.load(fh).get(dom_kernel)
    except OSError:
        pass
    result = {
        "metric": "DSA attn fwd+bwd packed tokens/s on 1 GPU at 32K; % MFMA/HBM roofline",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{w.name}: T={w.T} packed tokens, segments={list(w.seg_lens)}, Hq/Hkv/D={w.Hq}/{w.Hkv}/{w.D}, "
                               f"indexer {w.Hi}x{w.Di}, top_k={w.top_k}, fwd+bwd"},
        "roofline": {"bound": "mfma", "kernel": dom_kernel, "achieved": achieved, "peak": PEAK_MFMA_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / PEAK_MFMA_BF16_TFLOPS,
                     "executed": executed, "executed_frac": executed / PEAK_MFMA_BF16_TFLOPS,
                     "executed_pairs_over_selected": executed_pairs[dom] / S, "executed_frac_by_kernel": executed_by_kernel,
                     "traffic": traffic,
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of this command, scaled by a 1 GiB copy (profiles/)",
                     "algorithmic_flop": dom_flop, "avg_ms": stage_ms[dom]},
        "stage_ms": stage_ms,
        "passes_alone_ms": passes_alone,
        "ms_per_step_median": pct(0.5), "ms_per_step_p10": pct(0.1), "ms_per_step_p90": pct(0.9),
        "roofline_whole_op": {"compute_only_bound_ms": compute_bound_ms, "frac_compute_only": compute_bound_ms / ms_per_step,
                              "nominal_gather_roofline_ms": roof_total, "nominal_t_roof_ms": t_roof_ms, "stages": stage_roofline,
                              "note": "compute_only_bound = (F1 + 3.5*F3) / bf16 MFMA peak: selected-pair flop of indexer, "
                                      "forward and backward, the ceiling that applies to the tile kernels; the nominal figure "
                                      "prices the attention stages by the bytes a row gather of the selected keys would move, "
                                      "which the tile kernels do not move (K and V stay in cache)"},
        "device": torch.cuda.get_device_name(0),
    }
    if not args.only_step:
        it = min(it, 5)
        result["adjacent_kernels"] = prologue_stage(w, dev, it)
        result["reference_operator"] = reference_operator(w, t, it)
        result["vision_tower_operator"] = vision_tower_operator(dev, it)
    if not args.only_step or args.indexer_training:
        result["indexer_training"] = indexer_target_stage(w, t, min(it, 5))
    if not args.no_cpu_baseline and not args.only_step:
        result["cpu_baseline"] = cpu_baseline(w, torch.get_num_threads(), sample_only=args.cpu_sample)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
