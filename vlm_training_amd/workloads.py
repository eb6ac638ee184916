"""Synthetic packed batches for the five measurement configurations.

Everything is produced from ``torch.Generator(device='cpu').manual_seed(seed)`` in fp32 and then
cast, so the same call yields the same batch on any machine.  Segment lengths are literals.
The packing convention is the reference's: int32 ``cu_seqlens`` prefix sums with the pad tail as
one more segment (data/energon_dataloader.py:431-464, models/qwen3_vl/model.py:757-765).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    dtype: torch.dtype
    seg_lens: Tuple[int, ...]
    Hq: int
    Hkv: int
    D: int
    Hi: int
    Di: int
    top_k: int
    sigma: float
    seed: int
    image_runs: bool = False

    @property
    def T(self) -> int:
        return sum(self.seg_lens)

    @property
    def cu(self) -> List[int]:
        out = [0]
        for L in self.seg_lens:
            out.append(out[-1] + L)
        return out

    @property
    def max_seqlen(self) -> int:
        return max(self.seg_lens)

    def pair_counts(self) -> Tuple[int, int]:
        """(P, S): causal pairs and selected pairs."""
        P = S = 0
        for L in self.seg_lens:
            P += L * (L + 1) // 2
            d = min(L, self.top_k)
            S += d * (d + 1) // 2 + max(0, L - self.top_k) * self.top_k
        return P, S

    def executed_pairs(self, crossover: int = 24) -> Tuple[int, int]:
        """(query side, key side): the (query, key) pairs the tile kernels put through the matrix cores.  They walk
        whole tiles with the selection as a mask, so every causal pair of a visited tile is computed: on the query side
        (forward, dQ) the causal pairs of the rows below the tile/gather split (positions < top_k * crossover, rounded up
        to 256), on the key side (dK/dV) every causal pair."""
        split = (self.top_k * crossover + 255) // 256 * 256
        q_side = sum(min(L, split) * (min(L, split) + 1) // 2 for L in self.seg_lens)
        return q_side, self.pair_counts()[0]

    def work(self) -> Dict[str, float]:
        """Algorithmic flop / byte counts per fwd+bwd pass (bf16 element = 2 bytes)."""
        P, S = self.pair_counts()
        e = 2 if self.dtype == torch.bfloat16 else 4
        T, Hq, Hkv, D, Hi, Di, K = self.T, self.Hq, self.Hkv, self.D, self.Hi, self.Di, self.top_k
        F1 = P * (2 * Hi * Di + 2 * Hi)
        B2 = 4 * T * K
        F3 = 4 * Hq * D * S
        B3g = S * Hkv * 2 * D * e
        B3 = B3g + T * 2 * Hq * D * e
        F4 = 10 * Hq * D * S
        B4 = 2 * B3g + T * (3 * Hq + 2 * Hkv) * D * e + 8 * S
        return dict(P=P, S=S, F1=F1, B2=B2, F3=F3, B3_gather=B3g, B3=B3, F4=F4, B4=B4)


C1 = Workload("C1-toy", torch.float32, (256, 512, 384, 896), 8, 2, 64, 4, 32, 128, 1.0, 1)
C2 = Workload("C2-qwen3vl-2b", torch.bfloat16, (1799, 914, 680, 970, 1148, 1763, 918),
              16, 8, 128, 32, 64, 1024, 0.5, 2)
C3 = Workload("C3-qwen3vl-8b-32k", torch.bfloat16, (6144, 2048, 5120, 3072, 4096, 7168, 1024, 4096),
              32, 8, 128, 64, 128, 2048, 0.5, 3, image_runs=True)
C4 = Workload("C4-long-131k", torch.bfloat16, (131072,), 32, 8, 128, 64, 128, 2048, 0.5, 4)
C5 = Workload("C5-qwen3.5-short-segments", torch.bfloat16,
              (716, 65, 73, 107, 133, 129, 75, 135, 512, 1379, 214, 227, 270, 675, 972, 1669, 234, 740,
               208, 1112, 141, 1309, 367, 789, 407, 190, 354, 76, 74, 400, 333, 1147, 1152),
              16, 2, 256, 32, 128, 512, 0.5, 5)

WORKLOADS = {w.name.split("-")[0]: w for w in (C1, C2, C3, C4, C5)}


def scaled(w: Workload, seg_lens, top_k=None, name=None) -> Workload:
    """Same head geometry on other segment lengths (parity tests at sizes the CPU finishes)."""
    return Workload(name or (w.name + "-scaled"), w.dtype, tuple(seg_lens), w.Hq, w.Hkv, w.D, w.Hi, w.Di,
                    top_k if top_k is not None else w.top_k, w.sigma, w.seed, w.image_runs)


def head_shard(w: Workload, ways: int) -> Workload:
    """One GPU's share when the attention heads are split ``ways`` ways, as the reference's tensor parallelism does
    (``train/infra.py:385-469``: q/k/v projections column-parallel, so the operator sees Hq/ways and Hkv/ways heads of
    the same packed rows).  The indexer is left whole: its selection is shared by all heads."""
    if ways < 1 or w.Hq % ways or (w.Hkv % ways and ways % w.Hkv):
        raise ValueError(f"cannot split {w.Hq}/{w.Hkv} heads {ways} ways")
    hkv = max(w.Hkv // ways, 1)                         # kv heads are replicated once there are fewer than ranks
    return Workload(f"{w.name}-heads/{ways}", w.dtype, w.seg_lens, w.Hq // ways, hkv, w.D, w.Hi, w.Di, w.top_k, w.sigma, w.seed,
                    w.image_runs)


def make_inputs(w: Workload, device="cpu", with_dout: bool = True):
    """Returns dict(q,k,v,q_idx,k_idx,w_idx,dout,cu_seqlens,max_seqlen) on ``device``."""
    g = torch.Generator(device="cpu").manual_seed(w.seed)
    T = w.T

    def normal(*shape, sigma):
        return torch.randn(*shape, generator=g, dtype=torch.float32) * sigma

    t = dict(
        q=normal(T, w.Hq, w.D, sigma=w.sigma),
        k=normal(T, w.Hkv, w.D, sigma=w.sigma),
        v=normal(T, w.Hkv, w.D, sigma=w.sigma),
        q_idx=normal(T, w.Hi, w.Di, sigma=w.sigma),
        k_idx=normal(T, w.Di, sigma=w.sigma),
        w_idx=normal(T, w.Hi, sigma=w.sigma),
    )
    if w.image_runs:
        # image-patch runs: rows share one mean vector per run -> clustered top-k
        a = 0
        for L in w.seg_lens:
            runs = []
            if L >= 2048:
                runs.append((16, 16 + 1024))
            if L >= 4096:
                runs.append((2048, 3072))
            for r0, r1 in runs:
                for name in ("q", "k", "v", "q_idx", "k_idx", "w_idx"):
                    x = t[name]
                    m = torch.randn(*x.shape[1:], generator=g, dtype=torch.float32)
                    x[a + r0:a + r1] = x[a + r0:a + r1] + 0.5 * m
            a += L
    if with_dout:
        t["dout"] = normal(T, w.Hq, w.D, sigma=1.0)
    out = {name: x.to(w.dtype).to(device) for name, x in t.items()}
    out["cu_seqlens"] = torch.tensor(w.cu, dtype=torch.int32, device=device)
    out["max_seqlen"] = w.max_seqlen
    return out


def pack_lengths(sample_lengths, max_length: int, device="cpu"):
    """``cu_seqlens`` of one packed row as the reference's collate step builds it
    (train/energon_dataloader.py:431-464, ``PackedBatchEncoder.pack_selected_samples``): the samples back
    to back, then - if they do not fill ``max_length`` - the padding as one more segment, so that the
    last entry is always ``max_length``."""
    total = int(sum(sample_lengths))
    if total > max_length:
        raise ValueError(f"samples ({total} tokens) do not fit max_length={max_length}")
    cu = [0]
    for n in sample_lengths:
        cu.append(cu[-1] + int(n))
    if total < max_length:
        cu.append(max_length)
    return torch.tensor(cu, dtype=torch.int32, device=device)


def random_packed_workload(w: Workload, max_length: int, seed: int, mean_len: int = 1500, name=None) -> Workload:
    """A packed row of ``max_length`` tokens filled greedily with log-normal sample lengths (the mix the
    reference's packer sees: many short captions, a few long documents), padding tail included as the
    last segment.  Deterministic in ``seed``; same head geometry as ``w``."""
    g = torch.Generator().manual_seed(seed)
    lens, total = [], 0
    while True:
        n = int(torch.empty(1).log_normal_(mean=0.0, std=0.9, generator=g).item() * mean_len * 0.67) + 16
        if total + n > max_length - 64:
            break
        lens.append(n)
        total += n
    cu = pack_lengths(lens, max_length).tolist()
    segs = tuple(b - a for a, b in zip(cu[:-1], cu[1:]))
    return scaled(w, segs, name=name or f"{w.name}-packed{seed}")
