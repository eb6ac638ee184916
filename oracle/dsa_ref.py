"""CPU oracle for the packed-sequence DSA attention operator.  TEST INFRASTRUCTURE ONLY.

This module is the checker: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it.  The product package never does.

It restates, in plain fp32 torch on the CPU, the operator the reference reaches at

* ``train/model_attention.py:97-143``   (``varlen_attention_forward``: layout adapter +
  causal varlen attention, default scale ``D**-0.5``),
* ``models/qwen3_vl/model.py:25-46``    (``dispatch_varlen_attention``),
* ``models/qwen3_5/model.py:90-98``     (``SelfAttention._run_varlen_attn``),
* ``models/qwen3/model.py:125-129,149-171`` (``repeat_kv`` + causal SDPA: q head ``h`` reads
  kv head ``h // (Hq // Hkv)``; the only CPU-runnable attention in the reference),

and the four DSA stages the reference does not contain (lightning-indexer score, per-query
top-k with lowest-index ties, sparse softmax attention over the selected keys, its gradients).

Pinning status (what independent check fixes each function; see tests/test_oracle.py):

* ``dense_varlen_causal``    - library routine ``F.scaled_dot_product_attention(is_causal=True)``
  per segment + a pure-Python triple loop on tiny inputs.
* ``indexer_scores_segment`` - pure-Python loop, numpy einsum, special case Hi=1, w=1.
* ``topk_select_segment``    - pure-Python ``sorted`` with key (-score, index) on small rows and
  adversarial tie patterns (all equal, +-0.0, duplicates straddling the K-th place).
* ``sparse_attention``       - pure-Python loop over selected keys; with K >= longest segment it
  must equal ``dense_varlen_causal``; gradients by ``torch.autograd.gradcheck`` in fp64.
* ``selected_scores``        - a gather of the pinned ``indexer_scores_segment``; checked entry by entry in Python.
* ``indexer_kl``             - ``torch.nn.functional.kl_div`` (library routine) on rows without padding, and
  ``softmax - mass`` for its gradient.
* ``sparse_attention_key_rows`` - autograd of ``sparse_attention`` (dk, dv of every key row of a small packed batch).
* ``attention_mass``         - pure-Python loop on a tiny case; rows sum to one; with one kv head the
  mass-weighted sum of the selected value rows equals the head mean of ``sparse_attention``'s output.

The reference holds no golden vector for this path (its tests compare whole-model logits with
HuggingFace weights that are not in the tree), so the torch==2.11 ``varlen_attn`` boundary itself
is "parity unpinned": the anchor is the closed form ``softmax(QK^T/sqrt(D) + causal) V`` per segment.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F


# ----------------------------------------------------------------------------------------------
# cu_seqlens helpers (convention of the reference's producers: models/qwen3_vl/model.py:757-765,
# data/energon_dataloader.py:431-464 - int32 prefix sums, cu[0]=0, cu[-1]=T, pad tail = one more
# segment, zero-length segments allowed)
# ----------------------------------------------------------------------------------------------
def segments(cu_seqlens) -> List[Tuple[int, int]]:
    cu = [int(x) for x in (cu_seqlens.tolist() if hasattr(cu_seqlens, "tolist") else cu_seqlens)]
    if len(cu) < 2 or cu[0] != 0:
        raise ValueError("cu_seqlens must start at 0 and hold at least two entries")
    out = []
    for a, b in zip(cu[:-1], cu[1:]):
        if b < a:
            raise ValueError("cu_seqlens must be non-decreasing")
        out.append((a, b))
    return out


def check_packed(q, k, v, cu_seqlens):
    T, Hq, D = q.shape
    if k.shape != v.shape or k.shape[0] != T or k.shape[2] != D:
        raise ValueError("q/k/v shapes disagree")
    if Hq % k.shape[1] != 0:
        raise ValueError("Hq must be a multiple of Hkv")
    segs = segments(cu_seqlens)
    if segs[-1][1] != T:
        raise ValueError("cu_seqlens[-1] must equal the number of packed tokens")
    return segs


# ----------------------------------------------------------------------------------------------
# Dense reference semantics (what the reference computes today)
# ----------------------------------------------------------------------------------------------
def dense_varlen_causal(q, k, v, cu_seqlens, softmax_scale: Optional[float] = None, causal: bool = True):
    """softmax(Q K^T * scale + causal-within-segment) V with GQA by kv-head expansion.

    Follows models/qwen3/model.py:125-129 (``repeat_kv``: ``h -> h // n_rep``) and :166-169
    (``F.scaled_dot_product_attention(is_causal=True)``), applied per packed segment the way
    ``varlen_attn(cu_seq_q=cu, cu_seq_k=cu, window_size=(-1, 0))`` does
    (train/model_attention.py:123-132).  q (T,Hq,D), k/v (T,Hkv,D) -> (T,Hq,D), fp32 math.
    """
    segs = check_packed(q, k, v, cu_seqlens)
    T, Hq, D = q.shape
    G = Hq // k.shape[1]
    qf, kf, vf = q.float(), k.float(), v.float()
    out = torch.zeros_like(qf)
    for a, b in segs:
        if b == a:
            continue
        qs = qf[a:b].transpose(0, 1).unsqueeze(0)                       # (1,Hq,L,D)
        ks = kf[a:b].repeat_interleave(G, dim=1).transpose(0, 1).unsqueeze(0)
        vs = vf[a:b].repeat_interleave(G, dim=1).transpose(0, 1).unsqueeze(0)
        o = F.scaled_dot_product_attention(qs, ks, vs, is_causal=causal, scale=softmax_scale)
        out[a:b] = o[0].transpose(0, 1)
    return out


# ----------------------------------------------------------------------------------------------
# D1: lightning-indexer score
# ----------------------------------------------------------------------------------------------
def default_index_scale(Hi: int, Di: int) -> float:
    return (Di ** -0.5) * (Hi ** -0.5)


def indexer_scores_segment(q_idx, k_idx, w, scale: Optional[float] = None):
    """I[t,s] = scale * sum_j w[t,j] * relu(q_idx[t,j,:] . k_idx[s,:]) for s <= t, -inf above.

    One segment: q_idx (L,Hi,Di), k_idx (L,Di), w (L,Hi) -> (L,L) fp32.  The head loop keeps the
    accumulation order fixed (j ascending), all in fp32.
    """
    L, Hi, Di = q_idx.shape
    if scale is None:
        scale = default_index_scale(Hi, Di)
    qf, kf, wf = q_idx.float(), k_idx.float(), w.float()
    acc = torch.zeros(L, L, dtype=torch.float32)
    for j in range(Hi):
        acc += wf[:, j:j + 1] * torch.relu(qf[:, j, :] @ kf.t())
    acc *= scale
    above = torch.triu(torch.ones(L, L, dtype=torch.bool), diagonal=1)
    return acc.masked_fill_(above, float("-inf"))


# ----------------------------------------------------------------------------------------------
# D2: per-query top-k, total order (score descending, index ascending)
# ----------------------------------------------------------------------------------------------
def topk_select_segment(scores, top_k: int, base: int = 0):
    """scores (L,L) with row t valid on columns [0,t].  Returns (idx (L,K) int32, n (L,) int32).

    Row t keeps the ``n_t = min(K, t+1)`` valid columns that come first under (score descending,
    column ascending); written as ``base + column`` in ascending order, padded with -1.
    ``-0.0`` and ``+0.0`` compare equal (the column decides).  NaN is an error.
    A stable descending sort keeps the lower column first among equal scores, which
    ``torch.topk`` does not promise.
    """
    if top_k < 1:
        raise ValueError("top_k must be >= 1")
    L = scores.shape[0]
    K = top_k
    cols = torch.arange(L)
    valid = cols[None, :] <= cols[:, None]
    if torch.isnan(scores[valid]).any():
        raise ValueError("NaN in indexer scores")
    idx = torch.full((L, K), -1, dtype=torch.int32)
    n = torch.minimum(torch.arange(1, L + 1), torch.tensor(K)).to(torch.int32)
    dense_rows = min(L, K)
    if dense_rows > 0:
        tri = torch.arange(K)[None, :].expand(dense_rows, -1)
        keep = tri <= cols[:dense_rows, None]
        idx[:dense_rows] = torch.where(keep, tri + base, torch.tensor(-1)).to(torch.int32)
    if L > K:
        s = scores[K:].masked_fill(~valid[K:], float("-inf"))
        order = torch.sort(s, dim=1, descending=True, stable=True).indices[:, :K]
        idx[K:] = (torch.sort(order, dim=1).values + base).to(torch.int32)
    return idx, n


def topk_from_score_rows(rows: Sequence[torch.Tensor], top_k: int) -> List[List[int]]:
    """Ragged helper: each row is a 1-D fp32 tensor of valid scores; returns the ascending list of
    kept columns per row (same order rule as ``topk_select_segment``)."""
    out = []
    for r in rows:
        n = r.numel()
        if n <= top_k:
            out.append(list(range(n)))
            continue
        if torch.isnan(r).any():
            raise ValueError("NaN in indexer scores")
        order = torch.sort(r, descending=True, stable=True).indices[:top_k]
        out.append(sorted(order.tolist()))
    return out


def dsa_select(q_idx, k_idx, w, cu_seqlens, top_k: int, index_scale: Optional[float] = None):
    """Stages D1+D2 over a packed batch -> (idx (T,K) int32 global row ids, n (T,) int32)."""
    segs = segments(cu_seqlens)
    T = q_idx.shape[0]
    idx = torch.full((T, top_k), -1, dtype=torch.int32)
    n = torch.zeros(T, dtype=torch.int32)
    for a, b in segs:
        if b == a:
            continue
        if b - a <= top_k:      # every row is dense: scores cannot change the answer
            sc = torch.zeros(b - a, b - a)
        else:
            sc = indexer_scores_segment(q_idx[a:b], k_idx[a:b], w[a:b], index_scale)
        i_s, n_s = topk_select_segment(sc, top_k, base=a)
        idx[a:b], n[a:b] = i_s, n_s
    return idx, n


# ----------------------------------------------------------------------------------------------
# D3 (+ D4 through autograd): sparse attention over the selected keys
# ----------------------------------------------------------------------------------------------
def sparse_attention(q, k, v, idx, n, cu_seqlens, softmax_scale: Optional[float] = None,
                     chunk: int = 1024, return_lse: bool = False):
    """O[t,h] = sum_{s in sel(t)} softmax_s(q[t,h].k[s,h//G] * scale) v[s,h//G].

    ``idx`` (T,K) holds global packed row ids (ascending, -1 padded), ``n`` (T,) the counts.
    Built as masked dense attention per segment (boolean mask scattered from ``idx``), in fp32,
    from differentiable torch ops so that ``torch.autograd`` yields the D4 gradients.
    """
    segs = check_packed(q, k, v, cu_seqlens)
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    scale = softmax_scale if softmax_scale is not None else D ** -0.5
    cdt = torch.float64 if q.dtype == torch.float64 else torch.float32
    qf, kf, vf = q.to(cdt), k.to(cdt), v.to(cdt)
    outs, lses = [], []
    for a, b in segs:
        L = b - a
        if L == 0:
            continue
        ks = kf[a:b].repeat_interleave(G, dim=1).permute(1, 2, 0)       # (Hq,D,L)
        vs = vf[a:b].repeat_interleave(G, dim=1).permute(1, 0, 2)       # (Hq,L,D)
        for c0 in range(a, b, chunk):
            c1 = min(b, c0 + chunk)
            R = c1 - c0
            loc = idx[c0:c1].long() - a
            ok = idx[c0:c1] >= 0
            mask = torch.zeros(R, L + 1, dtype=torch.bool)
            mask.scatter_(1, torch.where(ok, loc, torch.tensor(L)), True)
            mask = mask[:, :L]
            logits = torch.matmul(qf[c0:c1].permute(1, 0, 2), ks) * scale      # (Hq,R,L)
            logits = logits.masked_fill(~mask[None], float("-inf"))
            lse = torch.logsumexp(logits, dim=-1)                                # (Hq,R)
            p = torch.exp(logits - lse[..., None])
            outs.append(torch.matmul(p, vs).permute(1, 0, 2))                    # (R,Hq,D)
            lses.append(lse)
    out = torch.cat(outs, dim=0) if outs else qf.new_zeros(0, Hq, D)
    if return_lse:
        return out, (torch.cat(lses, dim=1) if lses else qf.new_zeros(Hq, 0))
    return out


def attention_mass(q, k, idx, n, cu_seqlens, softmax_scale: Optional[float] = None, chunk: int = 256):
    """Target distribution of the indexer's training loss: the attention probability of every selected key,
    averaged over the query heads,

        mass[t,j] = 1/Hq * sum_h softmax_{s in sel(t)}(q[t,h].k[s,h//G] * scale) at s = idx[t,j]   (0 where idx = -1).

    Every head's softmax over sel(t) sums to one, so a row sums to one: the head sum needs no further
    normalisation.  Written as a gather over ``idx`` (not as the masked dense product ``sparse_attention``
    uses), so that the two restatements check each other: with one kv head,
    ``sum_j mass[t,j] v[idx[t,j]]`` is the head mean of the attention output.
    """
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    scale = softmax_scale if softmax_scale is not None else D ** -0.5
    cdt = torch.float64 if q.dtype == torch.float64 else torch.float32
    qf, kf = q.to(cdt), k.to(cdt)
    K = idx.shape[1]
    mass = torch.zeros(T, K, dtype=cdt)
    for c0 in range(0, T, chunk):
        c1 = min(T, c0 + chunk)
        ok = idx[c0:c1] >= 0                                                    # (R,K)
        rows = kf[idx[c0:c1].clamp(min=0).long()]                               # (R,K,Hkv,D)
        rows = rows.repeat_interleave(G, dim=2)                                 # (R,K,Hq,D): head h reads kv head h//G
        logits = torch.einsum("rhd,rkhd->rhk", qf[c0:c1], rows) * scale
        logits = logits.masked_fill(~ok[:, None, :], float("-inf"))
        p = torch.softmax(logits, dim=-1)
        p = torch.where(ok[:, None, :], p, torch.zeros((), dtype=cdt))          # rows without any key stay zero
        mass[c0:c1] = p.mean(dim=1)
    return mass


def sparse_attention_rows(q, k, v, idx, n, rows, softmax_scale: Optional[float] = None):
    """``sparse_attention`` for the query rows ``rows`` only -> (len(rows), Hq, D).

    Written as a gather (the selected key rows of a query are fetched and attended densely), not as the masked dense
    product of ``sparse_attention``: the two restatements check each other, and this one costs n[t] keys per row
    whatever the segment length, so single rows of a very long sequence can be checked.  Differentiable in q, k, v.
    """
    T, Hq, D = q.shape
    G = Hq // k.shape[1]
    scale = softmax_scale if softmax_scale is not None else D ** -0.5
    cdt = torch.float64 if q.dtype == torch.float64 else torch.float32
    outs = []
    for r in rows:
        sel = idx[r, : int(n[r])].long()
        ks = k[sel].to(cdt).repeat_interleave(G, dim=1)                         # (n,Hq,D): head h reads kv head h//G
        vs = v[sel].to(cdt).repeat_interleave(G, dim=1)
        logits = torch.einsum("hd,nhd->hn", q[r].to(cdt), ks) * scale
        p = torch.softmax(logits, dim=-1)
        outs.append(torch.einsum("hn,nhd->hd", p, vs))
    return torch.stack(outs) if outs else q.new_zeros(0, Hq, D, dtype=cdt)


def selected_scores(q_idx, k_idx, w, idx, n, cu_seqlens, index_scale: Optional[float] = None):
    """Indexer scores of the selected keys: sel[t,j] = score(t, idx[t,j]) (0 where idx = -1), fp32."""
    T, K = idx.shape
    sel = torch.zeros(T, K, dtype=torch.float32)
    for a, b in segments(cu_seqlens):
        if b == a:
            continue
        sc = indexer_scores_segment(q_idx[a:b], k_idx[a:b], w[a:b], index_scale)     # (L,L), row t, column s - a
        loc = (idx[a:b].long() - a).clamp(min=0)
        sel[a:b] = torch.where(idx[a:b] >= 0, torch.gather(sc.float(), 1, loc), torch.zeros(()))
    return sel


def indexer_kl(sel, mass, n):
    """loss[t] = KL(mass[t,:n[t]] || softmax(sel[t,:n[t]])) with 0 log 0 = 0, built from differentiable torch ops
    (``sel`` may require grad: autograd then gives softmax - mass per row)."""
    T, K = sel.shape
    ok = torch.arange(K)[None, :] < n[:, None]
    logq = torch.log_softmax(sel.masked_fill(~ok, float("-inf")), dim=-1)
    logq = torch.where(ok, logq, torch.zeros((), dtype=sel.dtype))
    p = torch.where(ok, mass.to(sel.dtype), torch.zeros((), dtype=sel.dtype))
    terms = torch.where(p > 0, p * (torch.log(p.clamp(min=1e-45)) - logq), torch.zeros((), dtype=sel.dtype))
    return terms.sum(-1)


def dsa_varlen_attn_ref(q, k, v, cu_seqlens, q_idx, k_idx, w, top_k: int,
                        softmax_scale: Optional[float] = None, index_scale: Optional[float] = None,
                        return_indices: bool = False):
    """Whole operator: D1 -> D2 -> D3 (fp32).  Indexer inputs get no gradient."""
    with torch.no_grad():
        idx, n = dsa_select(q_idx, k_idx, w, cu_seqlens, top_k, index_scale)
    out = sparse_attention(q, k, v, idx, n, cu_seqlens, softmax_scale)
    return (out, idx, n) if return_indices else out


def sparse_attention_grads(q, k, v, idx, n, cu_seqlens, dout, softmax_scale: Optional[float] = None):
    """(out, dq, dk, dv) in fp32 through autograd of ``sparse_attention``."""
    qf = q.detach().float().requires_grad_(True)
    kf = k.detach().float().requires_grad_(True)
    vf = v.detach().float().requires_grad_(True)
    out = sparse_attention(qf, kf, vf, idx, n, cu_seqlens, softmax_scale)
    dq, dk, dv = torch.autograd.grad(out, (qf, kf, vf), dout.float())
    return out.detach(), dq, dk, dv


def sparse_attention_key_rows(q, k, v, dout, idx, n, keys, softmax_scale: Optional[float] = None, batch: int = 32):
    """dK and dV of the key rows ``keys`` only -> (dk (len(keys),Hkv,D), dv (len(keys),Hkv,D)), fp32.

    Key-stationary restatement of the D4 gradients, written from the formulas and not through autograd: the queries
    that selected key ``s`` are looked up in ``idx``; each of them is attended over its own selected keys (a gather, as
    in ``sparse_attention_rows``) for its softmax and for ``delta = sum_j p_j dP_j``; then
        dV[s] = sum_t sum_h p[t,h,s] dO[t,h]          dK[s] = scale * sum_t sum_h p[t,h,s] (dP[t,h,s] - delta[t,h]) q[t,h]
    over the heads ``h`` of the key's kv head.  Costs n[t] keys per contributing query whatever the segment length, so
    single key rows of a very long sequence can be checked.  Pinned against autograd of ``sparse_attention``.
    """
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    scale = softmax_scale if softmax_scale is not None else D ** -0.5
    keys = [int(s) for s in keys]
    key_t = torch.tensor(keys, dtype=idx.dtype)
    hit = torch.zeros(T, dtype=torch.bool)
    for c0 in range(0, T, 8192):                                        # which queries selected any of the keys
        hit[c0:c0 + 8192] = torch.isin(idx[c0:c0 + 8192], key_t).any(dim=1)
    rows = torch.nonzero(hit).flatten()
    dk = torch.zeros(len(keys), Hkv, D)
    dv = torch.zeros(len(keys), Hkv, D)
    kh, vh = k.transpose(0, 1).contiguous(), v.transpose(0, 1).contiguous()        # (Hkv,T,D): one gather per kv head
    for b0 in range(0, rows.numel(), batch):
        r = rows[b0:b0 + batch]
        R = r.numel()
        sel = idx[r].long()                                             # (R,K), -1 padded
        ok = sel >= 0
        safe = sel.clamp(min=0).flatten()
        qr = q[r].float().view(R, Hkv, G, D)
        gr = dout[r].float().view(R, Hkv, G, D)
        at = sel[:, :, None] == torch.tensor(keys)[None, None, :]       # (R,K,len(keys)): at most one slot per (row, key)
        has = at.any(dim=1)                                             # (R,len(keys))
        slot = at.float().argmax(dim=1)                                 # (R,len(keys)): the slot, 0 where absent
        for h in range(Hkv):
            kg = kh[h][safe].float().view(R, -1, D)                     # (R,K,D)
            vg = vh[h][safe].float().view(R, -1, D)
            logits = torch.bmm(qr[:, h], kg.transpose(1, 2)) * scale    # (R,G,K)
            logits = logits.masked_fill(~ok[:, None, :], float("-inf"))
            p = torch.softmax(logits, dim=-1)
            dP = torch.bmm(gr[:, h], vg.transpose(1, 2))
            delta = (p * dP).sum(-1, keepdim=True)
            dS = p * (dP - delta)
            pick = slot[:, None, :].expand(R, G, len(keys))
            w_p = p.gather(2, pick) * has[:, None, :]                   # (R,G,len(keys)): p[t,h,s], 0 where t did not select s
            w_s = dS.gather(2, pick) * has[:, None, :]
            dv[:, h] += torch.einsum("rgj,rgd->jd", w_p, gr[:, h])
            dk[:, h] += torch.einsum("rgj,rgd->jd", w_s, qr[:, h]) * scale
    return dk, dv


# ----------------------------------------------------------------------------------------------
# Layout adapter of the HF-style entry (train/model_attention.py:110-118,141)
# ----------------------------------------------------------------------------------------------
def hf_layout_to_packed(x):
    """(1,H,T,D) -> (T,H,D) contiguous, as model_attention.py:110-117 does."""
    x = x.transpose(1, 2).contiguous()
    return x.view(-1, x.size(-2), x.size(-1))


# ----------------------------------------------------------------------------------------------
# Work accounting used by bench.py and the docs
# ----------------------------------------------------------------------------------------------
def pair_counts(cu_seqlens, top_k: int) -> Tuple[int, int]:
    """(P, S): causal pairs and selected pairs of a packed batch."""
    P = S = 0
    for a, b in segments(cu_seqlens):
        L = b - a
        P += L * (L + 1) // 2
        d = min(L, top_k)
        S += d * (d + 1) // 2 + max(0, L - top_k) * top_k
    return P, S
