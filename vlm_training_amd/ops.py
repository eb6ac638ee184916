"""Host side of the DSA packed-attention operator: torch tensors in, HIP kernels through the C ABI.

``dsa_varlen_attn`` is the operator (a ``torch.autograd.Function`` underneath).  With no indexer
inputs it is dense causal varlen attention, i.e. what the reference gets from
``varlen_attn(q, k, v, cu_seq_q=cu, cu_seq_k=cu, max_q=m, max_k=m, window_size=(-1, 0))``
(train/model_attention.py:123-132, models/qwen3_vl/model.py:41-46, models/qwen3_5/model.py:93-98).
torch is used for device memory and streams only; all arithmetic runs in the HIP library.
"""
from __future__ import annotations

import os

from typing import Optional, Tuple

import torch

from . import _lib


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("dsa attention runs on the GPU only (tensor on %s); there is no CPU path" % t.device)


def _as_bf16(t: torch.Tensor) -> torch.Tensor:
    # fp32/fp16 inputs are rounded to bf16 once; the kernels compute in bf16 MFMA with fp32 accumulation
    return (t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16)).contiguous()


def _as_bf16_x3(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor):
    """Three tensors to bf16; three fp32 ones by one launch instead of three casts."""
    if not (a.dtype == b.dtype == c.dtype == torch.float32) or not (a.is_cuda and a.numel()):
        return _as_bf16(a), _as_bf16(b), _as_bf16(c)
    a, b, c = a.contiguous(), b.contiguous(), c.contiguous()
    if (a.data_ptr() | b.data_ptr() | c.data_ptr()) & 15:
        return _as_bf16(a), _as_bf16(b), _as_bf16(c)
    # one buffer, each part on a 16-byte boundary
    offs, total = [], 0
    for t in (a, b, c):
        offs.append(total)
        total += (t.numel() + 7) // 8 * 8
    buf = torch.empty((total,), dtype=torch.bfloat16, device=a.device)
    ys = [buf[o:o + t.numel()].view(t.shape) for o, t in zip(offs, (a, b, c))]
    rc = _lib.load().dsa_round_bf16_x3(_ptr(a), _ptr(b), _ptr(c), a.numel(), b.numel(), c.numel(), _ptr(ys[0]), _ptr(ys[1]),
                                       _ptr(ys[2]), _stream(a.device))
    _lib.check(rc, "dsa_round_bf16_x3")
    return ys[0], ys[1], ys[2]


def _check_cu(cu_seqlens: torch.Tensor, T: int, max_seqlen: Optional[int] = None):
    if cu_seqlens.dim() != 1 or cu_seqlens.numel() < 2:
        raise ValueError("cu_seqlens must be 1-D with at least two entries")
    if cu_seqlens.dtype != torch.int32:
        cu_seqlens = cu_seqlens.to(torch.int32)
    if os.environ.get("DSA_DEBUG_META"):
        # The kernels trust the segment offsets (they hold every index to its buffer, so a bad table gives a wrong
        # result, not a fault).  With this switch the table is copied to the host and checked - one stall per call,
        # which is why it is not the default.
        cu = cu_seqlens.tolist()
        if cu[0] != 0 or cu[-1] != T:
            raise ValueError(f"cu_seqlens must start at 0 and end at T={T}, got [{cu[0]} ... {cu[-1]}]")
        if any(b < a for a, b in zip(cu[:-1], cu[1:])):
            raise ValueError("cu_seqlens must be non-decreasing")
        longest = max(b - a for a, b in zip(cu[:-1], cu[1:]))
        if max_seqlen is not None and longest > max_seqlen:
            raise ValueError(f"max_seqlen={max_seqlen} is below the longest segment ({longest})")
    return cu_seqlens.contiguous()


_KERNEL_HEAD_DIMS = (64, 128, 256)                   # head_dim instantiations of the tile and gather kernels
_KERNEL_HEAD_DIMS_DENSE = (64, 96, 128, 256)         # without a key selection the tile kernels also come at head_dim 96


def _check_qkv(q, k, v):
    if q.dim() != 3 or k.dim() != 3 or v.dim() != 3:
        raise ValueError("q, k, v must be (T, H, D)")
    T, Hq, D = q.shape
    if k.shape != v.shape or k.shape[0] != T or k.shape[2] != D:
        raise ValueError(f"q/k/v shapes disagree: {tuple(q.shape)} {tuple(k.shape)} {tuple(v.shape)}")
    Hkv = k.shape[1]
    if Hq % Hkv:
        raise ValueError(f"Hq={Hq} must be a multiple of Hkv={Hkv}")
    if q.dtype != k.dtype or q.dtype != v.dtype:
        raise ValueError("q, k, v must share a dtype")
    return T, Hq, Hkv, D


# ------------------------------------------------------------------------------------------------
# stage wrappers (also used by the tests to look at each stage on its own)
# ------------------------------------------------------------------------------------------------
def indexer_scores(q_idx, k_idx, w_idx, cu_seqlens, max_seqlen: int, index_scale: Optional[float] = None,
                   skip_dense_k: int = 0) -> torch.Tensor:
    """Stage D1 for every row: (T, ld) fp32, row t valid on columns [0, pos(t)] (key = seg_start + column)."""
    _require_cuda(q_idx, k_idx, w_idx, cu_seqlens)
    T, Hi, Di = q_idx.shape
    cu = _check_cu(cu_seqlens, T)
    scale = index_scale if index_scale is not None else (Di ** -0.5) * (Hi ** -0.5)
    ld = (max_seqlen + 31) // 32 * 32
    scores = torch.full((T, ld), float("-inf"), dtype=torch.float32, device=q_idx.device)
    lib = _lib.load()
    qi, ki, wi = _as_bf16_x3(q_idx, k_idx, w_idx)                      # keep the casts alive over the launch
    rc = lib.dsa_indexer_scores(_ptr(qi), _ptr(ki), _ptr(wi), _ptr(cu), T,
                                cu.numel() - 1, Hi, Di, scale, _lib.DSA_DTYPE_BF16, 0, T, skip_dense_k, _ptr(scores), ld,
                                _stream(q_idx.device))
    _lib.check(rc, "dsa_indexer_scores")
    return scores


def topk_from_scores(scores: torch.Tensor, cu_seqlens, top_k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Stage D2 on materialised scores (T, ld): returns (idx (T,K) int32, n (T,) int32)."""
    _require_cuda(scores, cu_seqlens)
    if scores.dtype != torch.float32 or scores.dim() != 2 or not scores.is_contiguous():
        raise ValueError("scores must be a contiguous (T, ld) fp32 tensor")
    T, ld = scores.shape
    cu = _check_cu(cu_seqlens, T)
    idx = torch.empty((T, top_k), dtype=torch.int32, device=scores.device)
    n = torch.empty((T,), dtype=torch.int32, device=scores.device)
    lib = _lib.load()
    rc = lib.dsa_topk_from_scores(_ptr(scores), ld, 0, T, _ptr(cu), T, cu.numel() - 1, top_k, _ptr(idx), _ptr(n),
                                  _stream(scores.device))
    _lib.check(rc, "dsa_topk_from_scores")
    return idx, n


def index_topk(q_idx, k_idx, w_idx, cu_seqlens, max_seqlen: int, top_k: int,
               index_scale: Optional[float] = None, return_scores: bool = False, bitmap=None):
    """Stages D1+D2: selected key rows per query, (idx (T,K) int32 ascending/-1 padded, n (T,) int32);
    ``return_scores=True`` adds the (T,K) fp32 indexer scores of the selected keys (0 past n[t]).  ``bitmap`` (uint8, the
    size of the forward's workspace) receives the inverted selection the forward would otherwise build from the list:
    pass it on as ``attn_fwd(..., ws=bitmap, bitmap_ready=True)``."""
    _require_cuda(q_idx, k_idx, w_idx, cu_seqlens)
    if q_idx.dim() != 3 or k_idx.dim() != 2 or w_idx.dim() != 2:
        raise ValueError("indexer tensors must be q_idx (T,Hi,Di), k_idx (T,Di), w_idx (T,Hi)")
    T, Hi, Di = q_idx.shape
    if k_idx.shape != (T, Di) or w_idx.shape != (T, Hi):
        raise ValueError("indexer tensor shapes disagree")
    if top_k < 1:
        raise ValueError("top_k must be >= 1")
    cu = _check_cu(cu_seqlens, T, max_seqlen)
    scale = index_scale if index_scale is not None else (Di ** -0.5) * (Hi ** -0.5)
    lib = _lib.load()
    idx = torch.empty((T, top_k), dtype=torch.int32, device=q_idx.device)
    n = torch.empty((T,), dtype=torch.int32, device=q_idx.device)
    ws_bytes = lib.dsa_index_topk_workspace_bytes(T, max_seqlen, top_k) if (max_seqlen > top_k or return_scores) else 0
    ws = torch.empty((max(ws_bytes, 4),), dtype=torch.uint8, device=q_idx.device)
    qi, ki, wi = _as_bf16_x3(q_idx, k_idx, w_idx)                      # keep the casts alive over the launch
    if os.environ.get("DSA_DEBUG_NAN"):
        # the device ranks NaN above +inf without a word; with this switch (one device-to-host copy) it is an error,
        # as it is in the CPU restatement of the selection
        if not (torch.isfinite(qi.float()).all() and torch.isfinite(ki.float()).all() and torch.isfinite(wi.float()).all()):
            raise ValueError("non-finite indexer inputs: their scores have no defined rank")
    if bitmap is not None:
        sel = torch.empty((T, top_k), dtype=torch.float32, device=q_idx.device) if return_scores else None
        rc = lib.dsa_index_topk_bitmap(_ptr(qi), _ptr(ki), _ptr(wi), _ptr(cu), T, cu.numel() - 1, Hi, Di, top_k, scale,
                                       _lib.DSA_DTYPE_BF16, max_seqlen, _ptr(idx), _ptr(n), _ptr(sel), _ptr(bitmap),
                                       bitmap.numel(), _ptr(ws), ws_bytes, _stream(q_idx.device))
        _lib.check(rc, "dsa_index_topk_bitmap")
        return (idx, n, sel) if return_scores else (idx, n)
    if return_scores:
        sel = torch.empty((T, top_k), dtype=torch.float32, device=q_idx.device)
        rc = lib.dsa_index_topk_scores(_ptr(qi), _ptr(ki), _ptr(wi), _ptr(cu), T, cu.numel() - 1, Hi, Di, top_k, scale,
                                       _lib.DSA_DTYPE_BF16, max_seqlen, _ptr(idx), _ptr(n), _ptr(sel), _ptr(ws), ws_bytes,
                                       _stream(q_idx.device))
        _lib.check(rc, "dsa_index_topk_scores")
        return idx, n, sel
    rc = lib.dsa_index_topk(_ptr(qi), _ptr(ki), _ptr(wi), _ptr(cu), T,
                            cu.numel() - 1, Hi, Di, top_k, scale, _lib.DSA_DTYPE_BF16, max_seqlen, _ptr(idx), _ptr(n),
                            _ptr(ws), ws_bytes, _stream(q_idx.device))
    _lib.check(rc, "dsa_index_topk")
    return idx, n


def indexer_kl(sel_scores, mass, n, grad_scale: Optional[float] = None, want_grad: bool = True):
    """KL(mass || softmax(sel_scores)) per query row over its selected keys -> (loss (T,) fp32, dscore (T,K) fp32 or
    None).  ``dscore`` = d(grad_scale * sum_t loss[t]) / d sel_scores; grad_scale defaults to 1/T (mean loss)."""
    _require_cuda(sel_scores, mass, n)
    T, K = sel_scores.shape
    if mass.shape != (T, K) or n.shape != (T,) or sel_scores.dtype != torch.float32 or mass.dtype != torch.float32:
        raise ValueError("sel_scores and mass must be (T,K) fp32, n (T,) int32")
    gs = float(grad_scale) if grad_scale is not None else 1.0 / max(T, 1)
    loss = torch.empty((T,), dtype=torch.float32, device=mass.device)
    dscore = torch.empty((T, K), dtype=torch.float32, device=mass.device) if want_grad else None
    sc, ms = sel_scores.contiguous(), mass.contiguous()
    rc = _lib.load().dsa_indexer_kl(_ptr(sc), _ptr(ms), _ptr(n), T, K, gs, _ptr(loss), _ptr(dscore), _stream(mass.device))
    _lib.check(rc, "dsa_indexer_kl")
    return loss, dscore


def indexer_bwd(q_idx, k_idx, w_idx, idx, n, dscore, cu_seqlens, max_seqlen: int, index_scale: Optional[float] = None):
    """Gradients of the selected indexer scores: (dq_idx (T,Hi,Di) bf16, dk_idx (T,Di) bf16, dw (T,Hi) fp32) for
    ``dscore`` (T,K) fp32 = dLoss/dScore at the selected keys."""
    _require_cuda(q_idx, k_idx, w_idx, idx, n, dscore, cu_seqlens)
    T, Hi, Di = q_idx.shape
    K = idx.shape[1]
    cu = _check_cu(cu_seqlens, T)
    if dscore.shape != (T, K) or dscore.dtype != torch.float32:
        raise ValueError("dscore must be (T,K) fp32")
    scale = index_scale if index_scale is not None else (Di ** -0.5) * (Hi ** -0.5)
    lib = _lib.load()
    qi, ki, wi = _as_bf16_x3(q_idx, k_idx, w_idx)
    d_kernel = next((d for d in (64, 128) if d >= Di), None)
    if d_kernel is not None and d_kernel != Di:          # e.g. 32-wide index heads: zero columns change no score
        pad = d_kernel - Di
        dq, dk, dw = indexer_bwd(torch.nn.functional.pad(qi, (0, pad)), torch.nn.functional.pad(ki, (0, pad)), wi, idx, n,
                                 dscore, cu_seqlens, max_seqlen, scale)
        return dq[..., :Di].contiguous(), dk[..., :Di].contiguous(), dw
    dq = torch.empty_like(qi)
    dk = torch.empty_like(ki)
    dw = torch.empty((T, Hi), dtype=torch.float32, device=qi.device)
    max_seqlen = T if max_seqlen is None else int(max_seqlen)
    ws_bytes = lib.dsa_indexer_bwd_workspace_bytes(T, Di, max_seqlen)
    ws = torch.empty((max(ws_bytes, 4),), dtype=torch.uint8, device=qi.device)
    rc = lib.dsa_indexer_bwd(_ptr(qi), _ptr(ki), _ptr(wi), _ptr(idx), _ptr(n), _ptr(dscore.contiguous()), _ptr(cu), T,
                             cu.numel() - 1, Hi, Di, K, scale, _lib.DSA_DTYPE_BF16, max_seqlen, _ptr(dq), _ptr(dk), _ptr(dw),
                             _ptr(ws), ws_bytes, _stream(qi.device))
    _lib.check(rc, "dsa_indexer_bwd")
    return dq, dk, dw


class _IndexerKL(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q_idx, k_idx, w_idx, mass, cu_seqlens, max_seqlen, top_k, index_scale, idx=None, n=None, sel=None):
        T = q_idx.shape[0]
        if sel is None:
            idx, n, sel = index_topk(q_idx, k_idx, w_idx, cu_seqlens, max_seqlen, top_k, index_scale, return_scores=True)
        loss_rows, dscore = indexer_kl(sel, mass, n, grad_scale=1.0 / max(T, 1))
        ctx.save_for_backward(q_idx, k_idx, w_idx, idx, n, dscore, cu_seqlens)
        ctx.max_seqlen, ctx.index_scale = max_seqlen, index_scale
        return loss_rows.mean()

    @staticmethod
    def backward(ctx, g):
        q_idx, k_idx, w_idx, idx, n, dscore, cu = ctx.saved_tensors
        # the gradients are linear in dscore: scale the (T,K) table by the incoming gradient, not the three results
        dq, dk, dw = indexer_bwd(q_idx, k_idx, w_idx, idx, n, dscore * g.to(torch.float32), cu, ctx.max_seqlen,
                                 ctx.index_scale)
        return (dq.to(q_idx.dtype), dk.to(k_idx.dtype), dw.to(w_idx.dtype), None, None, None, None, None, None, None, None)


@torch.compiler.disable
def indexer_kl_loss(indexer_q, indexer_k, indexer_w, mass, cu_seqlens, max_seqlen: Optional[int], top_k: int,
                    index_scale: Optional[float] = None, selection=None):
    """Training loss of the DSA indexer: mean over the packed tokens of KL(mass[t] || softmax of the indexer's scores
    over the keys it selected for t), differentiable w.r.t. indexer_q (T,Hi,Di), indexer_k (T,Di), indexer_w (T,Hi).

    ``mass`` is the detached target ``dsa_varlen_attn(..., return_mass=True)`` returned for the same indexer
    inputs and top_k.  ``selection=(idx, n, scores)`` as returned by ``dsa_varlen_attn(..., return_indices=True,
    return_scores=True)`` saves a second run of the indexer; without it the selection is recomputed here (it is
    deterministic, hence the same)."""
    T = indexer_q.shape[0]
    max_seqlen = T if max_seqlen is None else int(max_seqlen)
    idx, n, sel = selection if selection is not None else (None, None, None)
    return _IndexerKL.apply(indexer_q, indexer_k, indexer_w, mass, cu_seqlens, max_seqlen, int(top_k), index_scale, idx, n,
                            sel)


def set_tile_crossover(crossover: int) -> int:
    """Rows with pos < top_k * crossover use the MFMA tile kernels, later rows the gather kernels.
    Returns the previous value (tests use it to drive each path on its own)."""
    lib = _lib.load()
    old = lib.dsa_get_tile_crossover()
    _lib.check(lib.dsa_set_tile_crossover(int(crossover)), "dsa_set_tile_crossover")
    return old


def set_bwd_overlap(mode: int) -> int:
    """0: the backward's passes run one after the other on the caller's stream; 1 (default): launches of few
    workgroups run dQ beside dK/dV on a second stream of the library's own; 2: every launch does.  Same bits in every
    mode.  Returns the previous mode."""
    lib = _lib.load()
    old = lib.dsa_get_bwd_overlap()
    _lib.check(lib.dsa_set_bwd_overlap(int(mode)), "dsa_set_bwd_overlap")
    return old


def attn_fwd(q, k, v, idx, n, cu_seqlens, max_seqlen: int, softmax_scale: float, causal: bool = True, ws=None,
             bitmap_ready: bool = False):
    """Stage D3.  ``ws`` (optional, uint8) is used as the workspace instead of a fresh allocation: the autograd wrapper
    keeps it for the backward, so that the selection bitmap is built once.  ``bitmap_ready``: ``ws`` already holds the
    bitmap of this selection (``index_topk(..., bitmap=ws)``) and is only read."""
    T, Hq, Hkv, D = _check_qkv(q, k, v)
    cu = _check_cu(cu_seqlens, T)
    out = torch.empty((T, Hq, D), dtype=torch.bfloat16, device=q.device)
    lse = torch.empty((Hq, T), dtype=torch.float32, device=q.device)
    K = idx.shape[1] if idx is not None else 0
    lib = _lib.load()
    ws_bytes = lib.dsa_attn_fwd_workspace_bytes(T, max_seqlen, 1 if idx is not None else 0)
    if ws is None:
        ws = torch.empty((max(ws_bytes, 4),), dtype=torch.uint8, device=q.device)
    elif ws.numel() < ws_bytes:
        raise ValueError(f"forward workspace: have {ws.numel()} bytes, need {ws_bytes}")
    if bitmap_ready:
        rc = lib.dsa_attn_fwd_saved_bitmap(_ptr(q), _ptr(k), _ptr(v), _ptr(idx), _ptr(n), _ptr(cu), T, cu.numel() - 1, Hq, Hkv,
                                           D, K, softmax_scale, _lib.DSA_DTYPE_BF16, max_seqlen, 1 if causal else 0, _ptr(out),
                                           _ptr(lse), _ptr(ws), ws_bytes, _stream(q.device))
        _lib.check(rc, "dsa_attn_fwd_saved_bitmap")
        return out, lse
    rc = lib.dsa_attn_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(idx), _ptr(n), _ptr(cu), T, cu.numel() - 1, Hq, Hkv, D, K,
                          softmax_scale, _lib.DSA_DTYPE_BF16, max_seqlen, 1 if causal else 0, _ptr(out), _ptr(lse), _ptr(ws), ws_bytes,
                          _stream(q.device))
    _lib.check(rc, "dsa_attn_fwd")
    return out, lse


def attn_mass(q, k, lse, idx, n, cu_seqlens, max_seqlen: int, softmax_scale: Optional[float] = None,
              bitmap=None) -> torch.Tensor:
    """Head-averaged attention probability of every selected key, (T, K) fp32, rows summing to one: the target
    of the KL loss that trains the indexer.  ``lse`` (Hq, T) is the forward's second output for the same
    q, k, idx.  ``bitmap``: the selection bitmap of this idx/n and max_seqlen, if the caller holds it (the forward's
    workspace), so that none is built here.  Nothing here is differentiable (the target is detached in DSA's
    objective)."""
    _require_cuda(q, k, lse, idx, n, cu_seqlens)
    T, Hq, D = q.shape
    Hkv, K = k.shape[1], idx.shape[1]
    cu = _check_cu(cu_seqlens, T)
    if lse.shape != (Hq, T) or lse.dtype != torch.float32 or idx.shape[0] != T or n.shape != (T,):
        raise ValueError("lse must be (Hq,T) fp32, idx (T,K) int32, n (T,) int32")
    scale = float(softmax_scale) if softmax_scale is not None else D ** -0.5
    max_seqlen = T if max_seqlen is None else int(max_seqlen)
    lib = _lib.load()
    qb, kb = _as_bf16(q), _as_bf16(k)
    mass = torch.empty((T, K), dtype=torch.float32, device=q.device)
    ws_bytes = lib.dsa_attn_mass_workspace_bytes(T, cu.numel() - 1, Hq, Hkv, D, K, max_seqlen)
    if bitmap is not None:
        ws_bytes -= lib.dsa_attn_fwd_workspace_bytes(T, max_seqlen, 1)       # the partial tables alone (often nothing)
        ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=q.device) if ws_bytes else None
        rc = lib.dsa_attn_mass_saved_bitmap(_ptr(qb), _ptr(kb), _ptr(lse.contiguous()), _ptr(idx), _ptr(n), _ptr(cu), T,
                                            cu.numel() - 1, Hq, Hkv, D, K, scale, _lib.DSA_DTYPE_BF16, max_seqlen, _ptr(mass),
                                            _ptr(bitmap), bitmap.numel(), _ptr(ws), ws_bytes, _stream(q.device))
        _lib.check(rc, "dsa_attn_mass_saved_bitmap")
        return mass
    ws = torch.empty((max(ws_bytes, 4),), dtype=torch.uint8, device=q.device)
    rc = lib.dsa_attn_mass(_ptr(qb), _ptr(kb), _ptr(lse.contiguous()), _ptr(idx), _ptr(n), _ptr(cu), T, cu.numel() - 1, Hq,
                           Hkv, D, K, scale, _lib.DSA_DTYPE_BF16, max_seqlen, _ptr(mass), _ptr(ws), ws_bytes,
                           _stream(q.device))
    _lib.check(rc, "dsa_attn_mass")
    return mass


def attn_bwd(dout, q, k, v, out, lse, idx, n, cu_seqlens, max_seqlen: int, softmax_scale: float,
             parts: int = 15, buffers=None, causal: bool = True):
    """Stage D4.  ``parts``/``buffers`` exist for per-kernel timing: ``buffers=(dq, dk, dv, ws)`` reuses
    the outputs and workspace of an earlier full call."""
    T, Hq, Hkv, D = _check_qkv(q, k, v)
    cu = _check_cu(cu_seqlens, T)
    K = idx.shape[1] if idx is not None else 0
    lib = _lib.load()
    ws_bytes = lib.dsa_attn_bwd_workspace_bytes(T, Hq, max_seqlen, 1 if idx is not None else 0)
    if buffers is None:
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        ws = torch.empty((max(ws_bytes, 4),), dtype=torch.uint8, device=q.device)
    else:
        dq, dk, dv, ws = buffers
    rc = lib.dsa_attn_bwd_parts(_ptr(dout), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(idx), _ptr(n),
                                _ptr(cu), T, cu.numel() - 1, Hq, Hkv, D, K, softmax_scale, _lib.DSA_DTYPE_BF16,
                                max_seqlen, 1 if causal else 0, _ptr(dq), _ptr(dk), _ptr(dv), _ptr(ws), ws_bytes, parts,
                                _stream(q.device))
    _lib.check(rc, "dsa_attn_bwd")
    return (dq, dk, dv) if buffers is None else (dq, dk, dv, ws)


def attn_bwd_saved_bitmap(dout, q, k, v, out, lse, idx, n, cu_seqlens, max_seqlen: int, softmax_scale: float, fwd_ws,
                          causal: bool = True):
    """Stage D4 reading the selection bitmap out of the forward's workspace ``fwd_ws`` (None for dense attention); the
    scratch it allocates lives for the call only."""
    T, Hq, Hkv, D = _check_qkv(q, k, v)
    cu = _check_cu(cu_seqlens, T)
    K = idx.shape[1] if idx is not None else 0
    lib = _lib.load()
    N = cu.numel() - 1
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    sc_bytes = lib.dsa_attn_bwd_scratch_bytes(T, N, Hq, Hkv, D)
    scratch = torch.empty((max(sc_bytes, 4),), dtype=torch.uint8, device=q.device)
    rc = lib.dsa_attn_bwd_saved_bitmap(_ptr(dout), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(idx), _ptr(n),
                                       _ptr(cu), T, N, Hq, Hkv, D, K, softmax_scale, _lib.DSA_DTYPE_BF16, max_seqlen,
                                       1 if causal else 0, _ptr(dq), _ptr(dk), _ptr(dv), _ptr(fwd_ws),
                                       0 if fwd_ws is None else fwd_ws.numel(), _ptr(scratch), sc_bytes, _stream(q.device))
    _lib.check(rc, "dsa_attn_bwd_saved_bitmap")
    return dq, dk, dv


# ------------------------------------------------------------------------------------------------
# the operator
# ------------------------------------------------------------------------------------------------
def _split_stack(x: torch.Tensor, order: int) -> torch.Tensor:
    """fp32 (T,H,D) -> bf16 (T,H,4D): hi = bf16(x), lo = bf16(x - hi) stacked along head_dim, order 0 = [hi, lo, hi, 0],
    order 1 = [hi, hi, lo, 0] (one kernel)."""
    x = x.contiguous()
    T, H, D = x.shape
    y = torch.empty((T, H, 4 * D), dtype=torch.bfloat16, device=x.device)
    rc = _lib.load().dsa_split_bf16_stack(_ptr(x), T * H, D, order, _ptr(y), _stream(x.device))
    _lib.check(rc, "dsa_split_bf16_stack")
    return y


def _split_combine(y: torch.Tensor, part: int) -> torch.Tensor:
    """bf16 (T,H,4D) -> fp32 (T,H,D): y[..., :D] + y[..., part*D:(part+1)*D] (one kernel)."""
    T, H, D4 = y.shape
    out = torch.empty((T, H, D4 // 4), dtype=torch.float32, device=y.device)
    rc = _lib.load().dsa_split_bf16_combine(_ptr(y), T * H, D4 // 4, part, _ptr(out), _stream(y.device))
    _lib.check(rc, "dsa_split_bf16_combine")
    return out


def _split_stack_qkv(q, k, v):
    """The three operands of one call in one launch: q and v with order 0, k with order 1."""
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    (T, Hq, D), Hkv = q.shape, k.shape[1]
    yq = torch.empty((T, Hq, 4 * D), dtype=torch.bfloat16, device=q.device)
    ykv = torch.empty((2, T, Hkv, 4 * D), dtype=torch.bfloat16, device=q.device)
    rc = _lib.load().dsa_split_bf16_stack_qkv(_ptr(q), _ptr(k), _ptr(v), T * Hq, T * Hkv, D, _ptr(yq), _ptr(ykv[0]),
                                              _ptr(ykv[1]), _stream(q.device))
    _lib.check(rc, "dsa_split_bf16_stack_qkv")
    return yq, ykv[0], ykv[1]


def _split_combine_qkv(dq, dk, dv):
    """The three gradients back to fp32 in one launch: dq and dv with part 2, dk with part 1."""
    (T, Hq, D4), Hkv = dq.shape, dk.shape[1]
    D = D4 // 4
    oq = torch.empty((T, Hq, D), dtype=torch.float32, device=dq.device)
    okv = torch.empty((2, T, Hkv, D), dtype=torch.float32, device=dq.device)
    rc = _lib.load().dsa_split_bf16_combine_qkv(_ptr(dq), _ptr(dk), _ptr(dv), T * Hq, T * Hkv, D, _ptr(oq), _ptr(okv[0]),
                                                _ptr(okv[1]), _stream(dq.device))
    _lib.check(rc, "dsa_split_bf16_combine_qkv")
    return oq, okv[0], okv[1]


class _DsaVarlenAttn(torch.autograd.Function):
    """bf16 inputs go to the kernels as they are.  fp32 inputs with 4*D <= 256 are carried as split-bf16
    operands (x = hi + lo) stacked along head_dim, which keeps near-fp32 logits on the bf16 MFMA path:
        Q' = [q_hi, q_lo, q_hi, 0]   K' = [k_hi, k_hi, k_lo, 0]   ->  Q'.K' = q.k - q_lo.k_lo
        V' = [v_hi, v_lo, v_hi, 0]   ->  out = out'[0:D] + out'[D:2D]
        dO' = [g_hi, g_hi, g_lo, 0]  ->  dO'.V' = g.v - g_lo.v_lo ;  dq = dq'[0:D] + dq'[2D:3D],
                                         dk = dk'[0:D] + dk'[D:2D], dv = dv'[0:D] + dv'[2D:3D]
    Other dtypes / larger head_dim are rounded to bf16 once."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, max_seqlen, idx, n, softmax_scale, causal=True, want_mass=False, bitmap=None):
        in_dtype = q.dtype
        D = q.shape[-1]
        split = in_dtype == torch.float32 and 4 * D <= 256
        if split:
            qb, kb, vb = _split_stack_qkv(q, k, v)
        else:
            qb, kb, vb = _as_bf16(q), _as_bf16(k), _as_bf16(v)
        fwd_ws = None
        lib = _lib.load()
        if idx is not None and lib.dsa_get_tile_crossover() > 0:     # (crossover 0: no kernel reads a bitmap)
            # the selection bitmap - left by the top-k kernel (`bitmap`), else built by the forward - is kept for the
            # backward; nothing else is held in between (delta, the key-tile order and the partial sums of cut walks
            # are allocated when the backward runs)
            fwd_ws = bitmap if bitmap is not None else torch.empty(
                (max(lib.dsa_attn_fwd_workspace_bytes(qb.shape[0], int(max_seqlen), 1), 4),), dtype=torch.uint8, device=qb.device)
        out, lse = attn_fwd(qb, kb, vb, idx, n, cu_seqlens, int(max_seqlen), softmax_scale, causal, ws=fwd_ws,
                            bitmap_ready=fwd_ws is not None and bitmap is not None)
        ctx.fwd_ws = fwd_ws
        ctx.causal = bool(causal)
        ctx.save_for_backward(qb, kb, vb, out, lse, cu_seqlens, *(() if idx is None else (idx, n)))
        ctx.has_idx = idx is not None
        ctx.max_seqlen = int(max_seqlen)
        ctx.softmax_scale = softmax_scale
        ctx.in_dtype = in_dtype
        ctx.split = split
        ctx.D = D
        if split:
            res = _split_combine(out, 1)
        else:
            res = out if in_dtype == torch.bfloat16 else out.to(in_dtype)
        if not want_mass:
            return res
        # from the very operands and log-sum-exp of the forward, so that every row sums to one
        mass = attn_mass(qb, kb, lse, idx, n, cu_seqlens, int(max_seqlen), softmax_scale, bitmap=fwd_ws)
        ctx.mark_non_differentiable(mass)
        return res, mass

    @staticmethod
    def backward(ctx, dout, *_):
        saved = ctx.saved_tensors
        qb, kb, vb, out, lse, cu = saved[:6]
        idx, n = (saved[6], saved[7]) if ctx.has_idx else (None, None)
        D = ctx.D
        if ctx.split:
            db = _split_stack(dout.float(), 1)
        else:
            db = _as_bf16(dout)
        if ctx.fwd_ws is not None or idx is None:        # the forward's bitmap is read where it lies
            dq, dk, dv = attn_bwd_saved_bitmap(db, qb, kb, vb, out, lse, idx, n, cu, ctx.max_seqlen, ctx.softmax_scale,
                                               ctx.fwd_ws, causal=ctx.causal)
            ctx.fwd_ws = None
        else:
            dq, dk, dv = attn_bwd(db, qb, kb, vb, out, lse, idx, n, cu, ctx.max_seqlen, ctx.softmax_scale,
                                  causal=ctx.causal)
        if ctx.split:
            dq, dk, dv = _split_combine_qkv(dq, dk, dv)
        elif ctx.in_dtype != torch.bfloat16:
            dq, dk, dv = dq.to(ctx.in_dtype), dk.to(ctx.in_dtype), dv.to(ctx.in_dtype)
        return dq, dk, dv, None, None, None, None, None, None, None, None


@torch.compiler.disable                                  # a compiled caller (the reference compiles per block) breaks the graph here
def dsa_varlen_attn(q, k, v, cu_seqlens, max_seqlen: Optional[int] = None, *, indexer_q=None, indexer_k=None, indexer_w=None,
                    top_k: Optional[int] = None, index_scale: Optional[float] = None,
                    softmax_scale: Optional[float] = None, return_indices: bool = False, causal: bool = True,
                    return_mass: bool = False, return_scores: bool = False):
    """Packed causal attention over ``cu_seqlens`` segments, optionally sparsified by the DSA indexer.

    q (T,Hq,D), k/v (T,Hkv,D) contiguous, cu_seqlens (N+1,) int32 on the device, max_seqlen host int
    (the reference's callers already hold it: models/qwen3_vl/model.py:765) - any upper bound of the
    longest segment gives the same result, and ``None`` stands for the bound T, which needs no
    device-to-host copy of the segment lengths (train/model_attention.py:120-121 syncs for it).  Without indexer inputs
    every causal key of the token's own segment is attended (the reference's behaviour).  With
    ``indexer_q (T,Hi,Di)``, ``indexer_k (T,Di)``, ``indexer_w (T,Hi)`` and ``top_k`` each query keeps
    the top_k keys of its causal window under (indexer score descending, key index ascending).
    ``return_mass=True`` (with the indexer inputs) also returns the (T, top_k) fp32 table of head-averaged attention
    probabilities of the selected keys, rows summing to one and aligned with the indices: the detached target of the
    KL loss that trains the indexer.  ``return_scores=True`` appends the (T, top_k) fp32 indexer scores of the selected
    keys (every row is then scored, also those whose whole window is selected), which ``indexer_kl_loss`` takes as
    ``selection=(idx, n, scores)`` instead of running the indexer again.
    Gradients flow to q, k, v only.  A head_dim between the kernels' 64 / 128 / 256 is zero-padded to the
    next one and the output cut back (the scale stays that of the true head_dim).  ``causal=False`` (dense only) attends every key of the own segment, the
    vision towers' form of the call (models/qwen3_vl/model.py:423-428).
    """
    _require_cuda(q, k, v, cu_seqlens)
    T, Hq, Hkv, D = _check_qkv(q, k, v)
    max_seqlen = T if max_seqlen is None else int(max_seqlen)
    cu = _check_cu(cu_seqlens, T, max_seqlen)
    scale = float(softmax_scale) if softmax_scale is not None else D ** -0.5
    sparse = indexer_q is not None or indexer_k is not None or indexer_w is not None
    idx = n = bitmap = None
    if sparse and not causal:
        raise ValueError("DSA key selection is defined for causal attention only")
    if sparse:
        if indexer_q is None or indexer_k is None or indexer_w is None or top_k is None:
            raise ValueError("DSA needs indexer_q, indexer_k, indexer_w and top_k together")
        if indexer_q.shape[0] != T:
            raise ValueError("indexer tensors must cover the same T packed tokens as q")
        lib = _lib.load()
        if lib.dsa_get_tile_crossover() > 0:
            # the top-k kernel leaves the inverted selection here: forward and backward read it, nothing builds it again
            bitmap = torch.empty((max(lib.dsa_attn_fwd_workspace_bytes(T, int(max_seqlen), 1), 4),), dtype=torch.uint8,
                                 device=q.device)
        with torch.no_grad():
            if return_scores:
                idx, n, sel_scores = index_topk(indexer_q, indexer_k, indexer_w, cu, int(max_seqlen), int(top_k), index_scale,
                                                return_scores=True, bitmap=bitmap)
            else:
                idx, n = index_topk(indexer_q, indexer_k, indexer_w, cu, int(max_seqlen), int(top_k), index_scale, bitmap=bitmap)
    elif return_indices or return_scores:
        raise ValueError("return_indices / return_scores need the indexer inputs")
    dims = _KERNEL_HEAD_DIMS if sparse else _KERNEL_HEAD_DIMS_DENSE
    d_kernel = next((d for d in dims if d >= D), None)
    if d_kernel is None:
        raise ValueError(f"head_dim {D} is beyond the kernels' largest ({_KERNEL_HEAD_DIMS[-1]})")
    if d_kernel != D:
        # e.g. the 72-wide heads of the 1152/16 vision towers: zero columns change neither q.k nor the used part of p.v
        q, k, v = (torch.nn.functional.pad(x, (0, d_kernel - D)) for x in (q, k, v))
    if return_mass and not sparse:
        raise ValueError("return_mass needs the indexer inputs")
    out = _DsaVarlenAttn.apply(q.contiguous(), k.contiguous(), v.contiguous(), cu, int(max_seqlen), idx, n, scale,
                               bool(causal), bool(return_mass), bitmap)
    mass = None
    if return_mass:
        out, mass = out
    if d_kernel != D:
        out = out[..., :D]
    res = (out,) + ((idx, n) if return_indices else ()) + ((mass,) if return_mass else ()) + (
        (sel_scores,) if return_scores else ())
    return res if len(res) > 1 else out
