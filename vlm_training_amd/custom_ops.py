"""The operator as ``torch.library`` custom ops with fake (shape-only) implementations, so that a compiled block can
hold it without a graph break.

The reference compiles every transformer block (train/infra.py:236-248) and keeps its attention call out of the graph
with ``@torch.compiler.disable`` (models/qwen3_5/model.py:90-91); torch's own ``varlen_attn`` is a registered custom op
with a fake impl instead (torch/nn/attention/varlen.py).  ``ops.dsa_varlen_attn`` follows the reference (a graph break);
``dsa_varlen_attn_traceable`` below follows torch: three ops - selection, forward, backward - that ``torch.compile(...,
fullgraph=True)`` traces through, the backward wired with ``register_autograd``.  bf16 tensors, head_dim 64 / 128 / 256
(96 as well without a selection); the fp32 carrier, head_dim padding, the attention mass and the selected scores stay
with ``ops.dsa_varlen_attn``.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib, ops

_NS = "vlm_training_amd"


@torch.library.custom_op(f"{_NS}::index_topk", mutates_args=())
def _index_topk(q_idx: torch.Tensor, k_idx: torch.Tensor, w_idx: torch.Tensor, cu_seqlens: torch.Tensor, max_seqlen: int,
                top_k: int, index_scale: Optional[float]) -> Tuple[torch.Tensor, torch.Tensor]:
    return ops.index_topk(q_idx, k_idx, w_idx, cu_seqlens, max_seqlen, top_k, index_scale)


@_index_topk.register_fake
def _(q_idx, k_idx, w_idx, cu_seqlens, max_seqlen, top_k, index_scale):
    T = q_idx.shape[0]
    return q_idx.new_empty((T, top_k), dtype=torch.int32), q_idx.new_empty((T,), dtype=torch.int32)


@torch.library.custom_op(f"{_NS}::attn_fwd", mutates_args=())
def _attn_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor, max_seqlen: int,
              idx: Optional[torch.Tensor], n: Optional[torch.Tensor], softmax_scale: float,
              causal: bool) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(out (T,Hq,D) bf16, lse (Hq,T) fp32, the forward's workspace = the selection bitmap the backward reads)."""
    lib = _lib.load()
    nbytes = lib.dsa_attn_fwd_workspace_bytes(q.shape[0], max_seqlen, 1) if idx is not None else 0
    # every byte of an op's output has to be defined (a compiler may compare or cache it): the bitmap rows are written
    # by the forward, the alignment padding behind them - or the whole stand-in without a selection - is cleared here
    if nbytes:
        ws = torch.empty((nbytes,), dtype=torch.uint8, device=q.device)
        ws[-256:].zero_()
    else:
        ws = torch.zeros((4,), dtype=torch.uint8, device=q.device)
    out, lse = ops.attn_fwd(q, k, v, idx, n, cu_seqlens, max_seqlen, softmax_scale, causal, ws=ws)
    return out, lse, ws


@_attn_fwd.register_fake
def _(q, k, v, cu_seqlens, max_seqlen, idx, n, softmax_scale, causal):
    T, Hq, _ = q.shape
    nbytes = (T * ((max_seqlen + 31) // 32) * 4 + 255) // 256 * 256 if idx is not None else 4
    return (torch.empty_like(q), q.new_empty((Hq, T), dtype=torch.float32), q.new_empty((max(nbytes, 4),), dtype=torch.uint8))


@torch.library.custom_op(f"{_NS}::attn_bwd", mutates_args=())
def _attn_bwd(dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, lse: torch.Tensor,
              cu_seqlens: torch.Tensor, idx: Optional[torch.Tensor], n: Optional[torch.Tensor], fwd_ws: torch.Tensor,
              max_seqlen: int, softmax_scale: float, causal: bool) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    if idx is not None and _lib.load().dsa_get_tile_crossover() <= 0:      # gather-only forward: it built no bitmap
        return ops.attn_bwd(dout.contiguous(), q, k, v, out, lse, idx, n, cu_seqlens, max_seqlen, softmax_scale, causal=causal)
    return ops.attn_bwd_saved_bitmap(dout.contiguous(), q, k, v, out, lse, idx, n, cu_seqlens, max_seqlen, softmax_scale,
                                     fwd_ws if idx is not None else None, causal=causal)


@_attn_bwd.register_fake
def _(dout, q, k, v, out, lse, cu_seqlens, idx, n, fwd_ws, max_seqlen, softmax_scale, causal):
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)


def _setup_context(ctx, inputs, output):
    q, k, v, cu_seqlens, max_seqlen, idx, n, softmax_scale, causal = inputs
    out, lse, ws = output
    ctx.save_for_backward(q, k, v, out, lse, cu_seqlens, ws, *(() if idx is None else (idx, n)))
    ctx.has_idx = idx is not None
    ctx.max_seqlen, ctx.softmax_scale, ctx.causal = max_seqlen, softmax_scale, causal


def _backward(ctx, dout, dlse, dws):
    q, k, v, out, lse, cu, ws = ctx.saved_tensors[:7]
    idx, n = ctx.saved_tensors[7:9] if ctx.has_idx else (None, None)
    dq, dk, dv = _attn_bwd(dout, q, k, v, out, lse, cu, idx, n, ws, ctx.max_seqlen, ctx.softmax_scale, ctx.causal)
    return dq, dk, dv, None, None, None, None, None, None


_attn_fwd.register_autograd(_backward, setup_context=_setup_context)


def dsa_varlen_attn_traceable(q, k, v, cu_seqlens, max_seqlen: int, *, indexer_q=None, indexer_k=None, indexer_w=None,
                              top_k: Optional[int] = None, index_scale: Optional[float] = None,
                              softmax_scale: Optional[float] = None, causal: bool = True):
    """``ops.dsa_varlen_attn`` for bf16 (T,H,D) tensors, built from custom ops a compiler can trace through (no graph
    break).  ``max_seqlen`` is a host integer (an upper bound of the longest segment; the packed length always is)."""
    if q.dtype != torch.bfloat16 or k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16:
        raise ValueError("the traceable operator takes bf16 tensors; ops.dsa_varlen_attn carries other dtypes")
    scale = float(softmax_scale) if softmax_scale is not None else q.shape[-1] ** -0.5
    idx = n = None
    if indexer_q is not None:
        if indexer_k is None or indexer_w is None or top_k is None:
            raise ValueError("DSA needs indexer_q, indexer_k, indexer_w and top_k together")
        if not causal:
            raise ValueError("DSA key selection is defined for causal attention only")
        idx, n = _index_topk(indexer_q.detach(), indexer_k.detach(), indexer_w.detach(), cu_seqlens, int(max_seqlen), int(top_k),
                             index_scale)
    out, _, _ = _attn_fwd(q.contiguous(), k.contiguous(), v.contiguous(), cu_seqlens, int(max_seqlen), idx, n, scale, bool(causal))
    return out
