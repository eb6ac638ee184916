"""Attention layers with the reference's forward signatures, composed from library GEMMs and the HIP operator.

* ``Qwen3VLTextAttention``  - models/qwen3_vl/model.py:230-278: q/k/v projections -> per-head RMSNorm -> RoPE ->
  packed causal attention -> ``o_proj``;  ``forward(x, cos, sin, cu_seqlens, max_seqlen)``.
* ``SelfAttention``         - models/qwen3_5/model.py:76-136: the same with ``q_proj`` emitting ``[q | gate]`` per
  head, OffsetRMSNorm (``1 + weight``), a rotary width that may be smaller than head_dim, the output multiplied by
  ``sigmoid(gate)``, and DTensor unwrap / rewrap around the kernels (models/qwen3_5/model.py:124,132).
* ``DsaIndexer``            - the lightning indexer's projections as module parameters (the reference holds no
  indexer): hidden -> Hi*Di index queries, hidden -> Di index key (one per token), hidden -> Hi head weights.

The projections stay torch GEMMs.  Norm + RoPE + layout is one kernel (``qk_norm_rope``), the attention is
``dsa_varlen_attn`` (dense causal without an indexer: the reference's behaviour), the gate is one kernel.
With an indexer the layer keeps the top-k keys per query and leaves the indexer's KL loss in ``self.indexer_loss``
(the selection passes no gradient; the loss is what trains the indexer); ``indexer_losses(model)`` adds them up
for the training step (train/train_qwen.py:534-548: ``loss = out.loss + indexer_losses(model)``).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn

from .dtensor_utils import _dtensor_rewrap, _dtensor_unwrap, _local
from .model_attention import run_varlen_attn
from .ops import dsa_varlen_attn, indexer_kl_loss
from .prologue import qk_norm_rope, sigmoid_gate


@dataclass
class DsaConfig:
    """Indexer geometry of a DSA layer: ``index_heads`` x ``index_dim`` index queries per token, ``top_k`` keys kept."""
    index_heads: int
    index_dim: int
    top_k: int
    index_scale: Optional[float] = None          # default index_dim**-0.5 * index_heads**-0.5
    loss_weight: float = 1.0


class DsaIndexer(nn.Module):
    """hidden -> (index queries (T,Hi,Di), index key (T,Di), head weights (T,Hi)).

    The input is detached: the KL loss trains these three projections only, as in DSA's sparse training stage
    (the main model sees the indexer through the selection alone, which has no gradient)."""

    def __init__(self, hidden_size: int, cfg: DsaConfig):
        super().__init__()
        self.cfg = cfg
        self.q_proj = nn.Linear(hidden_size, cfg.index_heads * cfg.index_dim, bias=False)
        self.k_proj = nn.Linear(hidden_size, cfg.index_dim, bias=False)
        self.w_proj = nn.Linear(hidden_size, cfg.index_heads, bias=False)

    def forward(self, x: torch.Tensor):
        h = x.detach().reshape(-1, x.shape[-1])
        T = h.shape[0]
        iq = self.q_proj(h).view(T, self.cfg.index_heads, self.cfg.index_dim)
        return iq, self.k_proj(h), self.w_proj(h)


def _bf16(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16)


def attention_core(module, q_lin, k_lin, v_lin, cos, sin, cu_seqlens, max_seqlen, x=None, gate=None, offset=False):
    """(T,Hq,D), (T,Hkv,D), (T,Hkv,D) projection outputs (views with any token / head stride) -> (T,Hq,D).

    ``module`` supplies ``q_norm`` / ``k_norm`` (weight, eps) and optionally ``indexer``; the indexer's loss is left
    in ``module.indexer_loss``."""
    eps = getattr(module.q_norm, "eps", None)
    if eps is None:
        eps = getattr(module.q_norm, "variance_epsilon", 1e-6)
    q, k = qk_norm_rope(_bf16(q_lin), _bf16(k_lin), _local(module.q_norm.weight), _local(module.k_norm.weight), cos, sin,
                        eps=eps, offset=offset)
    v = _bf16(v_lin).contiguous()
    indexer = getattr(module, "indexer", None)
    module.indexer_loss = None
    if indexer is None:
        out = dsa_varlen_attn(q, k, v, cu_seqlens, max_seqlen)
    else:
        cfg = indexer.cfg
        iq, ik, iw = indexer(x)
        want_loss = torch.is_grad_enabled() and any(p.requires_grad for p in indexer.parameters())
        if want_loss:
            out, idx, n, mass, sel = dsa_varlen_attn(q, k, v, cu_seqlens, max_seqlen, indexer_q=iq, indexer_k=ik, indexer_w=iw,
                                                     top_k=cfg.top_k, index_scale=cfg.index_scale, return_indices=True,
                                                     return_mass=True, return_scores=True)
            module.indexer_loss = cfg.loss_weight * indexer_kl_loss(iq, ik, iw, mass, cu_seqlens, max_seqlen, cfg.top_k,
                                                                     cfg.index_scale, selection=(idx, n, sel))
        else:
            out = dsa_varlen_attn(q, k, v, cu_seqlens, max_seqlen, indexer_q=iq, indexer_k=ik, indexer_w=iw,
                                  top_k=cfg.top_k, index_scale=cfg.index_scale)
    if gate is not None:
        out = sigmoid_gate(out, _bf16(gate))
    return out


def indexer_losses(model: nn.Module):
    """Sum of the indexer losses the DSA layers of ``model`` left behind in their last forward (None if there is none)."""
    total = None
    for m in model.modules():
        loss = getattr(m, "indexer_loss", None)
        if loss is not None:
            total = loss if total is None else total + loss
    return total


class RMSNorm(nn.Module):
    """models/qwen3_vl/model.py:155-162.  Holds weight and eps; inside the attention layers the norm itself runs fused
    with RoPE, this forward is the stand-alone form."""

    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        return torch.nn.functional.rms_norm(x, self.weight.shape, self.weight, self.eps)


class OffsetRMSNorm(nn.Module):
    """models/qwen3_5/model.py:58-72: ``(1 + weight) * norm(x)``, weight initialised to zeros."""

    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.zeros(dim))

    def forward(self, x):
        return torch.nn.functional.rms_norm(x, self.weight.shape, 1.0 + self.weight, self.eps)


class Qwen3VLTextAttention(nn.Module):
    """models/qwen3_vl/model.py:230-278 with the same constructor (a config holding hidden_size,
    num_attention_heads, num_key_value_heads, head_dim, rms_norm_eps) and forward signature; ``dsa`` turns the
    layer into a DSA layer with its own indexer."""

    def __init__(self, cfg, dsa: Optional[DsaConfig] = None):
        super().__init__()
        self.num_heads = cfg.num_attention_heads
        self.num_kv_heads = cfg.num_key_value_heads
        self.head_dim = cfg.head_dim
        self.n_rep = self.num_heads // self.num_kv_heads
        self.q_proj = nn.Linear(cfg.hidden_size, self.num_heads * self.head_dim, bias=False)
        self.k_proj = nn.Linear(cfg.hidden_size, self.num_kv_heads * self.head_dim, bias=False)
        self.v_proj = nn.Linear(cfg.hidden_size, self.num_kv_heads * self.head_dim, bias=False)
        self.o_proj = nn.Linear(self.num_heads * self.head_dim, cfg.hidden_size, bias=False)
        self.q_norm = RMSNorm(self.head_dim, eps=cfg.rms_norm_eps)
        self.k_norm = RMSNorm(self.head_dim, eps=cfg.rms_norm_eps)
        self.indexer = DsaIndexer(cfg.hidden_size, dsa) if dsa is not None else None
        self.indexer_loss = None

    def forward(self, x, cos, sin, cu_seqlens, max_seqlen):
        total = x.shape[1]
        # head counts come from the projections' outputs, so a head-sharded (tensor-parallel) layer sees its own
        q = self.q_proj(x).view(total, -1, self.head_dim)
        k = self.k_proj(x).view(total, -1, self.head_dim)
        v = self.v_proj(x).view(total, -1, self.head_dim)
        (q, k, v), wrap = _dtensor_unwrap(q, k, v)
        out = attention_core(self, q, k, v, cos, sin, cu_seqlens, max_seqlen, x=x)   # (total, heads, head_dim)
        out = _dtensor_rewrap(out, wrap)
        return self.o_proj(out.reshape(1, total, -1).to(x.dtype))


class SelfAttention(nn.Module):
    """models/qwen3_5/model.py:76-136 (the full-attention layers of the hybrid stack): gated, OffsetRMSNorm, the
    rotary width is whatever the cos / sin tables have."""

    def __init__(self, cfg, dsa: Optional[DsaConfig] = None):
        super().__init__()
        self.num_heads = cfg.num_attention_heads
        self.num_kv_heads = cfg.num_key_value_heads
        self.head_dim = cfg.head_dim
        self.n_rep = self.num_heads // self.num_kv_heads
        self.q_proj = nn.Linear(cfg.hidden_size, self.num_heads * self.head_dim * 2, bias=False)
        self.k_proj = nn.Linear(cfg.hidden_size, self.num_kv_heads * self.head_dim, bias=False)
        self.v_proj = nn.Linear(cfg.hidden_size, self.num_kv_heads * self.head_dim, bias=False)
        self.o_proj = nn.Linear(self.num_heads * self.head_dim, cfg.hidden_size, bias=False)
        self.q_norm = OffsetRMSNorm(self.head_dim, eps=cfg.rms_norm_eps)
        self.k_norm = OffsetRMSNorm(self.head_dim, eps=cfg.rms_norm_eps)
        self.indexer = DsaIndexer(cfg.hidden_size, dsa) if dsa is not None else None
        self.indexer_loss = None

    # models/qwen3_5/model.py:90-98: the reference's name for the attention call of this layer (packed (T,H,D) tensors
    # in and out, outside any compiled graph).  The layer's own forward goes through ``attention_core``, which fuses
    # norm and RoPE in front of the same operator; this name is kept for code that calls the attention call directly.
    _run_varlen_attn = staticmethod(run_varlen_attn)

    def forward(self, x, cos, sin, cu_seqlens, max_seqlen):
        total = x.shape[1]
        D = self.head_dim
        qg = self.q_proj(x).view(total, -1, 2 * D)              # per head [q | gate]: both halves are read in place
        k = self.k_proj(x).view(total, -1, D)
        v = self.v_proj(x).view(total, -1, D)
        (qg, k, v), wrap = _dtensor_unwrap(qg, k, v)
        out = attention_core(self, qg[..., :D], k, v, cos, sin, cu_seqlens, max_seqlen, x=x, gate=qg[..., D:], offset=True)
        out = _dtensor_rewrap(out, wrap)
        return self.o_proj(out.reshape(1, total, -1).to(x.dtype))
