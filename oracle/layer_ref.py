"""CPU restatement of the reference's attention layers (TEST INFRASTRUCTURE ONLY: imported by tests/, never by the
package).

* ``qwen3vl_attention``  - models/qwen3_vl/model.py:246-278 (and train/model_attention.py:188-252, the same
  sequence on the HF modules): q/k/v projection, per-head ``F.rms_norm``, transpose, ``apply_rope``, transpose back,
  packed causal attention, ``o_proj``.
* ``qwen3_5_attention``  - models/qwen3_5/model.py:100-136 (train/model_attention.py:146-185): ``q_proj`` emits
  ``[q | gate]`` per head, the norms scale by ``1 + weight``, the rotary width may be below head_dim, the attention
  output is multiplied by ``sigmoid(gate)`` before ``o_proj``.
* ``dsa_layer``          - either of the two with the attention restricted to a given selection and the indexer's KL
  loss beside it (no counterpart in the reference: the formulas of oracle/dsa_ref.py on the layer's own q, k).

fp32 torch ops throughout, differentiable in every weight.  Pinned by tests/test_layer_oracle.py against library
routines used a different way (one ``F.scaled_dot_product_attention`` per segment with ``enable_gqa``, rotation
written with complex numbers) on small inputs.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import dsa_ref as R
from . import prologue_ref as P


def _project(x, wq, wk, wv, head_dim, gated):
    h = x.reshape(-1, x.shape[-1]).float()
    T = h.shape[0]
    qp = F.linear(h, wq.float())
    if gated:                                            # models/qwen3_5/model.py:111-112
        qg = qp.view(T, -1, 2 * head_dim)
        q, gate = qg[..., :head_dim], qg[..., head_dim:]
    else:
        q, gate = qp.view(T, -1, head_dim), None
    k = F.linear(h, wk.float()).view(T, -1, head_dim)
    v = F.linear(h, wv.float()).view(T, -1, head_dim)
    return q, k, v, gate


def _norm_rope(q, k, qn_w, kn_w, cos, sin, eps, offset):
    cos, sin = (c[0] if c.dim() == 3 else c for c in (cos, sin))
    return P.qk_norm_rope(q, k, qn_w.float(), kn_w.float(), cos.float(), sin.float(), eps, offset)


def qwen3vl_attention(x, wq, wk, wv, wo, qn_w, kn_w, cos, sin, cu_seqlens, head_dim, eps=1e-6):
    """x (1,T,hidden) -> (1,T,hidden), dense causal attention inside every segment."""
    q, k, v, _ = _project(x, wq, wk, wv, head_dim, gated=False)
    q, k = _norm_rope(q, k, qn_w, kn_w, cos, sin, eps, offset=False)
    out = R.dense_varlen_causal(q, k, v, cu_seqlens)
    return F.linear(out.reshape(1, out.shape[0], -1), wo.float())


def qwen3_5_attention(x, wq, wk, wv, wo, qn_w, kn_w, cos, sin, cu_seqlens, head_dim, eps=1e-6):
    q, k, v, gate = _project(x, wq, wk, wv, head_dim, gated=True)
    q, k = _norm_rope(q, k, qn_w, kn_w, cos, sin, eps, offset=True)
    out = R.dense_varlen_causal(q, k, v, cu_seqlens)
    out = P.sigmoid_gate(out, gate)
    return F.linear(out.reshape(1, out.shape[0], -1), wo.float())


def dsa_layer(x, wq, wk, wv, wo, qn_w, kn_w, cos, sin, cu_seqlens, head_dim, wiq, wik, wiw, index_heads, index_dim, idx, n,
              eps=1e-6, gated=False, index_scale=None, round_indexer_to_bf16=False):
    """(layer output, indexer KL loss) for the selection ``idx, n``: attention over the selected keys, and
    mean_t KL(attention mass of the selected keys || softmax of the indexer's scores of the selected keys).  The mass is
    detached and the indexer reads a detached input, as in the layer under test."""
    q, k, v, gate = _project(x, wq, wk, wv, head_dim, gated=gated)
    q, k = _norm_rope(q, k, qn_w, kn_w, cos, sin, eps, offset=gated)
    out = R.sparse_attention(q, k, v, idx, n, cu_seqlens)
    if gated:
        out = P.sigmoid_gate(out, gate)
    y = F.linear(out.reshape(1, out.shape[0], -1), wo.float())
    h = x.detach().reshape(-1, x.shape[-1]).float()
    T = h.shape[0]
    iq = F.linear(h, wiq.float()).view(T, index_heads, index_dim)
    ik = F.linear(h, wik.float())
    iw = F.linear(h, wiw.float())
    if round_indexer_to_bf16:
        # The layer under test hands the indexer kernels bf16 projections.  The indexer's gradient passes the gate
        # [q_idx.k_idx > 0], a step function: to compare gradients the checker must open the same gates, i.e. see the
        # same rounded values (straight-through: the rounding itself passes the gradient unchanged).
        iq, ik, iw = (t + (t.to(torch.bfloat16).float() - t).detach() for t in (iq, ik, iw))
    mass = R.attention_mass(q.detach(), k.detach(), idx, n, cu_seqlens)
    sel = R.selected_scores(iq, ik, iw, idx, n, cu_seqlens, index_scale)
    return y, R.indexer_kl(sel, mass, n).mean(), (iq, ik, iw)
