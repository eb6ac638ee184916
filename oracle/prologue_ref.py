"""CPU restatement of the element-wise work either side of the attention operator (TEST INFRASTRUCTURE ONLY:
imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg, never by the package).

Follows the reference line by line, in fp32 unless ``eager_bf16`` asks for the rounding of every eager
bf16 operation:

* ``rms_norm``      - models/qwen3_vl/model.py:155-162 (``F.rms_norm(x, shape, weight, eps)``) and the offset
                      variant ``F.rms_norm(x, shape, 1 + weight, eps)`` of models/qwen3_5/model.py:58-72.
* ``rotate_half``   - models/qwen3_vl/model.py:177-179.
* ``apply_rope``    - models/qwen3_vl/model.py:181-193 and, for a rotary width R < D,
                      models/qwen3_5/utils.py:88-110.
* ``qk_norm_rope``  - the sequence models/qwen3_vl/model.py:256-269 / models/qwen3_5/model.py:110-129:
                      norm per head, transpose, rope, transpose back, contiguous (T, H, D).
* ``sigmoid_gate``  - models/qwen3_5/model.py:135.

Pinned by tests/test_prologue_oracle.py: against ``torch.nn.functional.rms_norm``, against plain Python
loops on tiny inputs, by the closed forms (cos = 1, sin = 0 is the identity; a rotation keeps the norm
of every (i, i + R/2) pair; elements past R pass through) and by fp64 gradcheck of the hand-written
backward formulas the kernels implement.
"""
from __future__ import annotations

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, offset: bool = False) -> torch.Tensor:
    """F.rms_norm over the last dim: x * rsqrt(mean(x^2) + eps) * w, computed in fp32, returned in x.dtype."""
    xf = x.float()
    w = weight.float() + (1.0 if offset else 0.0)
    y = xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps) * w
    return y.to(x.dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    x1, x2 = x.chunk(2, dim=-1)
    return torch.cat((-x2, x1), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, eager_bf16: bool = False) -> torch.Tensor:
    """x (T, H, D); cos, sin (T, R), R <= D.  fp32 arithmetic with one rounding to x.dtype at the end, or -
    ``eager_bf16`` - the dtype of x after every multiply and add, as eager PyTorch evaluates the
    reference's expression when cos and sin were cast to the model dtype."""
    R = cos.shape[-1]
    xr, xp = x[..., :R], x[..., R:]
    c, s = cos[:, None, :], sin[:, None, :]
    if eager_bf16:
        c, s = c.to(x.dtype), s.to(x.dtype)
        out = (xr * c) + (rotate_half(xr) * s)
    else:
        wide = torch.promote_types(x.dtype, torch.float32)          # fp32, or fp64 for the gradient checks
        out = (xr.to(wide) * c.to(wide) + rotate_half(xr.to(wide)) * s.to(wide)).to(x.dtype)
    return torch.cat((out, xp), dim=-1) if xp.shape[-1] else out


def qk_norm_rope(q, k, qw, kw, cos, sin, eps: float = 1e-6, offset: bool = False, eager_bf16: bool = False):
    """q (T, Hq, D), k (T, Hkv, D) -> the (T, H, D) tensors the attention operator is called with."""
    qn, kn = rms_norm(q, qw, eps, offset), rms_norm(k, kw, eps, offset)
    return apply_rope(qn, cos, sin, eager_bf16).contiguous(), apply_rope(kn, cos, sin, eager_bf16).contiguous()


def sigmoid_gate(x: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(gate)


# ---- the backward formulas the kernels implement, written out (checked against autograd in fp64) ----
def rope_transpose(g: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Gradient of apply_rope w.r.t. its input: dn[i] = g[i] cos[i] + (i < R/2 ? g[i+R/2] sin[i+R/2] : -g[i-R/2] sin[i-R/2])."""
    R = cos.shape[-1]
    gr, gp = g[..., :R], g[..., R:]
    c, s = cos[:, None, :], sin[:, None, :]
    gs = gr * s
    g1, g2 = gs.chunk(2, dim=-1)
    dn = gr * c + torch.cat((g2, -g1), dim=-1)
    return torch.cat((dn, gp), dim=-1) if gp.shape[-1] else dn


def rms_norm_backward(dn: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float, offset: bool = False):
    """dx = rstd * (dn*w - xhat * mean(dn*w*xhat)),  dw = sum over rows of dn * xhat."""
    w = weight + (1.0 if offset else 0.0)
    rstd = torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)
    xh = x * rstd
    dx = rstd * (dn * w - xh * (dn * w * xh).mean(dim=-1, keepdim=True))
    dw = (dn * xh).reshape(-1, x.shape[-1]).sum(dim=0)
    return dx, dw
