"""The element-wise work either side of the attention operator, fused into single passes over HBM.

``qk_norm_rope``  replaces, in the reference's attention layers, ``q_norm(q)``/``k_norm(k)`` (F.rms_norm per
head), the transpose to (B, H, S, D), ``apply_rope``, the transpose back and the ``.contiguous()`` copies
(models/qwen3_vl/model.py:256-269; models/qwen3_5/model.py:110-129 with OffsetRMSNorm and a partial
rotary width): the projections' outputs go in as (T, H, D) *views* (any token / head stride, so the q
half of Qwen3.5's interleaved ``[q | gate]`` projection is read in place), the packed (T, H, D) tensors
the attention operator wants come out.  ``sigmoid_gate`` is ``out * torch.sigmoid(gate)``
(models/qwen3_5/model.py:135).  Both are ``torch.autograd.Function``s over the C ABI; there is no
fallback path.
"""
from __future__ import annotations

import torch

from . import _lib
from .ops import _ptr, _require_cuda, _stream


def _thd_strides(x, name):
    """(token stride, head stride) in elements of a (T, H, D) view whose last dim is contiguous."""
    if x.dim() != 3 or x.stride(2) != 1:
        raise ValueError(f"{name} must be a (T, H, D) view with a contiguous last dimension")
    if x.dtype != torch.bfloat16:
        raise ValueError(f"{name} must be bf16")
    return x.stride(0), x.stride(1)


def _cs(cos, sin, T):
    if cos.dim() == 3 and cos.shape[0] == 1:
        cos, sin = cos[0], sin[0]
    if cos.dim() != 2 or cos.shape != sin.shape or cos.shape[0] != T:
        raise ValueError("cos, sin must be (T, R) or (1, T, R)")
    if cos.dtype not in (torch.bfloat16, torch.float32) or sin.dtype != cos.dtype:
        raise ValueError("cos, sin must both be bf16 or both fp32")
    code = _lib.DSA_DTYPE_BF16 if cos.dtype == torch.bfloat16 else _lib.DSA_DTYPE_FP32
    return cos.contiguous(), sin.contiguous(), code


class _QkNormRope(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, q_weight, k_weight, cos, sin, eps, offset):
        _require_cuda(q, k, q_weight, k_weight, cos, sin)
        T, Hq, D = q.shape
        Hkv = k.shape[1]
        if k.shape[0] != T or k.shape[2] != D:
            raise ValueError(f"q/k shapes disagree: {tuple(q.shape)} {tuple(k.shape)}")
        (qt, qh), (kt, kh) = _thd_strides(q, "q"), _thd_strides(k, "k")
        cos, sin, cs_code = _cs(cos, sin, T)
        R = cos.shape[1]
        # the weights go in as the module holds them (fp32 master parameters, or bf16): a cast in front of the call would
        # be two more kernels per layer
        qw, kw = q_weight.detach().contiguous(), k_weight.detach().contiguous()
        if qw.dtype != kw.dtype or qw.dtype not in (torch.float32, torch.bfloat16):
            qw, kw = qw.float(), kw.float()
        if qw.numel() != D or kw.numel() != D:
            raise ValueError("norm weights must have head_dim elements")
        flags = (_lib.DSA_NORM_OFFSET if offset else 0) | (_lib.DSA_NORM_WEIGHT_BF16 if qw.dtype == torch.bfloat16 else 0)
        q_out = torch.empty((T, Hq, D), dtype=torch.bfloat16, device=q.device)
        k_out = torch.empty((T, Hkv, D), dtype=torch.bfloat16, device=q.device)
        q_rstd = torch.empty((T, Hq), dtype=torch.float32, device=q.device)
        k_rstd = torch.empty((T, Hkv), dtype=torch.float32, device=q.device)
        rc = _lib.load().dsa_qk_norm_rope_fwd(_ptr(q), qt, qh, _ptr(k), kt, kh, _ptr(qw), _ptr(kw), float(eps),
                                              flags, _ptr(cos), _ptr(sin), cs_code, R, T, Hq, Hkv, D,
                                              _ptr(q_out), _ptr(k_out), _ptr(q_rstd), _ptr(k_rstd), _stream(q.device))
        _lib.check(rc, "dsa_qk_norm_rope_fwd")
        ctx.save_for_backward(q, k, qw, kw, cos, sin, q_rstd, k_rstd)
        ctx.meta = (cs_code, R, flags, q_weight.dtype, k_weight.dtype)
        return q_out, k_out

    @staticmethod
    def backward(ctx, gq, gk):
        q, k, qw, kw, cos, sin, q_rstd, k_rstd = ctx.saved_tensors
        cs_code, R, flags, qw_dtype, kw_dtype = ctx.meta
        T, Hq, D = q.shape
        Hkv = k.shape[1]
        gq, gk = gq.contiguous().to(torch.bfloat16), gk.contiguous().to(torch.bfloat16)
        dq = torch.empty((T, Hq, D), dtype=torch.bfloat16, device=q.device)
        dk = torch.empty((T, Hkv, D), dtype=torch.bfloat16, device=q.device)
        dqw = torch.empty((D,), dtype=torch.float32, device=q.device)
        dkw = torch.empty((D,), dtype=torch.float32, device=q.device)
        lib = _lib.load()
        ws_bytes = lib.dsa_qk_norm_rope_bwd_workspace_bytes(T, D)
        ws = torch.empty((max(ws_bytes, 4),), dtype=torch.uint8, device=q.device)
        rc = lib.dsa_qk_norm_rope_bwd(_ptr(gq), _ptr(gk), _ptr(q), q.stride(0), q.stride(1), _ptr(k), k.stride(0),
                                      k.stride(1), _ptr(qw), _ptr(kw), flags, _ptr(cos), _ptr(sin), cs_code,
                                      R, _ptr(q_rstd), _ptr(k_rstd), T, Hq, Hkv, D, _ptr(dq), Hq * D, D, _ptr(dk), Hkv * D,
                                      D, _ptr(dqw), _ptr(dkw), _ptr(ws), ws_bytes, _stream(q.device))
        _lib.check(rc, "dsa_qk_norm_rope_bwd")
        return dq, dk, dqw.to(qw_dtype), dkw.to(kw_dtype), None, None, None, None


@torch.compiler.disable
def qk_norm_rope(q, k, q_weight, k_weight, cos, sin, eps: float = 1e-6, offset: bool = False):
    """q (T, Hq, D), k (T, Hkv, D) bf16 views -> rope(rms_norm(q)), rope(rms_norm(k)) as contiguous (T, H, D).

    ``offset=True`` scales by ``1 + weight`` (OffsetRMSNorm).  cos, sin: (T, R) or (1, T, R), R <= D a
    multiple of 16 (elements past R pass through unrotated)."""
    return _QkNormRope.apply(q, k, q_weight, k_weight, cos, sin, float(eps), bool(offset))


class _SigmoidGate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, gate):
        _require_cuda(x, gate)
        if x.dim() != 3 or not x.is_contiguous() or x.dtype != torch.bfloat16:
            raise ValueError("x must be a contiguous bf16 (T, H, D) tensor")
        if gate.shape != x.shape:
            raise ValueError("gate must have the shape of x")
        gt, gh = _thd_strides(gate, "gate")
        T, H, D = x.shape
        y = torch.empty_like(x)
        rc = _lib.load().dsa_sigmoid_gate_fwd(_ptr(x), _ptr(gate), gt, gh, T, H, D, _ptr(y), _stream(x.device))
        _lib.check(rc, "dsa_sigmoid_gate_fwd")
        ctx.save_for_backward(x, gate)
        return y

    @staticmethod
    def backward(ctx, gy):
        x, gate = ctx.saved_tensors
        T, H, D = x.shape
        gy = gy.contiguous().to(torch.bfloat16)
        dx, dgate = torch.empty_like(x), torch.empty_like(x)
        rc = _lib.load().dsa_sigmoid_gate_bwd(_ptr(gy), _ptr(x), _ptr(gate), gate.stride(0), gate.stride(1), T, H, D, _ptr(dx),
                                              _ptr(dgate), H * D, D, _stream(x.device))
        _lib.check(rc, "dsa_sigmoid_gate_bwd")
        return dx, dgate


@torch.compiler.disable
def sigmoid_gate(x, gate):
    """``x * torch.sigmoid(gate)`` for x (T, H, D) contiguous and gate a (T, H, D) view (strided allowed)."""
    return _SigmoidGate.apply(x, gate)
