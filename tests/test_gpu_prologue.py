"""GPU parity of the fused prologue / gate kernels (through the C ABI) against oracle/prologue_ref.py.

Tolerance: outputs are bf16, the oracle is fp32 arithmetic on the same bf16 inputs -> the bar of the
attention tests (|err| <= 2e-2 * max(1, |want|), cosine > 0.9995); the norm-weight gradients are fp32
sums over all rows and are compared relative to their scale."""
import pytest
import torch

from oracle import prologue_ref as P
from tests.util import assert_close_bf16
from vlm_training_amd import prologue

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _log(msg):
    print(msg, flush=True)


def _inputs(T, Hq, Hkv, D, R, seed, cs_dtype=torch.bfloat16, interleaved=False):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g)
    if interleaved:                                  # Qwen3.5: q_proj gives [q | gate] per head
        qg = (rn(T, Hq, 2 * D) * 1.5).bfloat16()
        q = qg[..., :D]
    else:
        q = (rn(T, Hq, D) * 1.5).bfloat16()
    k = (rn(T, Hkv, D) * 0.7).bfloat16()
    qw, kw = (rn(D) * 0.2 + 1).bfloat16(), (rn(D) * 0.2).bfloat16()
    pos = torch.arange(T, dtype=torch.float32)[:, None]
    inv = 1.0 / (10000.0 ** (torch.arange(0, R, 2, dtype=torch.float32) / max(R, 1)))
    ang = pos * inv[None, :]
    cos, sin = torch.cat((ang.cos(), ang.cos()), -1).to(cs_dtype), torch.cat((ang.sin(), ang.sin()), -1).to(cs_dtype)
    gq, gk = rn(T, Hq, D).bfloat16(), rn(T, Hkv, D).bfloat16()
    return q, k, qw, kw, cos, sin, gq, gk


@pytest.mark.parametrize("T,Hq,Hkv,D,R,offset,cs,inter", [
    (257, 32, 8, 128, 128, False, torch.bfloat16, False),     # Qwen3-VL-8B geometry, full rotary, odd T
    (64, 16, 2, 256, 64, True, torch.bfloat16, True),         # Qwen3.5: offset norm, partial rotary, interleaved q|gate
    (100, 6, 3, 64, 32, False, torch.float32, False),         # fp32 tables, heads not a multiple of the rows per wave
    (33, 5, 5, 128, 0, True, torch.bfloat16, False),          # no rotary part at all
])
def test_qk_norm_rope_forward_and_backward(T, Hq, Hkv, D, R, offset, cs, inter):
    _log(f"prologue T={T} Hq={Hq} Hkv={Hkv} D={D} R={R} offset={offset}")
    q, k, qw, kw, cos, sin, gq, gk = _inputs(T, Hq, Hkv, D, R, seed=T + D, cs_dtype=cs, interleaved=inter)
    # oracle: fp32 arithmetic on the same bf16 values, autograd for the gradients
    qf, kf = q.float().requires_grad_(True), k.float().requires_grad_(True)
    qwf, kwf = qw.float().requires_grad_(True), kw.float().requires_grad_(True)
    wq, wk = (qwf + 1, kwf + 1) if offset else (qwf, kwf)
    qn = qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + 1e-6) * wq
    kn = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + 1e-6) * wk
    rq, rk = P.apply_rope(qn, cos.float(), sin.float()), P.apply_rope(kn, cos.float(), sin.float())
    (rq * gq.float()).sum().backward(retain_graph=True)
    (rk * gk.float()).sum().backward()
    want_q, want_k = P.qk_norm_rope(q, k, qw, kw, cos, sin, 1e-6, offset)
    # HIP
    qd = q.to(DEV) if not inter else torch.cat((q, torch.zeros_like(q)), -1).to(DEV)[..., :D]
    qd = qd.detach().requires_grad_(True)
    kd = k.to(DEV).requires_grad_(True)
    qwd, kwd = qw.to(DEV).requires_grad_(True), kw.to(DEV).requires_grad_(True)
    oq, ok = prologue.qk_norm_rope(qd, kd, qwd, kwd, cos.to(DEV), sin.to(DEV), 1e-6, offset)
    assert oq.is_contiguous() and ok.is_contiguous() and oq.shape == (T, Hq, D)
    torch.autograd.backward((oq, ok), (gq.to(DEV), gk.to(DEV)))
    torch.cuda.synchronize()
    assert_close_bf16(oq, want_q, "q_out")
    assert_close_bf16(ok, want_k, "k_out")
    # the weights are read as the module holds them: fp32 parameters with the same values give the same bits
    with torch.no_grad():
        oq32, ok32 = prologue.qk_norm_rope(qd.detach(), kd.detach(), qw.float().to(DEV), kw.float().to(DEV), cos.to(DEV), sin.to(DEV),
                                           1e-6, offset)
    assert torch.equal(oq32, oq) and torch.equal(ok32, ok)
    # against an evaluation that never rounds: the reference (and the kernel, and `want_q` above) rounds F.rms_norm's
    # result to bf16 before the rotation, so the rotated value x*cos + rot(x)*sin carries up to (|cos| + |sin|)/2 <= 0.71
    # steps of that first rounding plus half a step of the final one - two bf16 steps bound it
    assert_close_bf16(oq, rq.detach(), "q_out vs fp32", steps=2)
    assert_close_bf16(qd.grad, qf.grad, "dq")
    assert_close_bf16(kd.grad, kf.grad, "dk")
    for name, got, want in (("dqw", qwd.grad, qwf.grad), ("dkw", kwd.grad, kwf.grad)):
        err = (got.float().cpu() - want).abs().max().item()
        assert err <= 2e-2 * max(1.0, want.abs().max().item()), (name, err, want.abs().max().item())


def test_qk_norm_rope_is_deterministic():
    q, k, qw, kw, cos, sin, gq, gk = (x.to(DEV) for x in _inputs(513, 8, 2, 128, 128, seed=3))
    outs = []
    for _ in range(2):
        a, b = (x.clone().requires_grad_(True) for x in (q, k))
        w1, w2 = (x.clone().requires_grad_(True) for x in (qw, kw))
        oq, ok = prologue.qk_norm_rope(a, b, w1, w2, cos, sin)
        torch.autograd.backward((oq, ok), (gq, gk))
        outs.append((oq.detach(), ok.detach(), a.grad, b.grad, w1.grad, w2.grad))
    for x, y in zip(*outs):
        assert torch.equal(x, y)


def test_sigmoid_gate_forward_and_backward_with_the_interleaved_gate():
    T, H, D = 130, 16, 256
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, H, D, generator=g).bfloat16()
    qg = (torch.randn(T, H, 2 * D, generator=g) * 2).bfloat16()
    gate = qg[..., D:]                               # the gate half of [q | gate], a strided view
    gy = torch.randn(T, H, D, generator=g).bfloat16()
    xf, gf = x.float().requires_grad_(True), gate.float().requires_grad_(True)
    want = P.sigmoid_gate(xf, gf)
    (want * gy.float()).sum().backward()
    xd = x.to(DEV).requires_grad_(True)
    qgd = qg.to(DEV).requires_grad_(True)
    y = prologue.sigmoid_gate(xd, qgd[..., D:])
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    assert_close_bf16(y, want.detach(), "gated out")
    assert_close_bf16(xd.grad, xf.grad, "dx")
    assert_close_bf16(qgd.grad[..., D:], gf.grad, "dgate")
    assert torch.count_nonzero(qgd.grad[..., :D]) == 0


def test_prologue_argument_errors():
    q, k, qw, kw, cos, sin, _, _ = (x.to(DEV) for x in _inputs(16, 4, 2, 128, 128, seed=1))
    with pytest.raises(ValueError):
        prologue.qk_norm_rope(q.float(), k, qw, kw, cos, sin)
    with pytest.raises(RuntimeError):
        prologue.qk_norm_rope(q, k, qw, kw, cos[:, :40].contiguous(), sin[:, :40].contiguous())   # R not a multiple of 16
    with pytest.raises(RuntimeError):
        prologue.qk_norm_rope(q.cpu(), k.cpu(), qw.cpu(), kw.cpu(), cos.cpu(), sin.cpu())
