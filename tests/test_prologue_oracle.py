"""Pins oracle/prologue_ref.py (no GPU): library routine, loops, closed forms, gradcheck."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import prologue_ref as P


def _rand(*shape, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype)


@pytest.mark.parametrize("offset", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rms_norm_is_the_library_routine(offset, dtype):
    x, w = _rand(5, 3, 64, seed=1, dtype=dtype), _rand(64, seed=2, dtype=dtype)
    want = F.rms_norm(x, (64,), (1.0 + w) if offset else w, 1e-6)
    got = P.rms_norm(x, w, 1e-6, offset)
    assert got.dtype == dtype
    assert torch.allclose(got.float(), want.float(), atol=1e-6 if dtype == torch.float32 else 2e-2, rtol=1e-6 if dtype == torch.float32 else 1e-2)


def test_rms_norm_against_a_python_loop():
    x, w = _rand(3, 2, 8, seed=3), _rand(8, seed=4)
    got = P.rms_norm(x, w, 1e-5)
    for t in range(3):
        for h in range(2):
            row = x[t, h].tolist()
            r = 1.0 / math.sqrt(sum(v * v for v in row) / 8 + 1e-5)
            for d in range(8):
                assert abs(got[t, h, d].item() - row[d] * r * w[d].item()) < 1e-5


def test_rope_against_a_python_loop_with_partial_rotary_width():
    T, H, D, R = 4, 2, 16, 8
    x = _rand(T, H, D, seed=5)
    ang = _rand(T, R // 2, seed=6)
    cos, sin = torch.cat((ang.cos(), ang.cos()), -1), torch.cat((ang.sin(), ang.sin()), -1)
    got = P.apply_rope(x, cos, sin)
    for t in range(T):
        for h in range(H):
            for d in range(D):
                if d >= R:
                    want = x[t, h, d].item()
                elif d < R // 2:
                    want = x[t, h, d].item() * cos[t, d].item() - x[t, h, d + R // 2].item() * sin[t, d].item()
                else:
                    want = x[t, h, d].item() * cos[t, d].item() + x[t, h, d - R // 2].item() * sin[t, d].item()
                assert abs(got[t, h, d].item() - want) < 1e-5


def test_rope_closed_forms():
    T, H, D = 6, 3, 32
    x = _rand(T, H, D, seed=7)
    ident = P.apply_rope(x, torch.ones(T, D), torch.zeros(T, D))
    assert torch.equal(ident, x)
    ang = _rand(T, D // 2, seed=8)
    cos, sin = torch.cat((ang.cos(), ang.cos()), -1), torch.cat((ang.sin(), ang.sin()), -1)
    y = P.apply_rope(x, cos, sin)
    # a rotation of every (i, i + D/2) pair: pair norms are kept, and the inverse angle undoes it
    n0 = x[..., :D // 2] ** 2 + x[..., D // 2:] ** 2
    n1 = y[..., :D // 2] ** 2 + y[..., D // 2:] ** 2
    assert torch.allclose(n0, n1, atol=1e-5)
    assert torch.allclose(P.apply_rope(y, cos, -sin), x, atol=1e-5)
    # quarter turn: (a, b) -> (-b, a)
    q = P.apply_rope(x, torch.zeros(T, D), torch.ones(T, D))
    assert torch.allclose(q, P.rotate_half(x))


def test_eager_bf16_chain_stays_within_bf16_steps_of_the_fp32_form():
    T, H, D = 64, 4, 128
    x = _rand(T, H, D, seed=9, dtype=torch.bfloat16)
    ang = _rand(T, D // 2, seed=10) * 3
    cos, sin = torch.cat((ang.cos(), ang.cos()), -1), torch.cat((ang.sin(), ang.sin()), -1)
    a = P.apply_rope(x, cos.bfloat16(), sin.bfloat16(), eager_bf16=True).float()
    b = P.apply_rope(x, cos.bfloat16(), sin.bfloat16(), eager_bf16=False).float()
    assert (a - b).abs().max().item() <= 3 * 2 ** -8 * max(1.0, b.abs().max().item())


@pytest.mark.parametrize("offset", [False, True])
def test_backward_formulas_match_autograd_in_fp64(offset):
    T, Hq, Hkv, D, R = 5, 4, 2, 16, 8
    dd = torch.float64
    q, k = _rand(T, Hq, D, seed=11).to(dd).requires_grad_(True), _rand(T, Hkv, D, seed=12).to(dd).requires_grad_(True)
    qw, kw = _rand(D, seed=13).to(dd).requires_grad_(True), _rand(D, seed=14).to(dd).requires_grad_(True)
    ang = _rand(T, R // 2, seed=15).to(dd)
    cos, sin = torch.cat((ang.cos(), ang.cos()), -1), torch.cat((ang.sin(), ang.sin()), -1)

    def f(q, k, qw, kw):
        w1, w2 = (qw + 1, kw + 1) if offset else (qw, kw)
        qn = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + 1e-6) * w1
        kn = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + 1e-6) * w2
        return P.apply_rope(qn, cos, sin), P.apply_rope(kn, cos, sin)

    assert torch.autograd.gradcheck(lambda *a: f(*a), (q, k, qw, kw), eps=1e-6, atol=1e-6)
    gq, gk = _rand(T, Hq, D, seed=16).to(dd), _rand(T, Hkv, D, seed=17).to(dd)
    yq, yk = f(q, k, qw, kw)
    want = torch.autograd.grad((yq * gq).sum() + (yk * gk).sum(), (q, k, qw, kw))
    dxq, dwq = P.rms_norm_backward(P.rope_transpose(gq, cos, sin), q.detach(), qw.detach(), 1e-6, offset)
    dxk, dwk = P.rms_norm_backward(P.rope_transpose(gk, cos, sin), k.detach(), kw.detach(), 1e-6, offset)
    for got, w in zip((dxq, dxk, dwq, dwk), want):
        assert torch.allclose(got, w, atol=1e-9)


def test_sigmoid_gate_is_out_times_sigmoid():
    x, g = _rand(7, 4, 16, seed=18), _rand(7, 4, 16, seed=19)
    want = x * (1 / (1 + torch.exp(-g)))
    assert torch.allclose(P.sigmoid_gate(x, g), want, atol=1e-6)
