"""GPU parity of the attention layers (torch GEMM projections around the HIP operator) against the CPU oracle of the
reference's layers, forward and every parameter gradient; and the installed forwards against the HF modules' own.

Layer-level tolerance: the values pass through several bf16 GEMMs on the device (the reference's own layer tests allow
atol 0.5 / rtol 0.1 on bf16 logits, models/tests/test_qwen3_5_exhaustive.py:84-88); here every tensor must agree with
the fp32 oracle to cosine > 0.9995 and max-abs <= 2e-2 of the tensor's largest magnitude."""
from types import SimpleNamespace

import pytest
import torch

from oracle import layer_ref as LR
from tests.util import cosine
from vlm_training_amd import DsaConfig, Qwen3VLTextAttention, SelfAttention, indexer_losses, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _log(msg):
    print(msg, flush=True)


def _close(got, want, name, rel=2e-2, min_cos=0.9995):
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    assert got.shape == want.shape, (name, got.shape, want.shape)
    assert torch.isfinite(got).all(), name
    err, ref = (got - want).abs().max().item(), want.abs().max().item()
    cos = cosine(got, want)
    assert err <= rel * ref + 1e-6 and cos > min_cos, f"{name}: max-abs {err:.4g} vs largest |want| {ref:.4g}, cosine {cos:.6f}"
    return err, cos


def _cfg(hidden, Hq, Hkv, D):
    return SimpleNamespace(hidden_size=hidden, num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D, rms_norm_eps=1e-6)


def _tables(T, R, dtype):
    inv = 1.0 / (1e6 ** (torch.arange(0, R, 2, dtype=torch.float32) / R))
    ang = torch.outer(torch.arange(T, dtype=torch.float32), inv)
    emb = torch.cat((ang, ang), -1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def _make(cls, cfg, dsa, seed, param_dtype):
    torch.manual_seed(seed)
    m = cls(cfg, dsa=dsa)
    with torch.no_grad():                                  # norms away from their trivial initial values
        m.q_norm.weight.add_(torch.randn_like(m.q_norm.weight) * 0.2)
        m.k_norm.weight.add_(torch.randn_like(m.k_norm.weight) * 0.2)
        for p in m.parameters():                           # the oracle reads the very values the device holds
            p.copy_(p.to(torch.bfloat16).float())
    return m.to(DEV).to(param_dtype)


def _oracle_args(m, x_cpu, cos, sin, cu):
    f = lambda p: p.detach().float().cpu().clone().requires_grad_(True)
    w = [f(m.q_proj.weight), f(m.k_proj.weight), f(m.v_proj.weight), f(m.o_proj.weight), f(m.q_norm.weight), f(m.k_norm.weight)]
    return w, (x_cpu, *w, cos.float().cpu(), sin.float().cpu(), cu)


@pytest.mark.parametrize("kind,hidden,Hq,Hkv,D,R,param_dtype", [
    ("qwen3vl", 256, 8, 2, 128, 128, torch.bfloat16),
    ("qwen3vl", 192, 6, 2, 64, 64, torch.float32),        # fp32 parameters under bf16 autocast, as the trainer runs
    ("qwen3_5", 256, 4, 1, 256, 64, torch.bfloat16),      # gated, (1 + w) norms, partial rotary
])
def test_dense_layers_match_the_reference_layer_oracle(kind, hidden, Hq, Hkv, D, R, param_dtype):
    _log(f"layer {kind} {Hq}/{Hkv}/{D} R={R} {param_dtype}")
    cu = [0, 300, 300, 812, 1024]
    T = cu[-1]
    cls = Qwen3VLTextAttention if kind == "qwen3vl" else SelfAttention
    m = _make(cls, _cfg(hidden, Hq, Hkv, D), None, seed=7, param_dtype=param_dtype)
    g = torch.Generator().manual_seed(8)
    x_cpu = torch.randn(1, T, hidden, generator=g).bfloat16().float()
    gy_cpu = torch.randn(1, T, hidden, generator=g).bfloat16().float()
    cos, sin = _tables(T, R, torch.float32)
    x = x_cpu.to(DEV).to(torch.bfloat16).requires_grad_(True)
    cu_d = torch.tensor(cu, dtype=torch.int32, device=DEV)
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=param_dtype == torch.float32):
        y = m(x, cos.to(DEV), sin.to(DEV), cu_d, 512)
    assert y.shape == (1, T, hidden) and m.indexer_loss is None
    y.backward(gy_cpu.to(DEV).to(y.dtype))
    xr = x_cpu.clone().requires_grad_(True)
    w, args = _oracle_args(m, xr, cos, sin, cu)
    fn = LR.qwen3vl_attention if kind == "qwen3vl" else LR.qwen3_5_attention
    ref = fn(*args, D, 1e-6)
    ref.backward(gy_cpu)
    res = [_close(y, ref, "out"), _close(x.grad, xr.grad, "dx")]
    for name, p, wr in zip(("q_proj", "k_proj", "v_proj", "o_proj", "q_norm", "k_norm"),
                           (m.q_proj.weight, m.k_proj.weight, m.v_proj.weight, m.o_proj.weight, m.q_norm.weight, m.k_norm.weight), w):
        res.append(_close(p.grad, wr.grad, f"d{name}"))
    _log("  " + " ".join(f"({e:.2e},{c:.6f})" for e, c in res))


@pytest.mark.parametrize("kind,top_k", [("qwen3vl", 64), ("qwen3_5", 48), ("qwen3vl", 4096)])
def test_dsa_layers_match_the_oracle_output_loss_and_every_gradient(kind, top_k):
    """A layer that owns its indexer: output and indexer loss against the oracle on the layer's own selection
    (checked bit-exact elsewhere), gradients of the main weights from the output and of the indexer's projections from
    the loss.  top_k beyond the longest segment must give the dense layer."""
    _log(f"dsa layer {kind} top_k={top_k}")
    hidden, Hq, Hkv, D, R = (256, 8, 2, 128, 128) if kind == "qwen3vl" else (256, 4, 1, 256, 64)
    Hi, Di = 8, 64
    cu = [0, 300, 700, 1024]
    T = cu[-1]
    cls = Qwen3VLTextAttention if kind == "qwen3vl" else SelfAttention
    dsa = DsaConfig(index_heads=Hi, index_dim=Di, top_k=top_k)
    m = _make(cls, _cfg(hidden, Hq, Hkv, D), dsa, seed=17, param_dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(18)
    x_cpu = torch.randn(1, T, hidden, generator=g).bfloat16().float()
    gy_cpu = torch.randn(1, T, hidden, generator=g).bfloat16().float()
    cos, sin = _tables(T, R, torch.float32)
    x = x_cpu.to(DEV).to(torch.bfloat16).requires_grad_(True)
    cu_d = torch.tensor(cu, dtype=torch.int32, device=DEV)
    y = m(x, cos.to(DEV), sin.to(DEV), cu_d, 512)
    loss = indexer_losses(m)
    assert loss is not None and loss.dim() == 0 and loss is m.indexer_loss
    torch.autograd.backward((y, loss * 5.0), (gy_cpu.to(DEV).to(y.dtype), None))
    # the layer's selection: the same deterministic call on the same indexer outputs
    with torch.no_grad():
        iq, ik, iw = m.indexer(x)
        idx, n = ops.index_topk(iq, ik, iw, cu_d, 512, top_k)
    xr = x_cpu.clone().requires_grad_(True)
    w, args = _oracle_args(m, xr, cos, sin, cu)
    f = lambda p: p.detach().float().cpu().clone().requires_grad_(True)
    wi = [f(m.indexer.q_proj.weight), f(m.indexer.k_proj.weight), f(m.indexer.w_proj.weight)]
    ref_y, ref_loss, _ = LR.dsa_layer(*args, D, *wi, Hi, Di, idx.cpu(), n.cpu(), gated=kind == "qwen3_5")
    torch.autograd.backward((ref_y, ref_loss * 5.0), (gy_cpu, None))
    res = [_close(y, ref_y, "out"), _close(x.grad, xr.grad, "dx")]
    assert abs(loss.item() - ref_loss.item()) <= 2e-3 * max(1.0, abs(ref_loss.item())), (loss.item(), ref_loss.item())
    for name, p, wr in zip(("q_proj", "k_proj", "v_proj", "o_proj", "q_norm", "k_norm"),
                           (m.q_proj.weight, m.k_proj.weight, m.v_proj.weight, m.o_proj.weight, m.q_norm.weight, m.k_norm.weight), w):
        res.append(_close(p.grad, wr.grad, f"d{name}"))
    for name, p, wr in zip(("iq", "ik", "iw"), (m.indexer.q_proj.weight, m.indexer.k_proj.weight, m.indexer.w_proj.weight), wi):
        if wr.grad.abs().max() > 0:
            # The indexer's gradient passes the ReLU gate [q_idx.k_idx > 0], which is discontinuous: the device rounds the
            # projections' outputs to bf16, the oracle does not, so a fraction of a percent of the gates near zero fall on
            # the other side and each moves its term by its full size.  Hence a wider bar than for the smooth paths.
            res.append(_close(p.grad, wr.grad, f"d{name}", rel=1e-1, min_cos=0.998))
    _log(f"  loss {loss.item():.5f} (oracle {ref_loss.item():.5f}) " + " ".join(f"({e:.2e},{c:.6f})" for e, c in res))
    if top_k >= 512:                                       # the whole window is selected: the dense layer, bit for bit
        dense = _make(cls, _cfg(hidden, Hq, Hkv, D), None, seed=17, param_dtype=torch.bfloat16)
        dense.load_state_dict({k_: v_ for k_, v_ in m.state_dict().items() if not k_.startswith("indexer.")})
        with torch.no_grad():
            assert torch.equal(dense(x, cos.to(DEV), sin.to(DEV), cu_d, 512), y)
    with torch.no_grad():                                  # no loss is built when nothing can train on it
        m(x, cos.to(DEV), sin.to(DEV), cu_d, 512)
        assert m.indexer_loss is None


def test_installed_forward_equals_the_hf_module_on_a_packed_row():
    """train/model_attention.py:265-299 installs the forwards on the HF classes.  Here: an HF Qwen3Attention with
    random weights, its own eager forward under a block-diagonal causal mask against the installed forward fed the
    cu_seqlens, same module, same inputs."""
    _log("HF installer")
    import vlm_training_amd as M
    from transformers.models.qwen3 import modeling_qwen3 as hf
    cfg = hf.Qwen3Config(hidden_size=256, num_attention_heads=8, num_key_value_heads=2, head_dim=64, intermediate_size=512,
                         num_hidden_layers=1, vocab_size=128, rms_norm_eps=1e-6, attention_dropout=0.0)
    cfg._attn_implementation = "eager"
    torch.manual_seed(3)
    attn = hf.Qwen3Attention(cfg, layer_idx=0).to(DEV).to(torch.bfloat16).eval()
    with torch.no_grad():
        attn.q_norm.weight.add_(torch.randn_like(attn.q_norm.weight) * 0.2)
    cu = [0, 200, 333, 512]
    T = cu[-1]
    g = torch.Generator().manual_seed(4)
    x = torch.randn(1, T, 256, generator=g).bfloat16().to(DEV)
    cos, sin = (t[None].to(DEV).to(torch.bfloat16) for t in _tables(T, 64, torch.float32))
    seg = torch.zeros(T, dtype=torch.long)
    for i, (a, b) in enumerate(zip(cu[:-1], cu[1:])):
        seg[a:b] = i
    allowed = (seg[:, None] == seg[None, :]) & (torch.arange(T)[:, None] >= torch.arange(T)[None, :])
    mask = torch.zeros(T, T).masked_fill(~allowed, float("-inf"))[None, None].to(DEV).to(torch.bfloat16)
    with torch.no_grad():
        want, _ = attn(x, (cos, sin), mask)
    undo = M.replace_attention_qwenvl()
    try:
        with torch.no_grad():
            got, none = attn(x, (cos, sin), M.return_mask(torch.tensor(cu, dtype=torch.int32, device=DEV)))
    finally:
        for owner, name, old in reversed(undo):
            setattr(owner, name, old)
    assert none is None and got.shape == want.shape
    e, c = _close(got, want, "installed forward vs HF eager")
    _log(f"  ({e:.2e},{c:.6f})")
