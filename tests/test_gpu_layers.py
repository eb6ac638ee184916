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
    ref_y, ref_loss, _ = LR.dsa_layer(*args, D, *wi, Hi, Di, idx.cpu(), n.cpu(), gated=kind == "qwen3_5",
                                      round_indexer_to_bf16=True)
    torch.autograd.backward((ref_y, ref_loss * 5.0), (gy_cpu, None))
    res = [_close(y, ref_y, "out"), _close(x.grad, xr.grad, "dx")]
    assert abs(loss.item() - ref_loss.item()) <= 2e-3 * max(1.0, abs(ref_loss.item())), (loss.item(), ref_loss.item())
    for name, p, wr in zip(("q_proj", "k_proj", "v_proj", "o_proj", "q_norm", "k_norm"),
                           (m.q_proj.weight, m.k_proj.weight, m.v_proj.weight, m.o_proj.weight, m.q_norm.weight, m.k_norm.weight), w):
        res.append(_close(p.grad, wr.grad, f"d{name}"))
    for name, p, wr in zip(("iq", "ik", "iw"), (m.indexer.q_proj.weight, m.indexer.k_proj.weight, m.indexer.w_proj.weight), wi):
        if wr.grad.abs().max() > 0:
            # the oracle rounds the indexer's projections to bf16 as the device does (round_indexer_to_bf16), so that both
            # open the same ReLU gates [q_idx.k_idx > 0]; what is left is the bf16 arithmetic of the kernels
            res.append(_close(p.grad, wr.grad, f"d{name}"))     # the same bar as every other tensor (observed cosine 0.99998)
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


def _block_causal_mask(cu, T, dtype):
    seg = torch.zeros(T, dtype=torch.long)
    for i, (a, b) in enumerate(zip(cu[:-1], cu[1:])):
        seg[a:b] = i
    allowed = (seg[:, None] == seg[None, :]) & (torch.arange(T)[:, None] >= torch.arange(T)[None, :])
    return torch.zeros(T, T).masked_fill(~allowed, float("-inf"))[None, None].to(DEV).to(dtype)


def _restore(undo):
    for owner, name, old in reversed(undo):
        setattr(owner, name, old)


@pytest.mark.parametrize("D,R", [(256, 64), (128, 128)])
def test_installed_gated_forward_equals_the_hf_qwen3_5_module_on_a_packed_row(D, R):
    """train/model_attention.py:146-185: the gated forward the installer puts on HF's Qwen3_5Attention ([q | gate]
    per head, (1 + weight) norms, partial rotary through HF's own apply_rotary_pos_emb, * sigmoid(gate)).  The HF
    module's eager forward under a block-diagonal causal mask against the installed forward fed the cu_seqlens - same
    module, same inputs, forward and the gradient of the input."""
    _log(f"HF installer, Qwen3.5 gated forward, head_dim {D}, rotary width {R}")
    import vlm_training_amd as M
    from transformers.models.qwen3_5 import modeling_qwen3_5 as hf
    cfg = hf.Qwen3_5TextConfig(hidden_size=256, num_attention_heads=4, num_key_value_heads=1, head_dim=D,
                               intermediate_size=512, num_hidden_layers=1, vocab_size=128, rms_norm_eps=1e-6,
                               attention_dropout=0.0)
    cfg._attn_implementation = "eager"
    torch.manual_seed(5)
    attn = hf.Qwen3_5Attention(cfg, layer_idx=0).to(DEV).to(torch.bfloat16).eval()
    with torch.no_grad():                                  # the norms' weights start at zero: move them
        attn.q_norm.weight.add_(torch.randn_like(attn.q_norm.weight) * 0.2)
        attn.k_norm.weight.add_(torch.randn_like(attn.k_norm.weight) * 0.2)
    cu = [0, 200, 200, 333, 512]
    T = cu[-1]
    g = torch.Generator().manual_seed(6)
    x_cpu = torch.randn(1, T, 256, generator=g).bfloat16()
    gy = torch.randn(1, T, 256, generator=g).bfloat16().to(DEV)
    cos, sin = (t[None].to(DEV).to(torch.bfloat16) for t in _tables(T, R, torch.float32))
    mask = _block_causal_mask(cu, T, torch.bfloat16)
    x1 = x_cpu.to(DEV).requires_grad_(True)
    want, _ = attn(x1, (cos, sin), mask)
    want.backward(gy)
    undo = M.replace_attention_qwenvl()
    try:
        assert type(attn).forward is M.qwen3_5_forward
        x2 = x_cpu.to(DEV).requires_grad_(True)
        got, none = attn(x2, (cos, sin), M.return_mask(torch.tensor(cu, dtype=torch.int32, device=DEV)))
        got.backward(gy)
    finally:
        _restore(undo)
    assert none is None and got.shape == want.shape
    res = [_close(got, want, "installed gated forward vs HF eager"), _close(x2.grad, x1.grad, "dx")]
    _log("  " + " ".join(f"({e:.2e},{c:.6f})" for e, c in res))


def test_installed_forward_reads_the_bound_of_every_new_offsets_tensor():
    """The installed forwards take the longest segment from the offsets tensor they are handed
    (train/model_attention.py:118-121 reads it every call).  Two packed rows in turn, equal in segment count, the
    second with a longer longest segment, its offsets tensor allocated after the first was freed (the caching allocator
    hands out the same block): with a DSA indexer on the module the bound sizes the score rows and the bitmap, so a
    bound kept from the first row would clip the second.  Both against the oracle on the module's own selection."""
    _log("HF installer with an indexer, two packed rows in turn")
    import vlm_training_amd as M
    from transformers.models.qwen3 import modeling_qwen3 as hf
    hidden, Hq, Hkv, D, Hi, Di, top_k = 256, 8, 2, 64, 8, 64, 48
    cfg = hf.Qwen3Config(hidden_size=hidden, num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D,
                         intermediate_size=512, num_hidden_layers=1, vocab_size=128, rms_norm_eps=1e-6, attention_dropout=0.0)
    torch.manual_seed(9)
    attn = hf.Qwen3Attention(cfg, layer_idx=0)
    attn.indexer = M.DsaIndexer(hidden, DsaConfig(index_heads=Hi, index_dim=Di, top_k=top_k))
    with torch.no_grad():
        for p in attn.parameters():
            p.copy_(p.to(torch.bfloat16).float())
    attn = attn.to(DEV).to(torch.bfloat16).eval()
    T = 512
    g = torch.Generator().manual_seed(10)
    x_cpu = torch.randn(1, T, hidden, generator=g).bfloat16().float()
    x = x_cpu.to(DEV).to(torch.bfloat16)
    cos, sin = (t.bfloat16().float() for t in _tables(T, D, torch.float32))      # the oracle reads the tables the device holds
    pe = (cos[None].to(DEV).to(torch.bfloat16), sin[None].to(DEV).to(torch.bfloat16))
    undo = M.replace_attention_qwenvl()
    ptrs = []
    try:
        for cu in ([0, 100, 260, 512], [0, 430, 460, 512]):          # longest 252, then 430
            cu_d = torch.tensor(cu, dtype=torch.int32, device=DEV)
            ptrs.append(cu_d.data_ptr())
            with torch.no_grad():
                got, _ = attn(x, pe, M.return_mask(cu_d))
                iq, ik, iw = attn.indexer(x)
                idx, n = ops.index_topk(iq, ik, iw, cu_d.reshape(-1), max(b - a for a, b in zip(cu[:-1], cu[1:])), top_k)
            f = lambda p: p.detach().float().cpu()
            want, _, _ = LR.dsa_layer(x_cpu, f(attn.q_proj.weight), f(attn.k_proj.weight), f(attn.v_proj.weight),
                                      f(attn.o_proj.weight), f(attn.q_norm.weight), f(attn.k_norm.weight), cos, sin, cu, D,
                                      f(attn.indexer.q_proj.weight), f(attn.indexer.k_proj.weight),
                                      f(attn.indexer.w_proj.weight), Hi, Di, idx.cpu(), n.cpu())
            e, c = _close(got, want, f"installed DSA forward, offsets {cu}")
            _log(f"  offsets {cu}: ({e:.2e},{c:.6f})")
            del cu_d, got
    finally:
        _restore(undo)
    _log(f"  the second offsets tensor {'reused' if ptrs[0] == ptrs[1] else 'did not reuse'} the first one's address")


def _one_rank_cuda_mesh():
    """A one-rank device mesh on the GPU over torch's fake process group: DTensors work, no collective ever runs."""
    import torch.distributed as dist
    from torch.distributed.device_mesh import init_device_mesh
    from torch.testing._internal.distributed.fake_pg import FakeStore
    created = False
    if not dist.is_initialized():
        dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=1)
        created = True
    return init_device_mesh("cuda", (1,)), created


@pytest.mark.parametrize("kind", ["qwen3_5", "qwen3vl", "hf_qwen3"])
def test_head_sharded_dtensor_projections_pass_through_layer_kernel_and_rewrap(kind, monkeypatch):
    """models/qwen3_5/model.py:124,132 and train/infra.py:446-451: under tensor parallelism q/k/v_proj are column
    parallel with DTensor outputs (sharded by head), the kernels see the local shards, and the kernel's output goes
    back under the same mesh and placements before the row-parallel o_proj.  One rank, so the local shard is the whole
    tensor: the parallelised layer must equal the plain one bit for bit, forward and input gradient."""
    _log(f"DTensor projections through the layer: {kind}")
    import copy

    import torch.distributed as dist
    from torch.distributed.tensor import DTensor, Replicate, Shard
    from torch.distributed.tensor.parallel import ColwiseParallel, RowwiseParallel, SequenceParallel, parallelize_module

    import vlm_training_amd as M
    from vlm_training_amd import layers as L, model_attention as MA
    hidden, T, cu = 256, 512, [0, 200, 333, 512]
    torch.manual_seed(21)
    undo = []
    if kind == "hf_qwen3":
        from transformers.models.qwen3 import modeling_qwen3 as hf
        cfg = hf.Qwen3Config(hidden_size=hidden, num_attention_heads=8, num_key_value_heads=2, head_dim=64,
                             intermediate_size=512, num_hidden_layers=1, vocab_size=128, rms_norm_eps=1e-6, attention_dropout=0.0)
        plain = hf.Qwen3Attention(cfg, layer_idx=0).to(DEV).to(torch.bfloat16).eval()
        R = 64
        undo = M.replace_attention_qwenvl()
    else:
        cls, (Hq, Hkv, D, R) = (SelfAttention, (4, 1, 256, 64)) if kind == "qwen3_5" else (Qwen3VLTextAttention, (8, 2, 128, 128))
        plain = _make(cls, _cfg(hidden, Hq, Hkv, D), None, seed=21, param_dtype=torch.bfloat16)
    mesh, created = _one_rank_cuda_mesh()
    seen = []
    real_rewrap = L._dtensor_rewrap

    def spy(tensor, wrap_info):
        out = real_rewrap(tensor, wrap_info)
        seen.append((wrap_info, out))
        return out

    monkeypatch.setattr(L, "_dtensor_rewrap", spy)
    import vlm_training_amd.dtensor_utils as DU
    monkeypatch.setattr(DU, "_dtensor_rewrap", spy)          # the HF forwards import it at call time
    try:
        tp = copy.deepcopy(plain)
        parallelize_module(tp, mesh, {
            "q_proj": ColwiseParallel(use_local_output=False), "k_proj": ColwiseParallel(use_local_output=False),
            "v_proj": ColwiseParallel(use_local_output=False), "q_norm": SequenceParallel(sequence_dim=2),
            "k_norm": SequenceParallel(sequence_dim=2), "o_proj": RowwiseParallel(output_layouts=Replicate())},
            src_data_rank=None)                              # shards are taken from the local copy: nothing is scattered
        assert isinstance(tp.q_proj.weight, DTensor) and isinstance(tp.q_norm.weight, DTensor)
        for name, p in tp.named_parameters():
            assert torch.equal(p.to_local(), plain.get_parameter(name)), name
        g = torch.Generator().manual_seed(22)
        x_cpu = torch.randn(1, T, hidden, generator=g).bfloat16()
        gy = torch.randn(1, T, hidden, generator=g).bfloat16().to(DEV)
        cos, sin = (t.to(DEV).to(torch.bfloat16) for t in _tables(T, R, torch.float32))
        outs, grads = [], []
        for m in (plain, tp):
            x = x_cpu.to(DEV).requires_grad_(True)
            cu_d = torch.tensor(cu, dtype=torch.int32, device=DEV)
            if kind == "hf_qwen3":
                y, _ = m(x, (cos[None], sin[None]), MA.return_mask(cu_d))
            else:
                y = m(x, cos, sin, cu_d, 256)
            y = y.to_local() if isinstance(y, DTensor) else y
            y.backward(gy)
            outs.append(y.detach())
            grads.append(x.grad)
        assert torch.equal(outs[0], outs[1]) and torch.equal(grads[0], grads[1])
        wraps = [(w, o) for w, o in seen if w is not None]
        assert len(wraps) == 1 and len(seen) == 2            # the plain layer's call wrapped nothing
        (w_mesh, w_place), rewrapped = wraps[0]
        assert isinstance(rewrapped, DTensor) and rewrapped.device_mesh == mesh and w_mesh == mesh
        assert tuple(rewrapped.placements) == tuple(w_place) == (Shard(1),)      # (T, heads, head_dim): sharded by head
        assert rewrapped.to_local().is_cuda
    finally:
        _restore(undo)
        if created:
            dist.destroy_process_group()


@pytest.mark.parametrize("sparse", [False, True])
def test_layer_under_activation_checkpointing_recomputes_to_the_same_bits(sparse):
    """train/infra.py:187-195 wraps every block in torch's checkpoint wrapper: the forward runs a second time inside the
    backward.  The operator keeps no state between calls and is deterministic, so a checkpointed layer must give the
    output and the gradients of the plain one bit for bit (the selection included: it is recomputed, not saved)."""
    _log(f"activation checkpointing, sparse={sparse}")
    from torch.utils.checkpoint import checkpoint
    hidden, Hq, Hkv, D = 256, 8, 2, 128
    dsa = DsaConfig(index_heads=8, index_dim=64, top_k=64) if sparse else None
    m = _make(Qwen3VLTextAttention, _cfg(hidden, Hq, Hkv, D), dsa, seed=41, param_dtype=torch.bfloat16)
    if sparse:
        for p in m.indexer.parameters():                   # the indexer's own loss is not what is checked here
            p.requires_grad_(False)
    cu = [0, 300, 700, 1024]
    T = cu[-1]
    g = torch.Generator().manual_seed(42)
    x_cpu = torch.randn(1, T, hidden, generator=g).bfloat16()
    gy = torch.randn(1, T, hidden, generator=g).bfloat16().to(DEV)
    cos, sin = (t.to(DEV).to(torch.bfloat16) for t in _tables(T, D, torch.float32))
    cu_d = torch.tensor(cu, dtype=torch.int32, device=DEV)
    results = []
    for wrapped in (False, True):
        for p in m.parameters():
            p.grad = None
        x = x_cpu.to(DEV).requires_grad_(True)
        y = checkpoint(m, x, cos, sin, cu_d, 512, use_reentrant=False) if wrapped else m(x, cos, sin, cu_d, 512)
        y.backward(gy)
        results.append([y.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in m.parameters() if p.grad is not None])
    assert len(results[0]) == len(results[1]) >= 8
    for a, b in zip(*results):
        assert torch.equal(a, b)
