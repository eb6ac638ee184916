"""CPU checks of the layer level: the oracle of the reference's attention layers against library routines used a
different way, the DTensor unwrap / rewrap helpers on a one-rank mesh, and the installer on the HF classes."""
import os

import pytest
import torch
import torch.nn.functional as F

from oracle import layer_ref as LR


def _weights(hidden, Hq, Hkv, D, gated, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g) * (s[-1] ** -0.5)
    return dict(wq=r(Hq * D * (2 if gated else 1), hidden), wk=r(Hkv * D, hidden), wv=r(Hkv * D, hidden), wo=r(hidden, Hq * D),
                qn_w=torch.randn(D, generator=g) * 0.2 + (0.0 if gated else 1.0),
                kn_w=torch.randn(D, generator=g) * 0.2 + (0.0 if gated else 1.0))


def _tables(T, R, theta=1e4):
    inv = 1.0 / (theta ** (torch.arange(0, R, 2, dtype=torch.float32) / R))
    ang = torch.outer(torch.arange(T, dtype=torch.float32), inv)          # (T, R/2)
    emb = torch.cat((ang, ang), -1)
    return emb.cos(), emb.sin(), ang


def _independent_layer(x, w, ang, cu, Hq, Hkv, D, R, gated, eps):
    """The layer written another way: F.rms_norm, the rotation of every (i, i + R/2) pair as a complex product,
    one SDPA call per segment with enable_gqa, explicit sigmoid."""
    h = x[0]
    T = h.shape[0]
    qp = h @ w["wq"].t()
    if gated:
        qg = qp.view(T, Hq, 2 * D)
        q, gate = qg[..., :D], qg[..., D:].reshape(T, Hq * D)
    else:
        q, gate = qp.view(T, Hq, D), None
    k = (h @ w["wk"].t()).view(T, Hkv, D)
    v = (h @ w["wv"].t()).view(T, Hkv, D)
    off = 1.0 if gated else 0.0
    q = F.rms_norm(q, (D,), w["qn_w"] + off, eps)
    k = F.rms_norm(k, (D,), w["kn_w"] + off, eps)

    def rot(t):
        z = torch.complex(t[..., : R // 2], t[..., R // 2: R]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
        return torch.cat((z.real, z.imag, t[..., R:]), -1)

    q, k = rot(q), rot(k)
    outs = []
    for a, b in zip(cu[:-1], cu[1:]):
        if b > a:
            o = F.scaled_dot_product_attention(q[a:b].transpose(0, 1)[None], k[a:b].transpose(0, 1)[None],
                                               v[a:b].transpose(0, 1)[None], is_causal=True, enable_gqa=True)
            outs.append(o[0].transpose(0, 1).reshape(b - a, Hq * D))
    out = torch.cat(outs)
    if gated:
        out = out * torch.sigmoid(gate)
    return (out @ w["wo"].t())[None]


@pytest.mark.parametrize("gated,R", [(False, 16), (True, 8), (True, 16)])
def test_layer_oracle_against_library_routines(gated, R):
    hidden, Hq, Hkv, D, eps = 24, 4, 2, 16, 1e-6
    cu = [0, 9, 9, 20, 23]
    T = cu[-1]
    x = torch.randn(1, T, hidden, generator=torch.Generator().manual_seed(1))
    w = _weights(hidden, Hq, Hkv, D, gated, seed=2)
    cos, sin, ang = _tables(T, R)
    fn = LR.qwen3_5_attention if gated else LR.qwen3vl_attention
    got = fn(x, w["wq"], w["wk"], w["wv"], w["wo"], w["qn_w"], w["kn_w"], cos, sin, cu, D, eps)
    want = _independent_layer(x, w, ang, cu, Hq, Hkv, D, R, gated, eps)
    assert got.shape == (1, T, hidden)
    assert torch.allclose(got, want, atol=2e-5), (got - want).abs().max()


def test_dsa_layer_with_full_selection_is_the_dense_layer_and_its_loss_is_a_kl():
    from oracle import dsa_ref as R_
    hidden, Hq, Hkv, D, Hi, Di = 24, 4, 2, 16, 3, 8
    cu = [0, 9, 20]
    T = cu[-1]
    g = torch.Generator().manual_seed(5)
    x = torch.randn(1, T, hidden, generator=g)
    w = _weights(hidden, Hq, Hkv, D, False, seed=6)
    wi = [torch.randn(Hi * Di, hidden, generator=g) * 0.2, torch.randn(Di, hidden, generator=g) * 0.2,
          torch.randn(Hi, hidden, generator=g) * 0.2]
    cos, sin, _ = _tables(T, D)
    h = x[0]
    idx, n = R_.dsa_select((h @ wi[0].t()).view(T, Hi, Di), h @ wi[1].t(), h @ wi[2].t(), cu, 32)     # K >= longest segment
    y, loss, _ = LR.dsa_layer(x, w["wq"], w["wk"], w["wv"], w["wo"], w["qn_w"], w["kn_w"], cos, sin, cu, D, *wi, Hi, Di, idx, n)
    dense = LR.qwen3vl_attention(x, w["wq"], w["wk"], w["wv"], w["wo"], w["qn_w"], w["kn_w"], cos, sin, cu, D)
    assert torch.allclose(y, dense, atol=1e-5)
    assert float(loss) >= 0.0
    idx4, n4 = R_.dsa_select((h @ wi[0].t()).view(T, Hi, Di), h @ wi[1].t(), h @ wi[2].t(), cu, 4)
    y4, loss4, _ = LR.dsa_layer(x, w["wq"], w["wk"], w["wv"], w["wo"], w["qn_w"], w["kn_w"], cos, sin, cu, D, *wi, Hi, Di, idx4, n4)
    assert not torch.allclose(y4, dense, atol=1e-3) and float(loss4) >= 0.0


# ------------------------------------------------------------------------------------------ DTensor helpers
def test_dtensor_unwrap_and_rewrap_on_a_one_rank_mesh():
    """models/qwen3_5/utils.py:13-42: local shards out, the same mesh and placements back on."""
    import torch.distributed as dist
    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.tensor import DTensor, Shard

    from vlm_training_amd.dtensor_utils import _dtensor_rewrap, _dtensor_unwrap, _local
    created = False
    if not dist.is_initialized():
        os.environ.setdefault("MASTER_ADDR", "127.0.0.1")
        os.environ.setdefault("MASTER_PORT", "29571")
        dist.init_process_group("gloo", rank=0, world_size=1)
        created = True
    try:
        mesh = init_device_mesh("cpu", (1,))
        q = torch.randn(6, 4, 8)
        dq = DTensor.from_local(q, mesh, [Shard(1)], run_check=False)         # sharded by head, as under column-parallel q_proj
        plain = torch.randn(6, 2, 8)
        (a, b), wrap = _dtensor_unwrap(dq, plain)
        assert not isinstance(a, DTensor) and torch.equal(a, q) and b is plain
        assert wrap[0] is mesh and tuple(wrap[1]) == (Shard(1),)
        back = _dtensor_rewrap(a * 2, wrap)
        assert isinstance(back, DTensor) and tuple(back.placements) == (Shard(1),) and torch.equal(back.to_local(), q * 2)
        (c,), none = _dtensor_unwrap(plain)
        assert none is None and c is plain and _dtensor_rewrap(plain, None) is plain
        assert torch.equal(_local(dq), q) and _local(plain) is plain
    finally:
        if created:
            dist.destroy_process_group()


# ------------------------------------------------------------------------------------------ installer
def test_installer_replaces_the_hf_forwards_and_masks_and_can_be_undone():
    """train/model_attention.py:265-299."""
    import importlib

    import vlm_training_amd as M
    mods = {name: importlib.import_module(name) for name in (
        "transformers.models.qwen3.modeling_qwen3", "transformers.models.qwen3_vl.modeling_qwen3_vl",
        "transformers.models.qwen3_vl_moe.modeling_qwen3_vl_moe", "transformers.models.qwen3_5.modeling_qwen3_5")}
    undo = M.replace_attention_qwenvl()
    try:
        assert mods["transformers.models.qwen3.modeling_qwen3"].Qwen3Attention.forward is M.qwen3vl_forward
        assert mods["transformers.models.qwen3_vl.modeling_qwen3_vl"].Qwen3VLTextAttention.forward is M.qwen3vl_forward
        assert mods["transformers.models.qwen3_vl_moe.modeling_qwen3_vl_moe"].Qwen3VLMoeTextAttention.forward is M.qwen3vl_forward
        assert mods["transformers.models.qwen3_5.modeling_qwen3_5"].Qwen3_5Attention.forward is M.qwen3_5_forward
        for m in mods.values():
            assert m.create_causal_mask is M.return_mask
        cu = torch.tensor([0, 5, 9], dtype=torch.int32)
        assert M.return_mask(cu, config=None).shape == (1, 3)
    finally:
        for owner, attr, old in reversed(undo):
            setattr(owner, attr, old)
    assert mods["transformers.models.qwen3.modeling_qwen3"].Qwen3Attention.forward is not M.qwen3vl_forward


def test_installer_patches_nothing_when_a_target_is_missing(monkeypatch):
    """A transformers build without one of the four models must leave the others as they were."""
    import importlib

    import vlm_training_amd.model_attention as MA
    qwen3 = importlib.import_module("transformers.models.qwen3.modeling_qwen3")
    before = qwen3.Qwen3Attention.forward
    real_import = importlib.import_module

    def failing(name, *a, **k):
        if name.endswith("modeling_qwen3_5"):
            raise ImportError("no qwen3_5 in this build")
        return real_import(name, *a, **k)

    monkeypatch.setattr(importlib, "import_module", failing)
    with pytest.raises(ImportError):
        MA.replace_attention_qwenvl()
    assert qwen3.Qwen3Attention.forward is before and qwen3.create_causal_mask is not MA.return_mask


# ------------------------------------------------------------------------------------------ longest segment
def test_longest_segment_follows_the_tensor_not_its_address():
    """train/model_attention.py:118-121 always uses the true maximum.  A new offsets tensor that lands on a freed
    tensor's address (what the caching allocator does every step) must get its own bound; views of one tensor share
    one read; an in-place write invalidates it."""
    from vlm_training_amd.model_attention import _BOUND_ATTR, longest_segment
    import numpy as np
    buf = np.array([0, 100, 260, 300], dtype=np.int32)                   # one block of memory, two tensors in turn
    a = torch.from_numpy(buf)
    ptr = a.data_ptr()
    assert longest_segment(a) == 160
    del a
    buf[1] = 200                                                         # "the next step's offsets" at the same address
    b = torch.from_numpy(buf)
    assert b.data_ptr() == ptr and b._version == 0 and b.numel() == 4    # what an address-keyed cache cannot tell apart
    assert longest_segment(b) == 200
    del b
    c = torch.tensor([0, 7, 9, 30], dtype=torch.int32)
    assert longest_segment(c) == 21 and getattr(c, _BOUND_ATTR)[3] == 21
    masked = c.unsqueeze_(0)                                            # what return_mask does: same object, version + 1
    assert masked is c and longest_segment(c.reshape(-1)) == 21 and longest_segment(c.squeeze()) == 21
    c[0, 1] = 1                                                          # in-place writes bump the version
    c[0, 2] = 2                                                          # [0,1,2,30] -> 28
    assert longest_segment(c.reshape(-1)) == 28
    assert longest_segment(torch.tensor([0], dtype=torch.int32)) == 1
    assert longest_segment(torch.tensor([0, 0, 0], dtype=torch.int32)) == 1
    # two separately built tensors with equal contents never share an entry
    d, e = torch.tensor([0, 4, 6], dtype=torch.int32), torch.tensor([0, 4, 6], dtype=torch.int32)
    assert longest_segment(d) == 4 and not hasattr(e, _BOUND_ATTR) and longest_segment(e) == 4
