"""The operator as torch.library custom ops (vlm_training_amd/custom_ops.py): shape-only implementations on the CPU, and on
the GPU torch's own checker plus a compiled block without a graph break (train/infra.py:236-248 compiles every block)."""
import pytest
import torch

from vlm_training_amd import _lib, custom_ops as C, ops, workloads as W


def _fake_inputs(T, Hq, Hkv, D, Hi, Di, dev):
    mk = lambda *s: torch.empty(*s, dtype=torch.bfloat16, device=dev)
    return (mk(T, Hq, D), mk(T, Hkv, D), mk(T, Hkv, D), torch.empty(4, dtype=torch.int32, device=dev), mk(T, Hi, Di), mk(T, Di),
            mk(T, Hi))


def test_fake_implementations_give_the_shapes_and_workspace_size_of_the_real_ones():
    from torch._subclasses.fake_tensor import FakeTensorMode
    lib = _lib.load()
    for T, msl, K in ((100, 64, 16), (8192, 1799, 1024), (32768, 7168, 2048)):
        with FakeTensorMode():
            q, k, v, cu, qi, ki, wi = _fake_inputs(T, 8, 2, 128, 4, 64, "cuda")
            idx, n = C._index_topk(qi, ki, wi, cu, msl, K, None)
            assert idx.shape == (T, K) and idx.dtype == torch.int32 and n.shape == (T,) and n.dtype == torch.int32
            out, lse, ws = C._attn_fwd(q, k, v, cu, msl, idx, n, 0.1, True)
            assert out.shape == q.shape and out.dtype == torch.bfloat16
            assert lse.shape == (8, T) and lse.dtype == torch.float32 and ws.dtype == torch.uint8
            assert ws.numel() == lib.dsa_attn_fwd_workspace_bytes(T, msl, 1)       # the size the real op allocates
            dq, dk, dv = C._attn_bwd(out, q, k, v, out, lse, cu, idx, n, ws, msl, 0.1, True)
            assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
            dense = C.dsa_varlen_attn_traceable(q, k, v, cu, msl)
            assert dense.shape == q.shape
    with pytest.raises(ValueError):
        C.dsa_varlen_attn_traceable(torch.zeros(4, 2, 64), torch.zeros(4, 2, 64), torch.zeros(4, 2, 64),
                                    torch.tensor([0, 4], dtype=torch.int32), 4)


def _packed(seed=31):
    w = W.scaled(W.C3, (300, 130, 82), top_k=64, name="custom-ops")
    return w, W.make_inputs(w, device="cuda")


@pytest.mark.gpu
def test_custom_ops_pass_the_library_checker():
    """torch.library.opcheck: schema, fake implementation against the real one, autograd registration, AOT dispatch."""
    w, t = _packed()
    cu, msl = t["cu_seqlens"], w.max_seqlen
    idx, n = ops.index_topk(t["q_idx"], t["k_idx"], t["w_idx"], cu, msl, w.top_k)
    torch.library.opcheck(C._index_topk, (t["q_idx"], t["k_idx"], t["w_idx"], cu, msl, w.top_k, None))
    q, k, v = (t[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
    for sel in ((idx, n), (None, None)):
        torch.library.opcheck(C._attn_fwd, (q, k, v, cu, msl, *sel, w.D ** -0.5, True),
                              test_utils=("test_schema", "test_faketensor", "test_autograd_registration", "test_aot_dispatch_static"))


@pytest.mark.gpu
@pytest.mark.parametrize("sparse", [True, False])
def test_a_compiled_block_holds_the_operator_without_a_graph_break(sparse):
    """projections -> operator -> projection compiled with fullgraph=True (any graph break is an error there): forward
    and every gradient equal the eager run of the same function and of ops.dsa_varlen_attn, bit for bit."""
    print(f"[custom ops] compiled block, sparse={sparse}", flush=True)
    w, t = _packed()
    cu, msl = t["cu_seqlens"], w.max_seqlen
    T, Hq, Hkv, D = w.T, w.Hq, w.Hkv, w.D
    hidden = 256
    g = torch.Generator().manual_seed(32)
    wq, wk, wv = (torch.randn(H * D, hidden, generator=g).mul_(hidden ** -0.5).bfloat16().cuda().requires_grad_(True) for H in (Hq, Hkv, Hkv))
    wo = torch.randn(hidden, Hq * D, generator=g).mul_((Hq * D) ** -0.5).bfloat16().cuda().requires_grad_(True)
    x = torch.randn(T, hidden, generator=g).bfloat16().cuda().requires_grad_(True)
    gy = torch.randn(T, hidden, generator=g).bfloat16().cuda()
    kw = dict(indexer_q=t["q_idx"], indexer_k=t["k_idx"], indexer_w=t["w_idx"], top_k=w.top_k) if sparse else {}

    def block(attn, x, wq, wk, wv, wo):
        q = (x @ wq.t()).view(T, Hq, D)
        k = (x @ wk.t()).view(T, Hkv, D)
        v = (x @ wv.t()).view(T, Hkv, D)
        return attn(q, k, v, cu, msl, **kw).reshape(T, Hq * D) @ wo.t()

    def run(fn, attn):
        for p in (x, wq, wk, wv, wo):
            p.grad = None
        y = fn(attn, x, wq, wk, wv, wo)
        y.backward(gy)
        return [y.detach().clone()] + [p.grad.clone() for p in (x, wq, wk, wv, wo)]

    want = run(block, ops.dsa_varlen_attn)
    eager = run(block, C.dsa_varlen_attn_traceable)
    compiled = torch.compile(block, fullgraph=True, backend="aot_eager")
    got = run(compiled, C.dsa_varlen_attn_traceable)
    again = run(compiled, C.dsa_varlen_attn_traceable)
    for name, a, b, c, d in zip(("y", "dx", "dwq", "dwk", "dwv", "dwo"), want, eager, got, again):
        assert torch.equal(a, b), f"{name}: traceable operator differs from ops.dsa_varlen_attn"
        assert torch.equal(a, c) and torch.equal(a, d), f"{name}: compiled block differs from the eager one"
