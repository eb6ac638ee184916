"""The operator under HIP graph capture: a captured forward+backward, replayed with eager work between the replays,
gives on every replay what the eager call gives.  (The library launches kernels and nothing else: no allocation, no
memset node, no synchronisation of its own.  With the backward's passes side by side - forced here, the launch being
too small for the default to choose it - the query-side pass is forked onto the library's second stream and joined
again, and the captured graph holds that fork and join too.)"""
import pytest
import torch

from vlm_training_amd import ops, workloads as W

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _log(msg):
    print(f"[graph] {msg}", flush=True)


@pytest.fixture(params=[1, 2], ids=["one-stream", "two-streams"])
def overlap(request):
    old = ops.set_bwd_overlap(request.param)
    yield request.param
    ops.set_bwd_overlap(old)


@pytest.mark.parametrize("sparse", [True, False])
def test_captured_step_replays_to_the_eager_result(sparse, overlap):
    _log(f"capture sparse={sparse} overlap={overlap}")
    w = W.scaled(W.C3, (700, 130, 260), top_k=128, name="graph")
    t = W.make_inputs(w, device=DEV)
    cu, msl = t["cu_seqlens"], w.max_seqlen
    kw = dict(indexer_q=t["q_idx"], indexer_k=t["k_idx"], indexer_w=t["w_idx"], top_k=w.top_k) if sparse else {}

    def step(q, k, v, dout):
        q.grad = k.grad = v.grad = None
        out = ops.dsa_varlen_attn(q, k, v, cu, msl, **kw)
        out.backward(dout)
        return out.detach(), q.grad, k.grad, v.grad

    q, k, v = (t[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
    dout = t["dout"].clone()
    want = [x.clone() for x in step(q, k, v, dout)]
    # static inputs for the graph; warm-up on a side stream as torch asks for before a capture
    sq, sk, sv = (t[x].clone().requires_grad_(True) for x in ("q", "k", "v"))
    sd = t["dout"].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step(sq, sk, sv, sd)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got = step(sq, sk, sv, sd)
    for replay in range(4):
        # other inputs first, so that a replay which computes nothing cannot pass on stale outputs; then the real ones
        with torch.no_grad():
            sq.copy_(torch.randn_like(sq)); sk.copy_(torch.randn_like(sk)); sv.copy_(torch.randn_like(sv))
        graph.replay()
        with torch.no_grad():
            sq.copy_(t["q"]); sk.copy_(t["k"]); sv.copy_(t["v"]); sd.copy_(t["dout"])
        eager = step(q, k, v, dout)                      # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b, c in zip(("out", "dq", "dk", "dv"), got, want, eager):
            assert torch.equal(a, b), f"replay {replay}: {name} differs from the eager result"
            assert torch.equal(c, b), f"replay {replay}: eager {name} changed"
