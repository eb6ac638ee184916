"""The entry point that allocates nothing: dsa_index_topk_noalloc against dsa_index_topk, through the C ABI.

Collected last (file name), so that a failure here cannot hide another test behind `pytest -x`."""
import ctypes

import pytest
import torch

from vlm_training_amd import _lib, workloads as W

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _ptr(x):
    return ctypes.c_void_p(x.data_ptr())


def _both(lib, w):
    """(idx, n) of the workspace entry point and of the static-scratch one on the same inputs."""
    t = W.make_inputs(w, device=DEV, with_dout=False)
    cu = t["cu_seqlens"]
    T, N, K = w.T, len(w.seg_lens), w.top_k
    scale = (w.Di ** -0.5) * (w.Hi ** -0.5)
    st = torch.cuda.current_stream().cuda_stream
    res = []
    for noalloc in (False, True):
        idx = torch.full((T, K), -7, dtype=torch.int32, device=DEV)
        n = torch.full((T,), -7, dtype=torch.int32, device=DEV)
        if noalloc:
            rc = lib.dsa_index_topk_noalloc(_ptr(t["q_idx"]), _ptr(t["k_idx"]), _ptr(t["w_idx"]), _ptr(cu), T, N, w.Hi, w.Di, K,
                                            scale, 0, w.max_seqlen, _ptr(idx), _ptr(n), st)
        else:
            nbytes = lib.dsa_index_topk_workspace_bytes(T, w.max_seqlen, K)
            ws = torch.empty((max(nbytes, 4),), dtype=torch.uint8, device=DEV)
            rc = lib.dsa_index_topk(_ptr(t["q_idx"]), _ptr(t["k_idx"]), _ptr(t["w_idx"]), _ptr(cu), T, N, w.Hi, w.Di, K, scale,
                                    0, w.max_seqlen, _ptr(idx), _ptr(n), _ptr(ws), nbytes, st)
        assert rc == 0, lib.dsa_last_error().decode()
        torch.cuda.synchronize()
        res.append((idx, n))
    return res


def test_index_topk_without_allocation_equals_the_workspace_entry_point():
    """Two calls in a row on the shared static scratch, the second on a smaller batch (so the scratch still holds the
    first call's longer rows): selections bit-identical to dsa_index_topk both times.  The first batch needs more score
    rows than the 32 MiB scratch holds at once, so the chunked loop runs several rounds."""
    lib = _lib.load()
    assert lib.dsa_index_topk_noalloc_scratch_bytes() == 32 << 20
    big = W.scaled(W.C3, (5000, 700, 4096, 33), top_k=512, name="noalloc-big")        # 9829 rows of 5024 columns: 6 chunks
    assert big.T * ((big.max_seqlen + 31) // 32 * 32) * 4 > 5 * lib.dsa_index_topk_noalloc_scratch_bytes()
    small = W.scaled(W.C2, (900, 64, 333), top_k=128, name="noalloc-small")
    for w in (big, small):
        (idx0, n0), (idx1, n1) = _both(lib, w)
        assert torch.equal(n0, n1), w.name
        assert torch.equal(idx0, idx1), w.name
        assert int(n1.min()) >= 1 and int((idx1 == -7).sum()) == 0


def test_index_topk_without_allocation_rejects_rows_beyond_the_scratch():
    lib = _lib.load()
    limit = lib.dsa_index_topk_noalloc_max_seqlen()
    assert limit == (32 << 20) // 16 // 32 * 32
    x = torch.zeros(8, dtype=torch.int32, device=DEV)
    rc = lib.dsa_index_topk_noalloc(_ptr(x), _ptr(x), _ptr(x), _ptr(x), limit + 64, 1, 4, 32, 8, 1.0, 0, limit + 32, _ptr(x),
                                    _ptr(x), None)
    assert rc == -3 and b"static scratch" in lib.dsa_last_error()


def test_index_topk_without_allocation_under_graph_capture():
    """The callers the entry point is for: a HIP graph captured around it (after one plain call on the device, which
    looks up the scratch address) replays to the selection of dsa_index_topk, on every replay, with eager work between
    the replays."""
    lib = _lib.load()
    w = W.scaled(W.C3, (1500, 40, 700), top_k=256, name="noalloc-graph")
    t = W.make_inputs(w, device=DEV, with_dout=False)
    cu = t["cu_seqlens"]
    T, N, K = w.T, len(w.seg_lens), w.top_k
    scale = (w.Di ** -0.5) * (w.Hi ** -0.5)
    (want_idx, want_n), _ = _both(lib, w)                       # includes the plain noalloc call that precedes a capture
    sq, sk, sw = (t[x].clone() for x in ("q_idx", "k_idx", "w_idx"))            # static inputs of the graph
    idx = torch.full((T, K), -7, dtype=torch.int32, device=DEV)
    n = torch.full((T,), -7, dtype=torch.int32, device=DEV)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.dsa_index_topk_noalloc(_ptr(sq), _ptr(sk), _ptr(sw), _ptr(cu), T, N, w.Hi, w.Di, K, scale, 0, w.max_seqlen,
                                        _ptr(idx), _ptr(n), torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.dsa_last_error().decode()
    for replay in range(3):
        sq.copy_(torch.randn_like(sq))                           # other inputs first: a replay that computes nothing must not pass
        graph.replay()
        torch.cuda.synchronize()
        assert not torch.equal(idx, want_idx)
        sq.copy_(t["q_idx"])
        _both(lib, W.scaled(W.C2, (600, 90), top_k=64, name="noalloc-between"))  # eager work on the same scratch in between
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(idx, want_idx) and torch.equal(n, want_n), f"replay {replay}"
