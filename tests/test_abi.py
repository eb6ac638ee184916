"""CPU-side checks of the boundary: the library loads and exports every symbol the header declares."""
import os
import re

import pytest
import torch

from vlm_training_amd import _lib, workloads as W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "dsa_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dsa_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 9
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(_lib.EXPORTS) == names
    assert lib.dsa_version().decode().startswith("dsa-attn-gfx950")


def test_workspace_sizes_without_a_gpu():
    lib = _lib.load()
    assert lib.dsa_index_topk_workspace_bytes(0, 0, 1) == 0
    b = lib.dsa_index_topk_workspace_bytes(32768, 7168, 2048)
    assert b == 32768 * 7168 * 4
    b4 = lib.dsa_index_topk_workspace_bytes(131072, 131072, 2048)
    assert b4 == 2048 * 131072 * 4                         # chunked: 1 GiB of score rows at a time
    up = lambda x: (x + 255) // 256 * 256                  # both parts are 256-byte aligned
    assert lib.dsa_attn_bwd_workspace_bytes(1000, 8, 640, 0) == up(1000 * 8 * 4)
    assert lib.dsa_attn_bwd_workspace_bytes(1000, 8, 640, 1) == up(1000 * 8 * 4) + up(1000 * 20 * 4)
    assert lib.dsa_attn_fwd_workspace_bytes(1000, 640, 1) == up(1000 * 20 * 4)
    assert lib.dsa_attn_bwd_bitmap_offset(1000, 8) == up(1000 * 8 * 4)   # forward workspace fits behind it
    assert lib.dsa_attn_fwd_workspace_bytes(1000, 640, 0) == 0
    old = lib.dsa_get_tile_crossover()
    assert old == 16 and lib.dsa_set_tile_crossover(-1) == -1 and lib.dsa_set_tile_crossover(3) == 0
    assert lib.dsa_get_tile_crossover() == 3 and lib.dsa_set_tile_crossover(old) == 0


def test_argument_errors_are_reported_not_thrown():
    lib = _lib.load()
    rc = lib.dsa_attn_fwd(None, None, None, None, None, None, 8, 1, 4, 3, 64, 0, 1.0, 0, 8, 1, None, None, None, 0, None)
    assert rc == -1 and b"cu_seqlens" in lib.dsa_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc, "dsa_attn_fwd")


def test_cpu_tensors_are_refused_loudly():
    from vlm_training_amd import ops
    q = torch.zeros(4, 2, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.dsa_varlen_attn(q, q, q, torch.tensor([0, 4], dtype=torch.int32), 4)


def test_workload_tables_match_the_measurement_plan():
    P, S = W.C1.pair_counts()
    assert (W.C1.T, P, S) == (2048, 640000, 229632)
    assert W.C2.T == 8192 and W.C3.T == 32768 and W.C4.T == 131072 and W.C5.T == 16384
    P3, S3 = W.C3.pair_counts()
    assert abs(P3 - 8.18e7) / 8.18e7 < 0.01 and abs(S3 - 5.09e7) / 5.09e7 < 0.01
    wk = W.C3.work()
    assert abs(wk["F1"] - 1.35e12) / 1.35e12 < 0.01 and abs(wk["B3_gather"] - 2.08e11) / 2.08e11 < 0.01
    t = W.make_inputs(W.scaled(W.C3, (2100, 50), top_k=8), device="cpu")
    assert t["q"].dtype == torch.bfloat16 and t["cu_seqlens"].tolist() == [0, 2100, 2150]
    t2 = W.make_inputs(W.scaled(W.C3, (2100, 50), top_k=8), device="cpu")
    assert torch.equal(t["q"], t2["q"]) and torch.equal(t["k_idx"], t2["k_idx"])
