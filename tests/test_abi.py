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
    # launch order of the key tiles (five words per entry and a header), and fp32 partial sums for key-tile walks
    # that a small launch cuts into pieces (16 KiB per token, at most 128 MiB, none above 131072 tokens)
    order = up(((1000 // 128 + 4096 + 1 + 4096) * 5 + 4) * 4) + up(1000 * 16384)
    assert lib.dsa_attn_bwd_workspace_bytes(1000, 8, 640, 0) == up(1000 * 8 * 4) + order
    assert lib.dsa_attn_bwd_workspace_bytes(1000, 8, 640, 1) == up(1000 * 8 * 4) + up(1000 * 20 * 4) + order
    big = lib.dsa_attn_bwd_workspace_bytes(32768, 32, 7168, 0) - up(32768 * 32 * 4) - up(((32768 // 128 + 4096 + 1 + 4096) * 5 + 4) * 4)
    assert big == 128 << 20
    assert lib.dsa_attn_bwd_workspace_bytes(262144, 1, 8, 0) == up(262144 * 4) + up(((262144 // 128 + 4096 + 1 + 4096) * 5 + 4) * 4)
    assert lib.dsa_attn_fwd_workspace_bytes(1000, 640, 1) == up(1000 * 20 * 4)
    assert lib.dsa_attn_bwd_bitmap_offset(1000, 8) == up(1000 * 8 * 4)   # forward workspace fits behind it
    assert lib.dsa_attn_fwd_workspace_bytes(1000, 640, 0) == 0
    old = lib.dsa_get_tile_crossover()
    # what the backward allocates when it runs: delta, the key-tile order, and partial sums only for launches small
    # enough to be cut into pieces (at most 1024 key-tile workgroups); the bitmap stays in the forward's workspace
    order_of = lambda T: up(((T // 128 + 4096 + 1 + 4096) * 5 + 4) * 4)
    assert lib.dsa_attn_bwd_scratch_bytes(32768, 8, 32, 8, 128) == up(32768 * 32 * 4) + order_of(32768)
    assert lib.dsa_attn_bwd_scratch_bytes(8192, 7, 16, 8, 128) == up(8192 * 16 * 4) + up(8192 * 16384) + order_of(8192)
    # attention mass: the bitmap alone when one workgroup holds every kv head (8 at head_dim 128, 4 at 256), else a
    # (T,K) table per group of kv heads
    assert lib.dsa_attn_mass_workspace_bytes(32768, 8, 32, 8, 128, 2048, 7168) == up(32768 * 224 * 4)
    assert lib.dsa_attn_mass_workspace_bytes(16384, 33, 16, 2, 256, 512, 1669) == up(16384 * 53 * 4)
    assert lib.dsa_attn_mass_workspace_bytes(1000, 3, 32, 16, 128, 64, 640) == up(1000 * 20 * 4) + up(2 * 1000 * 64 * 4)
    assert old == 24 and lib.dsa_set_tile_crossover(-1) == -1 and lib.dsa_set_tile_crossover(3) == 0
    assert lib.dsa_get_tile_crossover() == 3 and lib.dsa_set_tile_crossover(old) == 0
    assert lib.dsa_get_bwd_overlap() == 1 and lib.dsa_set_bwd_overlap(3) == -1 and lib.dsa_set_bwd_overlap(0) == 0
    assert lib.dsa_get_bwd_overlap() == 0 and lib.dsa_set_bwd_overlap(1) == 0


def test_argument_errors_are_reported_not_thrown():
    lib = _lib.load()
    rc = lib.dsa_attn_fwd(None, None, None, None, None, None, 8, 1, 4, 3, 64, 0, 1.0, 0, 8, 1, None, None, None, 0, None)
    assert rc == -1 and b"cu_seqlens" in lib.dsa_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc, "dsa_attn_fwd")
    # the entry points that read or leave a selection bitmap, and the small ones beside them: refused before any launch
    import ctypes
    cu = (ctypes.c_int32 * 2)(0, 8)
    rc = lib.dsa_attn_fwd_saved_bitmap(None, None, None, None, None, cu, 8, 1, 4, 2, 64, 0, 1.0, 0, 8, 1, None, None, None, 0, None)
    assert rc == -1 and b"idx is null" in lib.dsa_last_error()
    one = ctypes.c_int32(0)
    rc = lib.dsa_index_topk_bitmap(None, None, None, cu, 8, 1, 4, 64, 4, 1.0, 0, 8, ctypes.byref(one), ctypes.byref(one), None,
                                   None, 0, None, 0, None)
    assert rc == -3 and b"selection bitmap" in lib.dsa_last_error()
    assert lib.dsa_round_bf16_x3(None, None, None, 4, 0, 0, None, None, None, None) == -1
    assert lib.dsa_round_bf16_x3(None, None, None, 0, 0, 0, None, None, None, None) == 0       # nothing to do
    assert lib.dsa_split_bf16_stack_qkv(None, None, None, 0, 0, 64, None, None, None, None) == 0
    assert lib.dsa_split_bf16_combine_qkv(None, None, None, 4, 0, 64, None, None, None, None) == -1


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


# ------------------------------------------------------------------------------------------------------------
# the binding and the documentation follow the header
# ------------------------------------------------------------------------------------------------------------
def _header_prototypes():
    """name -> list of parameter type strings, parsed from include/dsa_attn.h."""
    text = open(os.path.join(ROOT, "include", "dsa_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    protos = {}
    for m in re.finditer(r"([A-Za-z_][\w \*]*?)\b(dsa_[a-z_0-9]+)\s*\(([^)]*)\)\s*;", text):
        params = [p.strip() for p in m.group(3).split(",")]
        if params == ["void"]:
            params = []
        protos[m.group(2)] = (m.group(1).strip(), [re.sub(r"\s*\b\w+$", "", p).strip() if not p.endswith("*") else p for p in params])
    return protos


def _ctype_of(c_type: str):
    from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
    t = c_type.replace("const ", "").strip()
    if t.endswith("*"):
        return c_char_p if t.startswith("char") else c_void_p
    return {"int": c_int, "float": c_float, "int64_t": c_int64, "size_t": c_size_t}[t]


def test_ctypes_signatures_follow_the_header_prototypes():
    protos = _header_prototypes()
    assert sorted(protos) == sorted(_lib.EXPORTS)
    for name, (ret, params) in protos.items():
        res, args = _lib._SIGNATURES[name]
        assert len(args) == len(params), (name, len(args), len(params))
        assert [_ctype_of(p) for p in params] == list(args), name
        assert _ctype_of(ret) == res, name
    assert len(protos["dsa_attn_fwd"][1]) == 21


def test_integration_stub_matches_the_header():
    """The ctypes stub a maintainer would copy out of the integration notes binds dsa_attn_fwd with the header's
    argument list, and its example call passes one value per argument."""
    from ctypes import c_float, c_int, c_size_t, c_void_p
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    m = re.search(r"lib\.dsa_attn_fwd\.argtypes = \[([^\]]*)\]", doc)
    assert m, "stub not found"
    short = {"P": c_void_p, "I": c_int, "F": c_float, "Z": c_size_t}
    stub = [short[x.strip()] for x in m.group(1).split(",")]
    assert stub == list(_lib._SIGNATURES["dsa_attn_fwd"][1])
    call = re.search(r"rc = lib\.dsa_attn_fwd\((.*?)\)\nif rc", doc, flags=re.S).group(1)
    call = re.sub(r"#.*", "", call)
    depth, nargs = 0, 1
    for ch in call:
        depth += ch in "([" 
        depth -= ch in ")]"
        nargs += ch == "," and depth == 0
    assert nargs == len(stub) == 21


def test_integration_notes_name_every_exported_symbol():
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    named = set(re.findall(r"`(dsa_[a-z0-9_]+)`", doc))
    missing = [name for name in _lib.EXPORTS if name not in named]
    assert not missing, missing
    unknown = [name for name in named if name.startswith("dsa_") and name not in _lib.EXPORTS
               and not name.startswith(("dsa_attn.h", "dsa_varlen_attn", "dsa_ref"))]
    assert not unknown, unknown
