"""ctypes binding of libdsa_attn.so (the C ABI declared in include/dsa_attn.h).

There is no CPU or eager fallback: if the library is missing, every operator raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdsa_attn.so")

DSA_DTYPE_BF16 = 0
DSA_DTYPE_FP32 = 1
DSA_NORM_OFFSET, DSA_NORM_WEIGHT_BF16 = 1, 2                                               # norm_flags of the prologue
DSA_BWD_DELTA, DSA_BWD_BITMAP, DSA_BWD_DQ, DSA_BWD_DKV, DSA_BWD_ALL = 1, 2, 4, 8, 15      # parts of dsa_attn_bwd_parts

_SIGNATURES = {
    "dsa_version": (c_char_p, []),
    "dsa_last_error": (c_char_p, []),
    "dsa_indexer_scores": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_int,
                                   c_int, c_int, c_int, c_void_p, c_int64, c_void_p]),
    "dsa_topk_from_scores": (c_int, [c_void_p, c_int64, c_int, c_int, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p,
                                     c_void_p]),
    "dsa_index_topk_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "dsa_index_topk": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                               c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "dsa_index_topk_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float,
                                       c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "dsa_index_topk_noalloc_scratch_bytes": (c_size_t, []),
    "dsa_index_topk_noalloc_max_seqlen": (c_int, []),
    "dsa_index_topk_scores": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float,
                                      c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "dsa_indexer_kl": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p, c_void_p, c_void_p]),
    "dsa_indexer_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                c_void_p]),
    "dsa_indexer_bwd_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "dsa_attn_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                             c_int, c_float, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "dsa_attn_fwd_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "dsa_attn_mass": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                              c_int, c_float, c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "dsa_attn_mass_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    "dsa_set_tile_crossover": (c_int, [c_int]),
    "dsa_get_tile_crossover": (c_int, []),
    "dsa_index_topk_bitmap": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                                      c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p]),
    "dsa_attn_fwd_saved_bitmap": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                          c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                          c_size_t, c_void_p]),
    "dsa_attn_mass_saved_bitmap": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                           c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p,
                                           c_size_t, c_void_p]),
    "dsa_set_bwd_overlap": (c_int, [c_int]),
    "dsa_get_bwd_overlap": (c_int, []),
    "dsa_attn_bwd_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "dsa_attn_bwd_bitmap_offset": (c_size_t, [c_int, c_int]),
    "dsa_attn_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                             c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p, c_void_p,
                             c_void_p, c_void_p, c_size_t, c_void_p]),
    "dsa_attn_bwd_parts": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int,
                                   c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    "dsa_attn_bwd_scratch_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "dsa_attn_bwd_saved_bitmap": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int,
                                          c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p]),
    "dsa_dense_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                              c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "dsa_dense_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                              c_int, c_int, c_float, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                              c_void_p]),
    "dsa_qk_norm_rope_bwd_workspace_bytes": (c_size_t, [c_int, c_int]),
    "dsa_qk_norm_rope_fwd": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_float,
                                     c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p,
                                     c_void_p, c_void_p, c_void_p, c_void_p]),
    "dsa_qk_norm_rope_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p,
                                     c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int,
                                     c_int, c_int, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p,
                                     c_void_p, c_void_p, c_size_t, c_void_p]),
    "dsa_sigmoid_gate_fwd": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_int, c_void_p, c_void_p]),
    "dsa_split_bf16_stack": (c_int, [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p]),
    "dsa_split_bf16_combine": (c_int, [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p]),
    "dsa_round_bf16_x3": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "dsa_split_bf16_stack_qkv": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p, c_void_p,
                                         c_void_p]),
    "dsa_split_bf16_combine_qkv": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p,
                                           c_void_p, c_void_p]),
    "dsa_sigmoid_gate_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_int, c_void_p,
                                     c_void_p, c_int64, c_int64, c_void_p]),
}

EXPORTS = tuple(_SIGNATURES)
_lib = None


class DsaLibraryError(RuntimeError):
    pass


def load():
    """Load the HIP library once; raise loudly when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise DsaLibraryError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or __graft_entry__.build()); there is no fallback path")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str):
    if rc != 0:
        msg = load().dsa_last_error().decode()
        exc = ValueError if rc == -1 else RuntimeError
        raise exc(f"{what} failed ({rc}): {msg}")
