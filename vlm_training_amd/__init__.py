"""MI355X-native packed-sequence DSA attention (gfx950 HIP kernels behind a C ABI)."""
from .model_attention import (dispatch_varlen_attention, run_varlen_attn, varlen_attention_forward,  # noqa: F401
                              varlen_attn)
from .ops import dsa_varlen_attn, index_topk, indexer_kl_loss  # noqa: F401
from .prologue import qk_norm_rope, sigmoid_gate  # noqa: F401

__all__ = ["dsa_varlen_attn", "index_topk", "indexer_kl_loss", "qk_norm_rope", "sigmoid_gate", "varlen_attn", "dispatch_varlen_attention", "run_varlen_attn",
           "varlen_attention_forward"]
