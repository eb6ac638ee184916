"""MI355X-native packed-sequence DSA attention (gfx950 HIP kernels behind a C ABI)."""
from .layers import DsaConfig, DsaIndexer, Qwen3VLTextAttention, SelfAttention, indexer_losses  # noqa: F401
from .model_attention import (dispatch_varlen_attention, qwen3_5_forward, qwen3_forward, qwen3vl_forward,  # noqa: F401
                              replace_attention_qwenvl, return_mask, run_varlen_attn, varlen_attention_forward,
                              varlen_attn)
from .custom_ops import dsa_varlen_attn_traceable  # noqa: F401
from .ops import dsa_varlen_attn, index_topk, indexer_kl_loss  # noqa: F401
from .prologue import qk_norm_rope, sigmoid_gate  # noqa: F401

__all__ = ["DsaConfig", "DsaIndexer", "Qwen3VLTextAttention", "SelfAttention", "indexer_losses", "qwen3_forward",
           "qwen3vl_forward", "qwen3_5_forward", "replace_attention_qwenvl", "return_mask", "dsa_varlen_attn", "dsa_varlen_attn_traceable", "index_topk", "indexer_kl_loss", "qk_norm_rope", "sigmoid_gate", "varlen_attn", "dispatch_varlen_attention", "run_varlen_attn",
           "varlen_attention_forward"]
