"""Drop-in entry points with the reference's own names and signatures.

* ``varlen_attention_forward(query, key, value, attention_mask)`` - train/model_attention.py:97-143
  (HF layout ``(1,H,T,D)``; ``attention_mask`` carries the 1-D ``cu_seqlens``; returns
  ``((1,T,Hq,D), None)``).
* ``dispatch_varlen_attention(q, k, v, cu_seqlens, max_seqlen, causal=True)`` -
  models/qwen3_vl/model.py:25-46 (``(T,H,D)`` in and out).
* ``varlen_attn(q, k, v, cu_seq_q, cu_seq_k, max_q, max_k, ...)`` - the torch routine both call
  (torch 2.11 ``window_size=(-1, 0)`` form used by the reference, torch 2.10 ``is_causal=`` form).
* ``run_varlen_attn`` - models/qwen3_5/model.py:90-98 (``SelfAttention._run_varlen_attn``).

* ``qwen3_forward`` / ``qwen3vl_forward`` / ``qwen3_5_forward`` - train/model_attention.py:146-252, the forwards
  the reference installs on the HF attention classes, and ``replace_attention_qwenvl`` / ``return_mask``
  (train/model_attention.py:255-299), the installer.

All of them take the DSA extension as keyword-only arguments (default off = reference behaviour).
"""
from __future__ import annotations

import torch

from .ops import dsa_varlen_attn

_DSA_KEYS = ("indexer_q", "indexer_k", "indexer_w", "top_k", "index_scale", "return_indices", "return_mass", "return_scores")


def varlen_attn(query, key, value, cu_seq_q, cu_seq_k, max_q, max_k, is_causal=None, return_aux=None,
                scale=None, window_size=None, **dsa):
    unknown = set(dsa) - set(_DSA_KEYS)
    if unknown:
        raise TypeError(f"unexpected arguments {sorted(unknown)}")
    # self-attention only.  The same tensor, or two views of the same memory, is the usual call and costs nothing to
    # check; two separately built tensors (a clone, a .to()) are compared by content, which copies from the device once
    # - torch's own routine accepts them (models/qwen3_vl/model.py:41-46 passes one tensor twice) - and cannot be
    # done while a stream is being captured.
    if cu_seq_q is not cu_seq_k and not (cu_seq_q.data_ptr() == cu_seq_k.data_ptr() and cu_seq_q.shape == cu_seq_k.shape
                                         and cu_seq_q.stride() == cu_seq_k.stride()):
        if cu_seq_q.is_cuda and torch.cuda.is_current_stream_capturing():
            raise ValueError("self-attention only: pass the same cu_seqlens tensor as cu_seq_q and cu_seq_k "
                             "(two tensors cannot be compared during stream capture)")
        if cu_seq_q.shape != cu_seq_k.shape or not torch.equal(cu_seq_q, cu_seq_k.to(cu_seq_q.device)):
            raise ValueError("self-attention only: cu_seq_q and cu_seq_k must hold the same offsets")
    if max_q != max_k:
        raise ValueError("self-attention only: max_q and max_k must agree")
    if window_size is not None:
        left, right = window_size
        if left != -1 or right not in (0, -1):
            raise NotImplementedError("sliding windows are not part of this operator")
        causal = right == 0
    else:
        causal = True if is_causal is None else bool(is_causal)
    if return_aux is not None:
        raise NotImplementedError("return_aux is not supported")
    return dsa_varlen_attn(query, key, value, cu_seq_q, None if max_q is None else int(max_q), softmax_scale=scale,
                           causal=causal, **dsa)


def dispatch_varlen_attention(q, k, v, cu_seqlens, max_seqlen, causal: bool = True, **dsa):
    return varlen_attn(q, k, v, cu_seq_q=cu_seqlens, cu_seq_k=cu_seqlens, max_q=max_seqlen, max_k=max_seqlen,
                       window_size=(-1, 0) if causal else (-1, -1), **dsa)  # (total, num_heads, head_dim)


@torch.compiler.disable
def run_varlen_attn(q, k, v, cu_seqlens, max_seqlen, **dsa):
    return varlen_attn(q, k, v, cu_seq_q=cu_seqlens, cu_seq_k=cu_seqlens, max_q=max_seqlen, max_k=max_seqlen,
                       window_size=(-1, 0), **dsa)


def _hf_indexer_to_packed(x):
    # accepts packed (T,...) tensors as they are, or HF-style tensors with a leading batch dim of 1
    return x if x is None or x.dim() < 3 or x.shape[0] != 1 else x.squeeze(0)


_BOUND_ATTR = "_dsa_longest_segment"      # (version, storage offset, numel, bound), kept on the tensor that owns the memory


@torch.compiler.disable                 # reads a value back from the device and writes an attribute: never part of a traced graph
def longest_segment(cu_seqlens) -> int:
    """Longest segment of a packed row, read back from the device once per ``cu_seqlens`` tensor: every layer of a
    step hands over the same tensor (or a view of it), so the copy (and its stall) is paid once per batch instead of
    once per layer as in the reference (train/model_attention.py:120-121).

    The value is kept as an attribute of the tensor *object* that owns the memory (the view's base), together with
    that tensor's version counter: it dies with the tensor, an in-place write invalidates it, and a new tensor that
    happens to get a freed tensor's address starts without it.  (An address is no identity: the caching allocator
    hands the same block to every step's offsets.)  While a stream is being captured nothing may be copied to the
    host: None is returned, which the operator reads as the packed length, an upper bound."""
    if cu_seqlens.is_cuda and torch.cuda.is_current_stream_capturing():
        return None
    owner = cu_seqlens._base if cu_seqlens._base is not None else cu_seqlens
    key = (owner._version, cu_seqlens.storage_offset(), cu_seqlens.numel())
    hit = getattr(owner, _BOUND_ATTR, None)
    if hit is not None and hit[:3] == key:
        return hit[3]
    flat = cu_seqlens.reshape(-1)
    bound = max(int((flat[1:] - flat[:-1]).max()), 1) if flat.numel() > 1 else 1
    try:
        setattr(owner, _BOUND_ATTR, key + (bound,))
    except AttributeError:               # a tensor subclass with __slots__: no cache, one copy per call
        pass
    return bound


def varlen_attention_forward(query, key, value, attention_mask, max_seqlen=None, **dsa):
    """(1,Hq,T,D),(1,Hkv,T,D),(1,Hkv,T,D), cu_seqlens -> ((1,T,Hq,D), None).

    ``max_seqlen`` (keyword, not in the reference's signature): the longest segment if the caller holds it; otherwise
    it is read from ``cu_seqlens`` once per tensor (``longest_segment``).  The selection bitmap and the score rows of
    the DSA path are sized by it, so a tight bound matters there."""
    # tensor-parallel runs hand over DTensors sharded by head: the kernels see the local shard
    # (train/model_attention.py:104-106)
    query, key, value = (x.to_local() if hasattr(x, "to_local") else x for x in (query, key, value))
    # batch, head, seq_len, dim -> batch, seq_len, head, dim -> (T, head, dim)
    query = query.transpose(1, 2).contiguous()
    key = key.transpose(1, 2).contiguous()
    value = value.transpose(1, 2).contiguous()
    query = query.view(-1, query.size(-2), query.size(-1))
    key = key.view(-1, key.size(-2), key.size(-1))
    value = value.view(-1, value.size(-2), value.size(-1))
    cu_seqlens = attention_mask.squeeze()
    # The reference reads the longest segment back to the host here, once per layer (train/model_attention.py:120-121).
    # Any upper bound gives the same result; a tight one keeps the DSA workspaces small.
    bound = int(max_seqlen) if max_seqlen is not None else longest_segment(cu_seqlens)
    attn_output = varlen_attn(query, key, value, cu_seq_q=cu_seqlens, cu_seq_k=cu_seqlens, max_q=bound,
                              max_k=bound, window_size=(-1, 0), **dsa)
    if isinstance(attn_output, tuple):
        return (attn_output[0].unsqueeze(0), None) + tuple(attn_output[1:])
    return attn_output.unsqueeze(0), None


# ------------------------------------------------------------------------------------------------------------
# forwards for the HF attention classes (train/model_attention.py:146-252) and their installer (:255-299)
# ------------------------------------------------------------------------------------------------------------
def _hf_layer_forward(self, hidden_states, position_embeddings, attention_mask, gated: bool, offset: bool):
    """q/k/v projections -> fused norm + RoPE -> packed attention (-> gate) -> o_proj on an HF attention module
    (``self`` holds q_proj, k_proj, v_proj, o_proj, q_norm, k_norm, head_dim).  ``attention_mask`` carries the 1-D
    cu_seqlens (``return_mask`` below makes HF pass it through untouched).  Returns ``(attn_output, None)``."""
    from .dtensor_utils import _dtensor_rewrap, _dtensor_unwrap
    from .layers import attention_core
    input_shape = hidden_states.shape[:-1]
    D = self.head_dim
    total = 1
    for s_ in input_shape:
        total *= s_
    qp = self.q_proj(hidden_states)
    if gated:                                              # per head [q | gate] (train/model_attention.py:156-158)
        qg = qp.view(total, -1, 2 * D)
        k = self.k_proj(hidden_states).view(total, -1, D)
        v = self.v_proj(hidden_states).view(total, -1, D)
        (qg, k, v), wrap = _dtensor_unwrap(qg, k, v)
        q, gate = qg[..., :D], qg[..., D:]
    else:
        q = qp.view(total, -1, D)
        k = self.k_proj(hidden_states).view(total, -1, D)
        v = self.v_proj(hidden_states).view(total, -1, D)
        (q, k, v), wrap = _dtensor_unwrap(q, k, v)
        gate = None
    cos, sin = position_embeddings
    cu_seqlens = attention_mask.reshape(-1)
    out = attention_core(self, q, k, v, cos, sin, cu_seqlens, longest_segment(cu_seqlens), x=hidden_states, gate=gate,
                         offset=offset)
    out = _dtensor_rewrap(out, wrap)
    out = out.reshape(*input_shape, -1).to(hidden_states.dtype)
    return self.o_proj(out), None


def qwen3_5_forward(self, hidden_states, position_embeddings, attention_mask, **kwargs):
    """train/model_attention.py:146-185: gated, (1 + weight) norms."""
    return _hf_layer_forward(self, hidden_states, position_embeddings, attention_mask, gated=True, offset=True)


def qwen3_forward(self, hidden_states, position_embeddings, attention_mask, **kwargs):
    """train/model_attention.py:188-219."""
    return _hf_layer_forward(self, hidden_states, position_embeddings, attention_mask, gated=False, offset=False)


def qwen3vl_forward(self, hidden_states, position_embeddings, attention_mask, **kwargs):
    """train/model_attention.py:221-252."""
    return _hf_layer_forward(self, hidden_states, position_embeddings, attention_mask, gated=False, offset=False)


def return_mask(attention_mask, **kwargs):
    """Stands in for HF's ``create_causal_mask`` so that the raw cu_seqlens reaches the attention layers
    (train/model_attention.py:255-262)."""
    return attention_mask.unsqueeze_(0)


def replace_attention_qwenvl():
    """Install the forwards above on the HF Qwen3 / Qwen3-VL / Qwen3-VL-MoE / Qwen3.5 attention classes and replace
    their ``create_causal_mask`` (train/model_attention.py:265-299).  Returns the list of (owner, attribute, previous
    value) it replaced, so that a caller (or a test) can put everything back."""
    import importlib
    targets = (
        ("transformers.models.qwen3.modeling_qwen3", "Qwen3Attention", qwen3vl_forward),
        ("transformers.models.qwen3_vl.modeling_qwen3_vl", "Qwen3VLTextAttention", qwen3vl_forward),
        ("transformers.models.qwen3_vl_moe.modeling_qwen3_vl_moe", "Qwen3VLMoeTextAttention", qwen3vl_forward),
        ("transformers.models.qwen3_5.modeling_qwen3_5", "Qwen3_5Attention", qwen3_5_forward),
    )
    # resolve every target before touching any: a transformers build without one of the models then fails with
    # nothing patched
    resolved = []
    for mod_name, cls_name, fwd in targets:
        mod = importlib.import_module(mod_name)
        resolved.append((mod, getattr(mod, cls_name), fwd, mod.create_causal_mask))
    undo = []
    for mod, cls, fwd, mask_fn in resolved:
        undo.append((cls, "forward", cls.forward))
        cls.forward = fwd
        undo.append((mod, "create_causal_mask", mask_fn))
        mod.create_causal_mask = return_mask
    return undo
