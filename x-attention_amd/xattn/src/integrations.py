"""Attention-call shapes of the reference's other integrations, on the HIP kernels.

The reference patches three model families.  Llama has its own module
(:mod:`xattn.src.load_llama`); the other two differ only in how they call the
operator, and those call shapes are kept here as functions a model's attention
forward can use directly:

* Qwen2-VL (eval/VLMEvalKit/vlmeval/inference_video.py:135-149): XAttention
  prefill from a given layer on, dense prefill before it, a decode kernel when
  one token meets a longer cache - :func:`prefill_or_decode`;
* HunyuanVideo (eval/HunyuanVideo/hyvideo/modules/attenion.py:132-166):
  non-causal XAttention over the valid tokens of a padded sequence, dense
  attention among the padding, dense everywhere while the threshold is 1 (the
  warm-up steps) - :func:`valid_padded_attention`.

K and V keep their own head count everywhere (no ``repeat_kv``).
"""
import torch

from .decode import single_decode_with_kv_cache
from .Xattention import Xattention_prefill, block_sparse_attention

__all__ = ["prefill_or_decode", "valid_padded_attention"]


def prefill_or_decode(query_states, key_states, value_states, stride=16, threshold=0.9, sparse=True, causal=True):
    """``[1, H, q_len, 128]`` attention output for one layer call.

    One query token against a longer cache is a decode step; anything else is a
    prefill: XAttention when ``sparse`` (the reference switches it on per layer,
    ``layer_idx > 2`` for Qwen2-VL), dense FlashAttention otherwise.
    """
    q_len, k_len = query_states.shape[2], key_states.shape[2]
    if q_len == 1 and k_len > 1:
        if query_states.shape[0] != 1:
            raise ValueError("batch size 1 only")
        out = single_decode_with_kv_cache(query_states[0, :, 0], key_states[0], value_states[0], kv_layout="HND")
        return out[None, :, None, :]
    if sparse:
        return Xattention_prefill(query_states, key_states, value_states, stride, norm=1, threshold=threshold,
                                  use_triton=True, causal=causal)
    return block_sparse_attention(query_states, key_states, value_states, causal=causal)


def valid_padded_attention(q, k, v, cu_seqlens_q, cu_seqlens_kv, stride=8, threshold=0.95):
    """Non-causal attention of a padded sequence in two independent parts.

    ``q, k, v`` are ``[1, H, s, 128]``; tokens ``[0, cu_seqlens[1])`` are the valid
    ones and attend each other through XAttention (dense while ``threshold >= 1``),
    tokens ``[cu_seqlens[1], cu_seqlens[2])`` are padding and attend each other
    densely; the outputs are concatenated (attenion.py:132-166).
    """
    q0, q1 = int(cu_seqlens_q[1]), int(cu_seqlens_q[2])
    k0, k1 = int(cu_seqlens_kv[1]), int(cu_seqlens_kv[2])
    parts = []
    if q0 > 0:
        qa, ka, va = q[:, :, :q0], k[:, :, :k0], v[:, :, :k0]
        if threshold < 1:
            parts.append(Xattention_prefill(qa, ka, va, stride=stride, norm=1, threshold=threshold, causal=False, kdb=1))
        else:
            parts.append(block_sparse_attention(qa, ka, va, causal=False))
    if q1 > q0:
        parts.append(block_sparse_attention(q[:, :, q0:q1], k[:, :, k0:k1], v[:, :, k0:k1], causal=False))
    return torch.cat(parts, dim=2)
