"""Llama attention forward on the HIP prefill and decode kernels.

Mirror of xattn/src/load_llama.py of mit-han-lab/x-attention: the same
``FastPrefillConfig`` / ``forward_eval`` / ``load_model`` names, with three
differences that the kernels make possible:

* K and V keep their ``H_kv`` heads - the reference repeats them to ``H`` heads
  before the operator (``repeat_kv``, load_llama.py:158-159), the kernels share
  a KV head among its query heads instead;
* the decode step (one new token against the cache) runs on
  :func:`xattn.src.decode.single_decode_with_kv_cache` where the reference
  calls flashinfer (load_llama.py:180-197);
* ``metric="full"`` is the same attention kernel visiting every visible block
  (the reference calls flash-attn, xattn/src/Fullprefill.py).

``metric="flex"`` and ``metric="minfer"`` are other sparse-attention methods the
reference carries for comparison; they are not provided here.
"""
import inspect
import time

import torch

from .decode import single_decode_with_kv_cache
from .Xattention import Xattention_prefill, block_sparse_attention

__all__ = ["FastPrefillConfig", "forward_eval", "patch_model", "load_model", "apply_rotary_pos_emb", "rotate_half"]


def rotate_half(x):
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, unsqueeze_dim=1):
    """Rotate-half rotary embedding on ``[B, H, L, d]`` tensors (load_llama.py:41-65)."""
    cos, sin = cos.unsqueeze(unsqueeze_dim), sin.unsqueeze(unsqueeze_dim)
    return q * cos + rotate_half(q) * sin, k * cos + rotate_half(k) * sin


class FastPrefillConfig(dict):
    """Settings of the prefill path (load_llama.py:224-259).

    threshold:  float - one tau for every layer and head;
                tensor ``[layers, heads]`` - per-layer rows of per-head taus, as
                produced by the threshold profiler;
                None - the profiled table of this stride,
                ``xattn.threshold.llama_threshold.llama_fuse_<stride>``
                (``[layers][heads]``; load_llama.py:254-261).  That module reads
                the tables from a JSON file the profiler writes, or can be
                replaced by the reference's own module of the same name (tables
                profiled on Llama-3.1-8B-Instruct, parameters of that model,
                not shipped here); without either it raises ``ValueError``.
    stride:     antidiagonal stride, 4, 8 or 16.
    metric:     "xattn" or "full".
    print_detail: print per-stage wall times (synchronises the device).
    """

    def __init__(self, threshold=None, print_detail=False, stride=16, metric="xattn"):
        super().__init__()
        if stride not in (4, 8, 16):
            raise ValueError("stride must be 4, 8 or 16")
        if metric not in ("xattn", "full"):
            raise NotImplementedError(f"metric {metric!r}: only 'xattn' and 'full' are provided")
        self.print_detail = print_detail
        self.metric = metric
        self.stride = stride
        if threshold is None:
            # the profiled [layers, heads] table of this stride (xattn/src/load_llama.py:254-261);
            # raises ValueError naming where a table is looked for when there is none
            from xattn.threshold import llama_threshold as tables

            threshold = torch.tensor(getattr(tables, f"llama_fuse_{stride}"), dtype=torch.float32)
        if isinstance(threshold, torch.Tensor):
            if threshold.dim() != 2:
                raise ValueError("a threshold tensor must be [layers, heads]")
            self.threshold = threshold.detach().to(torch.float32)
        else:
            self.threshold = float(threshold)

    def layer_threshold(self, layer_idx):
        """tau of one layer: a float or a ``[heads]`` tensor."""
        if isinstance(self.threshold, torch.Tensor):
            return self.threshold[layer_idx]
        return self.threshold


def _is_static_cache(cache):
    try:
        from transformers import StaticCache
    except ImportError:
        return False
    return isinstance(cache, StaticCache)


def _stamp(cfg, label, start):
    if cfg.print_detail:
        torch.cuda.synchronize()
        print(f"     {label} took: {time.time() - start:.6f} seconds")
    return time.time()


def forward_eval(self, hidden_states, position_embeddings=None, attention_mask=None, past_key_values=None,
                 past_key_value=None, cache_position=None, position_ids=None, **kwargs):
    """Attention layer forward, prefill on XAttention and decode on the cache
    kernel (load_llama.py:80-220).  Bound to every ``self_attn`` by
    :func:`patch_model`; ``self.fastprefillconfig`` carries the settings.

    Batch size must be 1 (the operator's own limit, Xattention.py:357).  A
    call with one query token and a longer cache is a decode step; everything
    else (first prefill, or a further chunk of a chunked prefill on top of the
    cache) goes through the prefill operator, whose causal mask is aligned to
    the end of the cache.
    """
    cfg = self.fastprefillconfig
    start = time.time()
    bsz, q_len, _ = hidden_states.size()
    if bsz != 1:
        raise ValueError("the XAttention forward handles batch size 1")
    heads = self.config.num_attention_heads
    kv_heads = self.config.num_key_value_heads
    head_dim = self.head_dim

    query_states = self.q_proj(hidden_states).view(bsz, q_len, heads, head_dim).transpose(1, 2)
    key_states = self.k_proj(hidden_states).view(bsz, q_len, kv_heads, head_dim).transpose(1, 2)
    value_states = self.v_proj(hidden_states).view(bsz, q_len, kv_heads, head_dim).transpose(1, 2)
    start = _stamp(cfg, "Reshape", start)

    if position_embeddings is None:
        cos, sin = self.rotary_emb(value_states, position_ids)
    else:
        cos, sin = position_embeddings
    query_states, key_states = apply_rotary_pos_emb(query_states, key_states, cos, sin)

    cache = past_key_values if past_key_values is not None else past_key_value
    if cache is not None:
        cache_kwargs = {"sin": sin, "cos": cos, "cache_position": cache_position}
        key_states, value_states = cache.update(key_states, value_states, self.layer_idx, cache_kwargs)
        if _is_static_cache(cache):
            # a preallocated cache hands back its whole buffer: keep what is filled (load_llama.py:152-154).
            # The last position comes from cache_position where the model code passes it, else from position_ids.
            pos = cache_position if cache_position is not None else (position_ids[0] if position_ids is not None else None)
            if pos is None:
                raise ValueError("a static cache needs cache_position or position_ids to know how much of it is filled")
            # reading the position costs a device-to-host copy: the first layer of a model forward does it, the
            # other layers (handed the same positions) reuse its value.  Nothing here depends on tensor
            # identity or version counters, which inference-mode tensors do not have.
            memo = getattr(cfg, "_filled_memo", None)
            if memo is None or self.layer_idx in (0, None):
                last = int(pos[-1])
                cfg._filled_memo = (last,)
            else:
                last = memo[0]
            filled = min(last + 1, key_states.shape[2])
            key_states, value_states = key_states[:, :, :filled], value_states[:, :, :filled]
    if key_states.device != query_states.device:
        key_states = key_states.to(query_states.device)
        value_states = value_states.to(query_states.device)
    k_len = key_states.shape[2]
    decoding = q_len != k_len and q_len == 1
    start = _stamp(cfg, "Past KV update", start)
    if cfg.print_detail:
        print(f"q length: {q_len} k length: {k_len}")

    if decoding:
        attn_output = single_decode_with_kv_cache(
            query_states[0, :, 0], key_states[0], value_states[0], kv_layout="HND"
        )[None, :, None, :]
    elif cfg.metric == "xattn":
        threshold = cfg.layer_threshold(self.layer_idx)
        attn_output = Xattention_prefill(
            query_states, key_states, value_states, cfg.stride, norm=1, threshold=threshold, use_triton=True
        )
    else:
        attn_output = block_sparse_attention(query_states, key_states, value_states, causal=True)
    start = _stamp(cfg, "Attention computation", start)

    if attn_output.size() != (bsz, heads, q_len, head_dim):
        raise ValueError(
            f"`attn_output` should be of size {(bsz, heads, q_len, head_dim)}, but is {attn_output.size()}"
        )
    attn_output = attn_output.transpose(1, 2).reshape(bsz, q_len, heads * head_dim)
    attn_output = self.o_proj(attn_output)
    _stamp(cfg, "Post-attention processing", start)
    if getattr(self, "_xattn_three_outputs", False):
        return attn_output, None, cache
    return attn_output, None


def patch_model(model, fastprefillconfig):
    """Binds :func:`forward_eval` to every attention layer of a Llama model that
    is already in memory (what load_llama.py:283-285 does after loading)."""
    for layer in model.model.layers:
        attn = layer.self_attn
        if attn.head_dim != 128:
            raise ValueError("the kernels are built for head_dim 128")
        # older releases of the model code unpack three values from the layer's forward
        attn._xattn_three_outputs = "past_key_values" not in inspect.signature(type(attn).forward).parameters
        attn.fastprefillconfig = fastprefillconfig
        attn.forward = forward_eval.__get__(attn)
    return model


def load_model(fastprefillconfig=None, name_or_path=""):
    """Loads a Llama checkpoint in bf16 on the GPU and patches its attention
    (load_llama.py:261-290).  Returns ``(model, tokenizer)``."""
    from transformers import AutoTokenizer
    from transformers.models.llama.modeling_llama import LlamaForCausalLM

    if fastprefillconfig is None:
        fastprefillconfig = FastPrefillConfig()
    model = LlamaForCausalLM.from_pretrained(name_or_path, device_map="cuda", torch_dtype=torch.bfloat16)
    model.eval()
    patch_model(model, fastprefillconfig)
    return model, AutoTokenizer.from_pretrained(name_or_path)
