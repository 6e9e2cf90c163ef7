"""Per-head threshold profiler on the HIP kernels.

Mirror of xattn/threshold/profile_threshold/profile_threshold.py of
mit-han-lab/x-attention: for every attention layer of a Llama model and every
calibration text, the fewest blocks holding ``coverage`` (0.9) of the TRUE
attention mass of each q-block row are found, the smallest antidiagonal
estimate among them is the row's cut, and the share of a head's total estimate
lying at or above the rows' cuts is that head's threshold for the text; the
maximum over texts is the profiled table (``[layers, heads]``), the input of
``FastPrefillConfig(threshold=...)``.

Differences from the reference: the true block mass comes from a kernel that
materialises nothing (the reference builds ``[128, L]`` probability slabs per
q-block in torch); K/V keep their ``H_kv`` heads; the layer's own attention
output is the dense HIP attention kernel (the reference calls flash-attn).
"""
import argparse
import json
import math

import torch

from xattn.src import hip_backend as _hb
from xattn.src.load_llama import apply_rotary_pos_emb
from xattn.src.Xattention import _check_qk, _stream_ptr, block_sparse_attention, estimate_and_select

__all__ = ["chunk_prefill_to_attn_sum", "profile_threshold_head", "xattn_prefill_profile", "forward_profile",
           "ProfileConfig", "profile_model"]


def chunk_prefill_to_attn_sum(query_states, key_states, block_size=128, causal=True):
    """True attention mass per 128x128 block, ``[1, H, Nq, Nk]`` fp32.

    Same quantity as profile_threshold.py:15-57 (softmax over the visible keys
    of each query row, summed over the block's rows and keys; rows past the
    sequence end carry nothing).  The reference always masks causally.
    """
    if block_size != 128:
        raise AssertionError("block_size must be 128")
    lib = _hb.lib()
    q = _check_qk(query_states, "query_states")
    k = _check_qk(key_states, "key_states")
    heads, q_len = q.shape[1], q.shape[2]
    kv_heads, k_len = k.shape[1], k.shape[2]
    nq, nk = (q_len + 127) // 128, (k_len + 127) // 128
    with torch.cuda.device(q.device):
        mass = torch.empty((1, heads, nq, nk), dtype=torch.float32, device=q.device)
        _hb.check(
            lib.xattn_block_mass(
                q.data_ptr(), k.data_ptr(), mass.data_ptr(), heads, kv_heads, q_len, k_len, 128,
                q.stride(1), q.stride(2), k.stride(1), k.stride(2), int(bool(causal)),
                1.0 / math.sqrt(128), _stream_ptr(q.device),
            ),
            "xattn_block_mass",
        )
    return mass


def profile_threshold_head(attn_sum, xattn_sum, coverage=0.9):
    """Per-head threshold from true block mass and estimate sums
    (profile_threshold.py:84-93).  ``attn_sum`` ``[1, H, Nq, Nk]`` fp32
    contiguous; ``xattn_sum`` ``[1, H, >=Nq, >=Nk]`` fp32 (the estimator's padded
    output is fine).  Returns ``[1, H]`` fp32."""
    lib = _hb.lib()
    _, heads, nq, nk = attn_sum.shape
    assert attn_sum.is_contiguous() and attn_sum.dtype == torch.float32
    assert xattn_sum.dtype == torch.float32 and xattn_sum.stride(3) == 1
    assert xattn_sum.shape[1] == heads and xattn_sum.shape[2] >= nq and xattn_sum.shape[3] >= nk
    with torch.cuda.device(attn_sum.device):
        rows = torch.empty((heads, nq, 2), dtype=torch.float32, device=attn_sum.device)
        _hb.check(
            lib.xattn_threshold_rows(
                attn_sum.data_ptr(), xattn_sum.data_ptr(), rows.data_ptr(), heads, nq, nk,
                xattn_sum.stride(1), xattn_sum.stride(2), float(coverage), _stream_ptr(attn_sum.device),
            ),
            "xattn_threshold_rows",
        )
    tot = rows.double().sum(1)
    return (tot[:, 0] / (tot[:, 1] + 1e-8)).float().unsqueeze(0)


class ProfileConfig:
    def __init__(self, stride=8, causal=True, coverage=0.9):
        self.stride = stride
        self.causal = causal
        self.coverage = coverage
        self.history_threshold = []   # one [layers, heads] tensor per text


def xattn_prefill_profile(self, query_states, key_states, value_states, block_size, stride, chunk_size=16384,
                          causal=True):
    """Profiles one layer on one text and returns the layer's (dense) attention
    output (profile_threshold.py:67-104)."""
    cfg = self.profile_config
    attn_sum = chunk_prefill_to_attn_sum(query_states, key_states, block_size)
    est = estimate_and_select(query_states, key_states, stride, 1.0, chunk_size, causal=causal, want_lists=False)
    # the estimate of a q-block row sums to block_size / stride, the true mass to block_size
    xattn_sum = est["sums"].unsqueeze(0) * stride
    threshold_head = profile_threshold_head(attn_sum, xattn_sum, cfg.coverage)
    if self.layer_idx == 0:
        cfg.history_threshold.append(threshold_head)
    else:
        cfg.history_threshold[-1] = torch.cat([cfg.history_threshold[-1], threshold_head], dim=0)
    return block_sparse_attention(query_states, key_states, value_states, causal=causal)


def forward_profile(self, hidden_states, position_embeddings=None, attention_mask=None, past_key_values=None,
                    past_key_value=None, cache_position=None, position_ids=None, **kwargs):
    """Attention layer forward used while profiling (profile_threshold.py:106-172): prefill only."""
    bsz, q_len, _ = hidden_states.size()
    if bsz != 1:
        raise ValueError("the profiler handles batch size 1")
    heads, kv_heads, head_dim = self.config.num_attention_heads, self.config.num_key_value_heads, self.head_dim
    query_states = self.q_proj(hidden_states).view(bsz, q_len, heads, head_dim).transpose(1, 2)
    key_states = self.k_proj(hidden_states).view(bsz, q_len, kv_heads, head_dim).transpose(1, 2)
    value_states = self.v_proj(hidden_states).view(bsz, q_len, kv_heads, head_dim).transpose(1, 2)
    if position_embeddings is None:
        cos, sin = self.rotary_emb(value_states, position_ids)
    else:
        cos, sin = position_embeddings
    query_states, key_states = apply_rotary_pos_emb(query_states, key_states, cos, sin)
    cache = past_key_values if past_key_values is not None else past_key_value
    if cache is not None:
        key_states, value_states = cache.update(
            key_states, value_states, self.layer_idx, {"sin": sin, "cos": cos, "cache_position": cache_position})
    assert key_states.shape[2] == q_len, "profiling runs on a plain prefill (no earlier cache content)"
    attn_output = xattn_prefill_profile(
        self, query_states, key_states, value_states, 128, self.profile_config.stride,
        causal=self.profile_config.causal)
    attn_output = self.o_proj(attn_output.transpose(1, 2).reshape(bsz, q_len, heads * head_dim))
    if getattr(self, "_xattn_three_outputs", False):
        return attn_output, None, cache
    return attn_output, None


def profile_model(model, profile_config, batches):
    """Binds :func:`forward_profile` to every attention layer, runs the model over
    ``batches`` (an iterable of ``input_ids`` tensors ``[1, L]``) and returns the
    profiled ``[layers, heads]`` table: the maximum over texts
    (profile_threshold.py:193-216)."""
    import inspect

    for layer in model.model.layers:
        attn = layer.self_attn
        attn._xattn_three_outputs = "past_key_values" not in inspect.signature(type(attn).forward).parameters
        attn.profile_config = profile_config
        attn.forward = forward_profile.__get__(attn)
    with torch.no_grad():
        for ids in batches:
            model(ids.to(model.device), use_cache=False)
    return torch.stack(profile_config.history_threshold).max(0)[0]


def main():
    from transformers import AutoTokenizer
    from transformers.models.llama.modeling_llama import LlamaForCausalLM

    parser = argparse.ArgumentParser()
    parser.add_argument("--name_or_path", type=str, default="meta-llama/Llama-3.1-8B-Instruct")
    parser.add_argument("--stride", type=int, default=8)
    parser.add_argument("--texts", type=str, default="xattn/threshold/profile_threshold/text.json",
                        help="JSON list of calibration texts")
    parser.add_argument("--out", type=str, default=None, help="write the table here (torch.save) instead of printing")
    parser.add_argument("--write-tables", type=str, default=None,
                        help="add the table as llama_fuse_<stride> to this JSON file, the form "
                             "xattn.threshold.llama_threshold reads for FastPrefillConfig()")
    args = parser.parse_args()
    model = LlamaForCausalLM.from_pretrained(args.name_or_path, device_map="cuda", torch_dtype=torch.bfloat16).eval()
    tokenizer = AutoTokenizer.from_pretrained(args.name_or_path)
    with open(args.texts) as f:
        texts = json.load(f)
    batches = (tokenizer(t, return_tensors="pt").input_ids for t in texts)
    table = profile_model(model, ProfileConfig(stride=args.stride), batches)
    if args.write_tables:
        from xattn.threshold.llama_threshold import write_tables

        write_tables(args.write_tables, **{f"llama_fuse_{args.stride}": table.float().cpu()})
    if args.out:
        torch.save(table, args.out)
    elif not args.write_tables:
        print(table.tolist())


if __name__ == "__main__":
    main()
