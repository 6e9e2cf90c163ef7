"""Names of ``xattn/src/kernels.py`` of mit-han-lab/x-attention, kept as thin
seams over the fused HIP estimator.

The reference runs two Triton kernels back to back - the strided-reshape GEMM
and the softmax / block-sum pass over the score matrix it wrote.  Here both
live in one estimator that never materialises the scores.  The two names are
kept for callers that use them on their own: the first asks the estimator to
dump its raw scores, the second runs a stand-alone softmax / block-sum kernel
over a caller-supplied score matrix.  ``xattn_estimate`` uses neither.
"""
import math

import torch

from . import hip_backend as _hb
from .Xattention import _check_qk, _stream_ptr

__all__ = ["flat_group_gemm_fuse_reshape", "softmax_fuse_block_sum"]


def flat_group_gemm_fuse_reshape(query_states, key_states, stride, chunk_start, chunk_end, is_causal=True):
    """``out[m, n] = sum_i Q[m*S + S-1-i] . K[n*S + i]`` for a chunk of queries.

    Same contract as xattn/src/kernels.py:325-363: ``query_states`` is
    ``[1, H, q_len, 128]`` (a query chunk whose first reshaped row sits at key
    position ``chunk_start``), ``key_states`` ``[1, H_kv, kv_len, 128]``; both
    lengths multiples of ``stride * 128``; the result is ``[1, H, q_len/S,
    kv_len/S]`` in the input dtype.  With ``is_causal`` the 256x256 tiles that lie
    entirely beyond the chunk's diagonal are returned as zeros (the reference
    leaves its skipped 128x128 tiles uninitialised).
    """
    lib = _hb.lib()
    q = _check_qk(query_states, "query_states")
    k = _check_qk(key_states, "key_states")
    heads, q_len = q.shape[1], q.shape[2]
    kv_heads, kv_len = k.shape[1], k.shape[2]
    assert q_len % (stride * 128) == 0 and kv_len % (stride * 128) == 0
    n_rq, n_rk = q_len // stride, kv_len // stride
    assert chunk_end - chunk_start == n_rq
    out = torch.zeros((heads, n_rq, n_rk), dtype=torch.float32, device=q.device)
    k_used = k[:, :, : chunk_end * stride] if is_causal else k
    used_rk = k_used.shape[2] // stride
    chunk = stride * 128
    with torch.cuda.device(q.device):
        ws_bytes = lib.xattn_estimate_workspace_bytes(heads, q_len, k_used.shape[2], stride, 128, chunk, 0)
        if ws_bytes == 0:
            raise _hb.XattnHipError("estimator rejected the problem geometry")
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
        sums = torch.empty((heads, q_len // 128, k_used.shape[2] // 128), dtype=torch.float32, device=q.device)
        scores = out if used_rk == n_rk else torch.zeros((heads, n_rq, used_rk), dtype=torch.float32, device=q.device)
        _hb.check(
            lib.xattn_estimate_block_sums(
                q.data_ptr(), k_used.data_ptr(), sums.data_ptr(), ws.data_ptr(), ws_bytes, scores.data_ptr(),
                heads, kv_heads, q_len, k_used.shape[2], 128,
                q.stride(1), q.stride(2), k_used.stride(1), k_used.stride(2),
                stride, 128, chunk, 0, q_len // chunk, int(bool(is_causal)), 0,
                1.0 / math.sqrt(128) / stride, None, 0, 1, 1, -1, 0, 0, _stream_ptr(q.device),
            ),
            "xattn_estimate_block_sums",
        )
        if scores is not out:
            out[:, :, :used_rk] = scores
    return out.to(query_states.dtype).unsqueeze(0)


def softmax_fuse_block_sum(attn_weights_slice, reshaped_block_size, segment_size, chunk_start, chunk_end,
                           real_q_len, scale, is_causal=True):
    """Row softmax of a score matrix and its sums over
    ``reshaped_block_size`` x ``reshaped_block_size`` tiles.

    Same contract as xattn/src/kernels.py:238-289: ``attn_weights_slice`` is
    ``[1, H, q_r, k_r]`` raw scores of a query chunk whose row 0 sits at key
    position ``chunk_start``; ``scale`` multiplies them and already contains
    log2(e) (the softmax is taken with exp2); with ``is_causal`` row ``i`` sees
    keys ``<= chunk_start + i``; rows at positions ``>= real_q_len`` come out as
    zeros.  Returns ``[1, H, q_r / rbs, k_r / rbs]`` in the input dtype.
    ``segment_size`` only sets the reference kernel's inner tile; it is checked
    and otherwise unused.  The fused estimator does not go through here.
    """
    lib = _hb.lib()
    x = attn_weights_slice
    if not x.is_cuda:
        raise _hb.XattnHipError("attn_weights_slice must live on a ROCm device (no CPU fallback exists)")
    if x.dtype != torch.bfloat16:
        raise TypeError(f"attn_weights_slice must be torch.bfloat16, got {x.dtype}")
    batch_size, num_heads, q_len, k_len = x.shape
    assert batch_size == 1
    assert q_len % reshaped_block_size == 0
    assert k_len % segment_size == 0
    assert segment_size % reshaped_block_size == 0
    assert x.stride(-1) == 1
    assert chunk_end - chunk_start == q_len
    if x.stride(1) % 8 or x.stride(2) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    with torch.cuda.device(x.device):
        out = torch.empty((1, num_heads, q_len // reshaped_block_size, k_len // reshaped_block_size),
                          dtype=torch.float32, device=x.device)
        _hb.check(
            lib.xattn_softmax_block_sums(
                x.data_ptr(), out.data_ptr(), num_heads, q_len, k_len, x.stride(1), x.stride(2),
                reshaped_block_size, chunk_start, real_q_len, float(scale), int(bool(is_causal)),
                _stream_ptr(x.device),
            ),
            "xattn_softmax_block_sums",
        )
    return out.to(attn_weights_slice.dtype)
