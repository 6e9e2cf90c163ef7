"""Names of ``xattn/src/kernels.py`` of mit-han-lab/x-attention, kept as thin
seams over the fused HIP estimator.

The reference runs two Triton kernels back to back - the strided-reshape GEMM
and the softmax / block-sum pass over the score matrix it wrote.  Here both
live in one estimator that never materialises the scores, so only the first
name has a stand-alone meaning: it asks the estimator to also dump its raw
scores (a debugging path).  ``softmax_fuse_block_sum`` on a caller-supplied
score matrix is not provided; ``xattn_estimate`` returns the block sums.
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
                1.0 / math.sqrt(128) / stride, None, 0, 1, _stream_ptr(q.device),
            ),
            "xattn_estimate_block_sums",
        )
        if scores is not out:
            out[:, :, :used_rk] = scores
    return out.to(query_states.dtype).unsqueeze(0)


def softmax_fuse_block_sum(*args, **kwargs):
    """Not available as a separate pass: the estimator fuses it (see
    ``xattn.src.Xattention.xattn_estimate``, which returns the block sums)."""
    raise NotImplementedError(
        "softmax_fuse_block_sum is fused into the HIP estimator; call xattn_estimate for the block sums"
    )
