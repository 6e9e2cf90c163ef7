"""Single-token decode attention over a KV cache on the HIP kernel.

Stands where the reference's Llama attention forward calls the third-party
``flashinfer.single_decode_with_kv_cache(q, k, v, kv_layout="HND")``
(xattn/src/load_llama.py:180-197), with that function's name and the arguments
the reference uses, so the decode branch keeps its shape.
"""
import math

import torch

from . import hip_backend as _hb
from .Xattention import _stream_ptr

__all__ = ["single_decode_with_kv_cache"]


def single_decode_with_kv_cache(q, k, v, kv_layout="NHD", sm_scale=None, out=None, workspace=None,
                                static_scratch=False):
    """``out[h] = softmax(q[h] . K[h // g]^T * sm_scale) V[h // g]``.

    q ``[H, 128]``; k, v ``[kv_len, H_kv, 128]`` for ``kv_layout="NHD"`` (the
    third-party default) or ``[H_kv, kv_len, 128]`` for ``"HND"`` (what the
    reference passes); bf16 on one GPU, feature dimension contiguous, any head
    and token strides that are multiples of 8 elements (sliced cache views are
    taken as they are).  ``g = H / H_kv`` is at most 32.  ``sm_scale`` defaults
    to ``1/sqrt(128)``.  Returns ``[H, 128]`` in q's dtype.  ``workspace`` may
    carry a uint8 tensor of at least ``xattn_decode_workspace_bytes`` bytes to
    avoid the per-call allocation.  ``static_scratch=True`` (with ``out`` given)
    allocates nothing at all: the partial results go to a device array inside the
    library, shared by every such call on the GPU - calls that may overlap on
    one GPU must then be ordered by the caller.
    """
    lib = _hb.lib()
    if kv_layout not in ("NHD", "HND"):
        raise KeyError(f"Invalid kv_layout {kv_layout}")
    if q.dim() != 2 or k.dim() != 3 or v.dim() != 3:
        raise ValueError("q must be [H, d], k and v three-dimensional")
    if kv_layout == "NHD":
        k, v = k.transpose(0, 1), v.transpose(0, 1)
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise _hb.XattnHipError("single_decode_with_kv_cache runs on the GPU only (there is no CPU fallback)")
    if not (q.dtype == k.dtype == v.dtype == torch.bfloat16):
        raise ValueError("q, k, v must be bfloat16")
    if k.shape != v.shape:
        raise ValueError("k and v must have the same shape")
    heads, dim = q.shape
    kv_heads, kv_len = k.shape[0], k.shape[1]
    if dim != 128 or k.shape[2] != 128:
        raise ValueError("head_dim must be 128")
    if kv_len < 1:
        raise ValueError("the cache holds no token")
    if heads % kv_heads or heads // kv_heads > 32:
        raise ValueError("num_qo_heads must be a multiple (at most 32x) of num_kv_heads")
    if k.device != q.device or v.device != q.device:
        raise ValueError("q, k, v must live on one device")
    if q.stride(1) != 1:
        q = q.contiguous()
    if k.stride(2) != 1 or k.stride(0) % 8 or k.stride(1) % 8 or k.data_ptr() % 16:
        k = k.contiguous()
    if v.stride(2) != 1 or v.stride(0) % 8 or v.stride(1) % 8 or v.data_ptr() % 16:
        v = v.contiguous()
    if q.stride(0) % 8 or q.data_ptr() % 16:
        q = q.clone(memory_format=torch.contiguous_format)
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(128)
    with torch.cuda.device(q.device):
        ws_bytes = lib.xattn_decode_workspace_bytes(heads, kv_heads, kv_len)
        if static_scratch:
            if workspace is not None:
                raise ValueError("static_scratch and workspace exclude each other")
        elif workspace is None:
            workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
        elif workspace.numel() * workspace.element_size() < ws_bytes or workspace.device != q.device:
            raise ValueError(f"workspace must hold {ws_bytes} bytes on {q.device}")
        if out is None:
            out = torch.empty((heads, 128), dtype=q.dtype, device=q.device)
        elif out.shape != (heads, 128) or out.dtype != q.dtype or out.stride(1) != 1 or out.device != q.device:
            raise ValueError("out must be [H, 128], q's dtype and device, rows contiguous")
        if static_scratch:
            _hb.check(
                lib.xattn_decode_fwd_static(
                    q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), heads, kv_heads, kv_len, 128,
                    q.stride(0), k.stride(0), k.stride(1), v.stride(0), v.stride(1), out.stride(0),
                    float(sm_scale), _stream_ptr(q.device),
                ),
                "xattn_decode_fwd_static",
            )
            return out
        _hb.check(
            lib.xattn_decode_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), workspace.data_ptr(),
                workspace.numel() * workspace.element_size(), heads, kv_heads, kv_len, 128,
                q.stride(0), k.stride(0), k.stride(1), v.stride(0), v.stride(1), out.stride(0),
                float(sm_scale), _stream_ptr(q.device),
            ),
            "xattn_decode_fwd",
        )
    return out
