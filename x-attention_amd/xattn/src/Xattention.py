"""XAttention prefill operator on MI355X: same names, arguments and results as
``xattn/src/Xattention.py`` of mit-han-lab/x-attention, computed by the HIP
kernels of ``libxattn_hip.so``.

Differences a caller can rely on:

* ``key_states`` / ``value_states`` may carry fewer heads than ``query_states``
  (grouped-query attention by KV-head sharing; the reference asserts equal
  head counts and its callers ``repeat_kv`` first).  Passing repeated K/V
  still works.
* ``use_triton`` selects which of the reference's two estimator branches is
  reproduced, both on the HIP kernels: ``True`` (the default everywhere in the
  reference's integrations) gives the Triton-branch result, where every query
  chunk sees all earlier keys; ``False`` gives the torch-branch result, which
  for ``k_len % chunk_size == 0`` restricts each query chunk to the keys of
  its own chunk (xattn/src/Xattention.py:201).
* block sums are kept in fp32 for the selection; ``attn_sums`` is cast to the
  query dtype only on return.
* tensors must be bf16 on a ROCm device; there is no CPU or eager fallback.
"""
import math

import torch

from . import hip_backend as _hb

__all__ = ["Xattention_prefill", "xattn_estimate", "default_chunk_size", "estimate_and_select", "block_sparse_attention"]

BLOCK = 128
WORKSPACE_LIMIT = 2 << 30   # bytes of estimator workspace per launch
GROUP_LIMIT = 2 << 30       # bytes of block sums + column lists the operator holds at a time


def default_chunk_size(k_len):
    """Chunk rule of xattn/src/Xattention.py:322-331 (chunk * 2^ceil(log2 k_len) <= 2^28)."""
    p = 1 << (k_len - 1).bit_length()
    return int(max(min(max(2048, p), 128 * 1024 * 2048 // p), 2048))


def _stream_ptr(device):
    return torch.cuda.current_stream(device).cuda_stream


def _mark(marks, label):
    if marks is not None:
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        marks.append((label, ev))


def _check_qk(x, name):
    if not x.is_cuda:
        raise _hb.XattnHipError(f"{name} must live on a ROCm device (no CPU fallback exists)")
    if x.dtype != torch.bfloat16:
        raise TypeError(f"{name} must be torch.bfloat16, got {x.dtype}")
    if x.dim() != 4 or x.shape[0] != 1:
        raise AssertionError(f"{name} must be [1, heads, len, 128] (batch 1 only)")
    if x.shape[-1] != 128:
        raise AssertionError("head_dim must be 128")
    if x.stride(-1) != 1 or x.stride(1) % 8 or x.stride(2) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    return x


def slab_pairs_for(select_mode, stride, perm=None):
    """(query offset, key offset) pairs of the reshape for a ``select_mode`` of
    xattn/src/Xattention.py:72-135, or None for the default antidiagonal one.
    A pair (a, b) adds ``Q[m*S + a] . K[n*S + b]`` to score[m, n]."""
    S = stride
    if select_mode in ("inverse", ""):
        return None
    if select_mode == "slash":
        return [(i, i) for i in range(S)]
    if select_mode == "random":
        if perm is None:
            perm = torch.randperm(S)
        return [(int(perm[i]), i) for i in range(S)]
    if select_mode == "double":
        # key slab i becomes K_i + K_(i+1): each query offset meets two key offsets
        return [(S - 1 - i, i) for i in range(S)] + [(S - 1 - i, (i + 1) % S) for i in range(S)]
    if select_mode == "triple":
        # ... then that sum plus its own right-rolled copy: K_(i-1) + 2 K_i + K_(i+1)
        base = [(S - 1 - i, i) for i in range(S)]
        return base + base + [(S - 1 - i, (i + 1) % S) for i in range(S)] + [(S - 1 - i, (i - 1) % S) for i in range(S)]
    raise ValueError(f"unknown select_mode {select_mode!r}")


def _tau_per_head(threshold, heads, device):
    """float, 0-d tensor or [H] tensor -> float64 [H] on device, rounded the way
    the reference rounds it (a tensor keeps its own precision, utils.py:91-92)."""
    if isinstance(threshold, torch.Tensor):
        t = threshold.detach().to(torch.float64).reshape(-1)
        if t.numel() == 1:
            t = t.expand(heads)
        if t.numel() != heads:
            raise ValueError(f"threshold tensor must have 1 or {heads} entries")
        return t.contiguous().to(device)
    return torch.full((heads,), float(threshold), dtype=torch.float64, device=device)


class _Plan:
    """Geometry, buffers and kernel launchers of one estimate -> select pass."""

    def __init__(self, query_states, key_states, stride, threshold, chunk_size, causal, norm, use_triton,
                 keep_sink, keep_recent, block_size, want_lists, dump_scores, slab_pairs=None, softmax=True, kdb=1,
                 want_mask=True, group_limit=None, want_sums=True):
        self.lib = _hb.lib()
        self.kdb = int(kdb)
        self.softmax = bool(softmax)
        self.n_pairs = 0 if slab_pairs is None else len(slab_pairs)
        self.pairs = None
        if self.n_pairs:
            flat = [int(v) for pr in slab_pairs for v in pr]
            self.pairs = (_hb.c_i32 * len(flat))(*flat)
        q = _check_qk(query_states, "query_states")
        k = _check_qk(key_states, "key_states")
        if k.device != q.device:
            k = k.to(q.device)
        self.q, self.k = q, k
        self.heads, self.q_len = q.shape[1], q.shape[2]
        self.kv_heads, self.k_len = k.shape[1], k.shape[2]
        if block_size != BLOCK:
            raise AssertionError("block_size must be 128")
        if stride not in (4, 8, 16):
            raise ValueError("stride must be 4, 8 or 16")
        if self.heads % self.kv_heads:
            raise AssertionError("query heads must be a multiple of key/value heads")
        if chunk_size % block_size:
            raise AssertionError("chunk_size must be a multiple of block_size")
        if self.kdb != 1:
            if use_triton:
                raise ValueError("use_triton and kdb cannot be used together")     # xattn/src/Xattention.py:140-141
            if self.kdb < 1 or (block_size // stride) % self.kdb or self.n_pairs:
                raise ValueError("kdb must divide block_size // stride and needs select_mode='inverse'")
        if not norm > 0:
            raise ValueError("norm must be positive")
        self.stride, self.chunk_size, self.block_size = stride, chunk_size, block_size
        self.causal, self.keep_sink, self.keep_recent = bool(causal), bool(keep_sink), bool(keep_recent)
        dev = self.dev = q.device
        q_pad = -self.q_len % chunk_size
        k_pad = -self.k_len % chunk_size
        self.q_chunks = (self.q_len + q_pad) // chunk_size
        assert (self.k_len + k_pad) // chunk_size >= self.q_chunks
        self.nqb, self.nkb = (self.q_len + q_pad) // block_size, (self.k_len + k_pad) // block_size
        self.blocks_per_chunk = chunk_size // block_size
        # the torch branch hides "the last k_pad // stride reshaped keys" with a slice that covers every key
        # when that count is 0 (xattn/src/Xattention.py:67,201) - also when 0 < k_pad < stride
        self.own_chunk_only = self.causal and (not use_triton) and k_pad // stride == 0
        self.scale = 1.0 / math.sqrt(128) / stride / norm
        # Query rows (after subsampling) from which the block sums are all-zero.  Torch branch: the last
        # q_pad // stride // kdb rows of the last chunk - all of that chunk when that count is 0 but there is
        # padding, the slice [-0:] of xattn/src/Xattention.py:237-238.  Triton branch: rows whose position on
        # the key axis is at or beyond the real reshaped key length (xattn/src/kernels.py:70, Xattention.py:169).
        n_rq = (self.q_len + q_pad) // stride // self.kdb
        if use_triton:
            self.zero_rows_from = max(0, n_rq - k_pad // stride)
        elif q_pad // stride == 0:
            self.zero_rows_from = n_rq
        elif q_pad // stride // self.kdb == 0:
            self.zero_rows_from = n_rq - chunk_size // stride // self.kdb
        else:
            self.zero_rows_from = n_rq - q_pad // stride // self.kdb
        self.list_cols = (self.k_len + block_size - 1) // block_size
        # The estimator's workspace grows with (query rows per call) x (key blocks); very long
        # sequences are processed in groups of query chunks that keep it under WORKSPACE_LIMIT.
        per_chunk = self.lib.xattn_estimate_workspace_bytes(
            self.heads, self.q_len, self.k_len, stride, block_size, chunk_size, 1)
        if per_chunk == 0:
            raise _hb.XattnHipError("estimator rejected the problem geometry")
        self.chunks_per_call = max(1, min(self.q_chunks, WORKSPACE_LIMIT // per_chunk))
        self.ws_bytes = self.lib.xattn_estimate_workspace_bytes(
            self.heads, self.q_len, self.k_len, stride, block_size, chunk_size, self.chunks_per_call)
        # Block sums, mask and column lists hold a window of q-block rows: all of them, or - when a byte
        # limit is given and they would exceed it - one group of whole query chunks at a time, which the
        # caller works through with window(); the buffers are reused from group to group.
        # Without the block sums (the operator never looks at them) normalisation and selection run as one
        # pass that keeps them in LDS; rows of more than 8192 key blocks and subsampled query rows go
        # through memory (xattn_estimate_select's limits).
        self.fused = (not want_sums) and (not dump_scores) and self.kdb == 1 and self.nkb <= 8192
        per_row = self.heads * ((0 if self.fused else self.nkb * 4) + (self.nkb if want_mask else 0)
                                + ((self.list_cols + 1) * 4 if want_lists else 0))
        self.chunks_per_group = self.q_chunks
        if group_limit is not None and per_row * self.nqb > group_limit:
            self.chunks_per_group = max(1, min(self.q_chunks, group_limit // (per_row * self.blocks_per_chunk)))
        self.win_rows = self.chunks_per_group * self.blocks_per_chunk
        self.win_row0 = 0
        with torch.cuda.device(dev):
            self.workspace = torch.empty(self.ws_bytes, dtype=torch.uint8, device=dev)
            self.sums = None
            if not self.fused:
                self.sums = torch.empty((self.heads, self.win_rows, self.nkb), dtype=torch.float32, device=dev)
            self.scores = None
            if dump_scores:
                self.scores = torch.zeros(
                    (self.heads, (self.q_len + q_pad) // stride // self.kdb, (self.k_len + k_pad) // stride),
                    dtype=torch.float32, device=dev)
            self.tau = _tau_per_head(threshold, self.heads, dev)
            self.mask = None
            if want_mask:
                self.mask = torch.empty((self.heads, self.win_rows, self.nkb), dtype=torch.uint8, device=dev)
            self.col_idx = self.col_cnt = None
            if want_lists:
                self.col_idx = torch.empty((self.heads, self.win_rows, self.list_cols), dtype=torch.int32, device=dev)
                self.col_cnt = torch.empty((self.heads, self.win_rows), dtype=torch.int32, device=dev)

    def groups(self):
        """(first chunk, end chunk) of every group of query chunks the buffers can hold."""
        return [(c, min(self.q_chunks, c + self.chunks_per_group))
                for c in range(0, self.q_chunks, self.chunks_per_group)]

    def window(self, chunk_begin):
        """Points the buffers at the group of query chunks that starts at ``chunk_begin``."""
        self.win_row0 = chunk_begin * self.blocks_per_chunk

    def estimate(self, chunk_begin, chunk_end, stream):
        if chunk_end - chunk_begin > self.chunks_per_call:
            for c in range(chunk_begin, chunk_end, self.chunks_per_call):
                self.estimate(c, min(chunk_end, c + self.chunks_per_call), stream)
            return
        q, k = self.q, self.k
        _hb.check(
            self.lib.xattn_estimate_block_sums(
                q.data_ptr(), k.data_ptr(), self.sums.data_ptr(), self.workspace.data_ptr(), self.ws_bytes,
                self.scores.data_ptr() if self.scores is not None else None,
                self.heads, self.kv_heads, self.q_len, self.k_len, 128,
                q.stride(1), q.stride(2), k.stride(1), k.stride(2),
                self.stride, self.block_size, self.chunk_size, chunk_begin, chunk_end,
                int(self.causal), int(self.own_chunk_only), self.scale, self.pairs, self.n_pairs,
                int(self.softmax), self.kdb, self.zero_rows_from, self.win_row0, self.win_rows, stream,
            ),
            "xattn_estimate_block_sums",
        )

    def estimate_select(self, chunk_begin, chunk_end, stream, stages=3):
        """Estimator and selection of query chunks [chunk_begin, chunk_end) without block sums in memory
        (``self.fused`` plans only).  ``stages``: 1 = the MFMA pass, 2 = normalise and select, 3 = both."""
        if chunk_end - chunk_begin > self.chunks_per_call:
            for c in range(chunk_begin, chunk_end, self.chunks_per_call):
                self.estimate_select(c, min(chunk_end, c + self.chunks_per_call), stream, stages)
            return
        q, k = self.q, self.k
        lists = self.col_idx is not None
        _hb.check(
            self.lib.xattn_estimate_select(
                q.data_ptr(), k.data_ptr(), None, self.workspace.data_ptr(), self.ws_bytes,
                self.heads, self.kv_heads, self.q_len, self.k_len, 128,
                q.stride(1), q.stride(2), k.stride(1), k.stride(2),
                self.stride, self.block_size, self.chunk_size, chunk_begin, chunk_end,
                int(self.causal), int(self.own_chunk_only), self.scale, self.pairs, self.n_pairs,
                int(self.softmax), self.zero_rows_from, self.win_row0, self.win_rows,
                self.tau.data_ptr(), self.mask.data_ptr() if self.mask is not None else None,
                self.col_idx.data_ptr() if lists else None, self.col_cnt.data_ptr() if lists else None,
                self.list_cols, int(self.keep_sink), int(self.keep_recent), stages, stream,
            ),
            "xattn_estimate_select",
        )

    def run(self, chunk_begin, chunk_end, stream):
        """Estimate and selection of query chunks [chunk_begin, chunk_end), by whichever path the plan uses."""
        if self.fused:
            self.estimate_select(chunk_begin, chunk_end, stream)
        else:
            self.estimate(chunk_begin, chunk_end, stream)
            self.select(chunk_begin * self.blocks_per_chunk, chunk_end * self.blocks_per_chunk, stream)

    def select(self, row_begin, row_end, stream):
        lists = self.col_idx is not None
        _hb.check(
            self.lib.xattn_select_blocks(
                self.sums.data_ptr(), self.tau.data_ptr(), self.mask.data_ptr() if self.mask is not None else None,
                self.col_idx.data_ptr() if lists else None, self.col_cnt.data_ptr() if lists else None,
                self.list_cols, self.heads, self.nqb, self.nkb, row_begin, row_end, self.nkb - self.nqb,
                int(self.causal), int(self.keep_sink), int(self.keep_recent),
                self.list_cols, self.q_len, self.k_len - self.q_len, self.blocks_per_chunk,
                self.win_row0, self.win_rows, stream,
            ),
            "xattn_select_blocks",
        )

    def result(self):
        return dict(sums=self.sums, mask=self.mask, col_idx=self.col_idx, col_cnt=self.col_cnt,
                    scores=self.scores, tau=self.tau)


def estimate_and_select(
    query_states,
    key_states,
    stride,
    threshold,
    chunk_size,
    causal=True,
    norm=1,
    use_triton=True,
    keep_sink=False,
    keep_recent=False,
    block_size=BLOCK,
    want_lists=True,
    dump_scores=False,
    marks=None,
    slab_pairs=None,
    softmax=True,
    kdb=1,
    want_mask=True,
    want_sums=True,
):
    """Runs the estimator and selection kernels over all query chunks, one launch each.

    Returns a dict with fp32 ``sums`` [H, Nq_p, Nk_p], uint8 ``mask`` of the same
    shape, and (when ``want_lists``) ``col_idx`` [H, Nq_p, pitch] / ``col_cnt``
    [H, Nq_p] for :func:`block_sparse_attention` (``want_mask=False`` skips the
    byte mask, which the attention kernel does not read).

    ``want_sums=False`` (what the operator asks for) leaves ``sums`` out of the
    result: normalisation and selection then run as one pass that keeps the block
    sums in LDS (``xattn_estimate_select``); lists and mask are the same.

    ``marks``, when a list, receives ``(label, torch.cuda.Event)`` pairs recorded
    on the current stream before the estimator, between its MFMA pass and what
    follows (normalisation + selection, or - with block sums - between
    estimator and selection) and after selection (for per-kernel timing).
    """
    plan = _Plan(query_states, key_states, stride, threshold, chunk_size, causal, norm, use_triton,
                 keep_sink, keep_recent, block_size, want_lists, dump_scores, slab_pairs, softmax, kdb,
                 want_mask=want_mask, want_sums=want_sums)
    with torch.cuda.device(plan.dev):
        stream = _stream_ptr(plan.dev)
        _mark(marks, "estimate_begin")
        if plan.fused and marks is None:
            plan.estimate_select(0, plan.q_chunks, stream)
        elif plan.fused:
            # the two passes as separate calls, so that an event can sit between them
            for c in range(0, plan.q_chunks, plan.chunks_per_call):
                plan.estimate_select(c, min(plan.q_chunks, c + plan.chunks_per_call), stream, stages=1)
                if c == 0 and plan.chunks_per_call >= plan.q_chunks:
                    _mark(marks, "select_begin")
                plan.estimate_select(c, min(plan.q_chunks, c + plan.chunks_per_call), stream, stages=2)
            if plan.chunks_per_call < plan.q_chunks:
                _mark(marks, "select_begin")
        else:
            plan.estimate(0, plan.q_chunks, stream)
            _mark(marks, "select_begin")
            plan.select(0, plan.nqb, stream)
        _mark(marks, "select_end")
    return plan.result()


def xattn_estimate(
    query_states,
    key_states,
    block_size,
    stride,
    norm=1,
    softmax=True,
    threshold=0.9,
    chunk_size=16384,
    select_mode="inverse",
    use_triton=True,
    causal=True,
    kdb: int = 1,
    keep_sink=False,
    keep_recent=False,
):
    """Antidiagonal block scores and the thresholded block mask.

    Same contract as xattn/src/Xattention.py:13-299: returns
    ``(attn_sums, simple_masks)``, both ``[1, H, Nq_p, Nk_p]`` over the lengths
    padded to multiples of ``chunk_size``; ``attn_sums`` in the query dtype,
    ``simple_masks`` bool.  ``select_mode`` ("inverse", "slash", "random",
    "double", "triple"; the reference has the last four in its torch branch only,
    Xattention.py:72-135) and ``softmax=False`` (:231-234) run on the same
    kernel; "random" draws ``torch.randperm(stride)`` like the reference.
    ``kdb != 1`` (every kdb-th reshaped query row, :88-93, :174-181, :217-222,
    :245) exists in the reference's torch branch only: it needs
    ``use_triton=False`` (the reference raises otherwise, :140-141) and the
    default ``select_mode``.
    """
    if kdb != 1 and use_triton:
        raise ValueError("use_triton and kdb cannot be used together")
    r = estimate_and_select(
        query_states, key_states, stride, threshold, chunk_size, causal=causal, norm=norm,
        use_triton=use_triton, keep_sink=keep_sink, keep_recent=keep_recent, block_size=block_size,
        want_lists=False, slab_pairs=slab_pairs_for(select_mode, stride), softmax=softmax, kdb=kdb,
    )
    attn_sums = r["sums"].to(query_states.dtype).unsqueeze(0)
    simple_masks = r["mask"].view(torch.bool).unsqueeze(0)
    return attn_sums, simple_masks


def block_sparse_attention(query_states, key_states, value_states, col_idx=None, col_cnt=None,
                           causal=True, softmax_scale=None, out=None, q_blocks=None, stream=None, idx_row0=0):
    """Attention of each 128-token query block over the key blocks listed for it
    (``col_idx``/``col_cnt`` as written by :func:`estimate_and_select`; ``None``
    visits every visible block = dense FlashAttention).  Stands in for
    ``block_sparse_attn_func`` at xattn/src/Xattention.py:377-391.
    Returns ``[1, H, q_len, 128]`` as a transposed view of ``[1, q_len, H, 128]``.
    ``out`` (a ``[1, q_len, H, 128]`` buffer), ``q_blocks=(begin, end)`` and ``stream``
    (a ``torch.cuda.Stream``) let a caller fill the output chunk by chunk;
    ``idx_row0`` says which q-block row 0 of ``col_idx``/``col_cnt`` holds when
    the lists cover a window of q-blocks only.
    """
    lib = _hb.lib()
    q = _check_qk(query_states, "query_states")
    k = _check_qk(key_states, "key_states")
    v = _check_qk(value_states, "value_states")
    dev = q.device
    if k.device != dev:
        k = k.to(dev)
    if v.device != dev:
        v = v.to(dev)
    heads, q_len = q.shape[1], q.shape[2]
    kv_heads, k_len = k.shape[1], k.shape[2]
    if v.shape[1] != kv_heads or v.shape[2] != k_len:
        raise AssertionError("key_states and value_states must agree in heads and length")
    if (col_idx is None) != (col_cnt is None):
        raise AssertionError("col_idx and col_cnt go together")
    out_given = out is not None
    if out is None:
        out = torch.empty((1, q_len, heads, 128), dtype=torch.bfloat16, device=dev)
    qb0, qb1 = q_blocks if q_blocks is not None else (0, -1)
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(128)
    if col_idx is not None:
        assert col_idx.dtype == torch.int32 and col_cnt.dtype == torch.int32
        assert col_idx.is_contiguous() and col_cnt.is_contiguous()
        assert col_idx.shape[0] == heads and col_cnt.shape == col_idx.shape[:2]
        pitch, idx_rows = col_idx.shape[2], col_idx.shape[1]
        if q_blocks is None:
            qb0, qb1 = idx_row0, min((q_len + 127) // 128, idx_row0 + idx_rows)
            if out_given is False and (qb0 != 0 or qb1 != (q_len + 127) // 128):
                # lists that cover only some q-blocks fill only those rows of the output: a caller who means
                # that passes the buffer to fill (and usually q_blocks); a fresh buffer would come back with
                # uninitialised rows
                raise ValueError("col_idx / col_cnt do not cover every q-block: pass `out` (and `q_blocks`) to fill part of it")
    else:
        pitch, idx_rows = 0, 0
    with torch.cuda.device(dev):
        stream_ptr = stream.cuda_stream if stream is not None else _stream_ptr(dev)
        _hb.check(
            lib.xattn_block_sparse_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                col_idx.data_ptr() if col_idx is not None else None,
                col_cnt.data_ptr() if col_cnt is not None else None,
                pitch, idx_rows, idx_row0, heads, kv_heads, q_len, k_len, 128,
                q.stride(1), q.stride(2), k.stride(1), k.stride(2), v.stride(1), v.stride(2),
                out.stride(2), out.stride(1), qb0, qb1, int(bool(causal)), scale,
                stream_ptr,
            ),
            "xattn_block_sparse_fwd",
        )
    return out.transpose(1, 2)


def Xattention_prefill(
    query_states,
    key_states,
    value_states,
    stride,
    norm=1,
    threshold=0.8,
    block_size=128,
    use_triton=True,
    causal=True,
    kdb=1,
    chunk_size=None,
    keep_sink=False,
    keep_recent=False,
    pipeline_chunks=False,
):
    """Sparse prefill attention: antidiagonal estimate -> block selection ->
    block-sparse FlashAttention.  Signature, defaults and result layout of
    xattn/src/Xattention.py:302-402.  ``pipeline_chunks=True`` (not in the
    reference) issues the three stages query chunk by query chunk on separate HIP
    streams instead of one launch per stage; the result is the same."""
    batch_size, _, k_len, _ = key_states.shape
    assert block_size == 128
    assert batch_size == 1
    if chunk_size is None:
        chunk_size = default_chunk_size(k_len)
    if pipeline_chunks:
        return _prefill_pipelined(query_states, key_states, value_states, stride, norm, threshold, block_size,
                                  use_triton, causal, chunk_size, keep_sink, keep_recent, kdb)
    # One launch per stage when the block sums and column lists of the whole sequence fit GROUP_LIMIT
    # (128k tokens: 0.26 GB); longer sequences go through the three stages one group of query chunks at a
    # time on buffers of one group, so the extra memory stays bounded however long the sequence is.
    plan = _Plan(query_states, key_states, stride, threshold, chunk_size, causal, norm, use_triton,
                 keep_sink, keep_recent, block_size, True, False, kdb=kdb, want_mask=False, group_limit=GROUP_LIMIT,
                 want_sums=False)
    dev = plan.dev
    v = _check_qk(value_states, "value_states")
    nb = (plan.q_len + block_size - 1) // block_size
    with torch.cuda.device(dev):
        stream = _stream_ptr(dev)
        out = torch.empty((1, plan.q_len, plan.heads, 128), dtype=torch.bfloat16, device=dev)
        bpc = plan.blocks_per_chunk
        for c0, c1 in plan.groups():
            plan.window(c0)
            plan.run(c0, c1, stream)
            qb0, qb1 = c0 * bpc, min(nb, c1 * bpc)
            if qb0 < qb1:
                block_sparse_attention(plan.q, plan.k, v, plan.col_idx, plan.col_cnt, causal=causal, out=out,
                                       q_blocks=(qb0, qb1), idx_row0=plan.win_row0)
    return out.transpose(1, 2)


_side_streams = {}


def _streams(dev):
    """Two side streams per device, default priority, created once."""
    key = (dev.type, dev.index)
    if key not in _side_streams:
        _side_streams[key] = (torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev))
    return _side_streams[key]


def _prefill_pipelined(query_states, key_states, value_states, stride, norm, threshold, block_size, use_triton,
                       causal, chunk_size, keep_sink, keep_recent, kdb=1):
    """Chunk-by-chunk orchestration on three HIP streams: the estimator of query
    chunk c runs on the caller's stream, the selection of chunk c on a second
    stream as soon as its block sums exist, and the attention of chunk c's query
    blocks on a third as soon as its column lists exist - so selection and
    attention of earlier chunks fill the compute units the estimator's tail
    leaves idle.  The caller's stream waits for both side streams before the
    function returns, which also makes every temporary safe to free."""
    plan = _Plan(query_states, key_states, stride, threshold, chunk_size, causal, norm, use_triton,
                 keep_sink, keep_recent, block_size, True, False, kdb=kdb)
    dev = plan.dev
    q = plan.q
    k = plan.k
    v = _check_qk(value_states, "value_states")
    if v.device != dev:
        v = v.to(dev)
    nb = (plan.q_len + block_size - 1) // block_size
    with torch.cuda.device(dev):
        main = torch.cuda.current_stream(dev)
        s_sel, s_att = _streams(dev)
        out = torch.empty((1, plan.q_len, plan.heads, 128), dtype=torch.bfloat16, device=dev)
        start = torch.cuda.Event()
        start.record(main)
        s_sel.wait_event(start)
        s_att.wait_event(start)
        bpc = plan.blocks_per_chunk
        for c in range(plan.q_chunks):
            plan.estimate(c, c + 1, main.cuda_stream)
            ev = torch.cuda.Event()
            ev.record(main)
            s_sel.wait_event(ev)
            plan.select(c * bpc, (c + 1) * bpc, s_sel.cuda_stream)
            ev2 = torch.cuda.Event()
            ev2.record(s_sel)
            qb0, qb1 = c * bpc, min(nb, (c + 1) * bpc)
            if qb0 < qb1:
                s_att.wait_event(ev2)
                block_sparse_attention(q, k, v, plan.col_idx, plan.col_cnt, causal=causal, out=out,
                                       q_blocks=(qb0, qb1), stream=s_att)
        done_sel, done_att = torch.cuda.Event(), torch.cuda.Event()
        done_sel.record(s_sel)
        done_att.record(s_att)
        main.wait_event(done_sel)
        main.wait_event(done_att)
    return out.transpose(1, 2)
