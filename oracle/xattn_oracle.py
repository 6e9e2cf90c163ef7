"""CPU oracle for the XAttention prefill path.  TEST INFRASTRUCTURE ONLY.

This module is a checker, not a product path: only ``tests/``, the smoke test
and the ``cpu_baseline`` leg of the benchmark may import it.  The shipped
operator never calls into it and raises when its HIP library is missing.

It restates, in plain device-agnostic torch, the algorithm of the reference
(``mit-han-lab/x-attention``); every function names the reference lines it
follows (paths relative to the reference checkout):

* :func:`antidiagonal_scores`      - xattn/src/Xattention.py:84-94 + 182-185
                                     (== xattn/src/kernels.py:219-230)
* :func:`estimate_chunk_block_sums`- xattn/src/Xattention.py:174-252 (torch branch)
* :func:`find_blocks_chunked`      - xattn/src/utils.py:44-191 (prefill branch)
* :func:`xattn_estimate`           - xattn/src/Xattention.py:13-299
* :func:`default_chunk_size`       - xattn/src/Xattention.py:322-331
* :func:`block_sparse_attention`   - the un-vendored ``block_sparse_attn==0.0.1``
                                     call at xattn/src/Xattention.py:377-391,
                                     restated as dense softmax attention under
                                     the expanded block mask (and token-causal).
* :func:`Xattention_prefill`       - xattn/src/Xattention.py:302-402
* :func:`chunk_prefill_to_attn_sum`,
  :func:`profile_threshold_head`   - xattn/threshold/profile_threshold/
                                     profile_threshold.py:15-57 and :84-93
* :func:`single_decode_with_kv_cache` - the un-vendored ``flashinfer==0.1.6``
                                     call at xattn/src/load_llama.py:191-196,
                                     restated as one softmax attention row per
                                     query head over the whole cache.

Pinning status (what independent evidence each function is checked against,
see tests/test_oracle_*.py):

* antidiagonal_scores: brute force over the full Q.K^T on tiny inputs
  (sum of S x S antidiagonals), and pointer-form vs concatenation-form.
* estimate_chunk_block_sums: torch.softmax in fp64 on the brute-force scores,
  row-mass invariant (a real q-block row sums to block_size/stride), zeros
  above the block diagonal, zero padded rows, chunk-size independence when
  ``pad0_quirk=False``.
* find_blocks_chunked: golden input/output vectors produced by the
  reference's own ``xattn/src/utils.py`` (tests/golden/find_blocks_*.pt,
  made by tests/golden/make_find_blocks_golden.py), plus a brute-force
  sorted-prefix enumeration.
* block_sparse_attention: PARITY UNPINNED against block_sparse_attn itself
  (third-party CUDA, absent from the reference tree, no reference test holds
  results for it).  It is pinned to the mathematics only: all-True mask ==
  torch scaled_dot_product_attention, and a per-row python loop on tiny
  inputs.
* single_decode_with_kv_cache: PARITY UNPINNED against flashinfer itself
  (third-party CUDA, absent from the reference tree and from this image).
  Pinned to the mathematics: equals torch scaled_dot_product_attention with
  repeated KV heads, and the last row of causal prefill attention.
* chunk_prefill_to_attn_sum: a full softmax matrix on tiny inputs summed per
  block by a python loop; every real q-block row sums to its number of rows.
  profile_threshold_head: a hand-worked example and a python re-derivation
  from the definition (fewest blocks reaching the coverage, minimum estimate
  among them, share of the estimate at or above it).  The reference module
  itself needs flash_attn and a GPU at import and cannot be run here.
* xattn_estimate / Xattention_prefill glue: invariants (block-tril, forced
  sink/diagonal, keep_sink row, keep_recent diagonal) and tiny hand cases.
"""

import math

import torch
import torch.nn.functional as F

NEG_INF = float("-inf")


# --------------------------------------------------------------------------- #
# A3: antidiagonal (stride-S reversed reshape) scores
# --------------------------------------------------------------------------- #
def reshape_inverse(query_states, key_states, stride, kdb=1):
    """Concatenation form of the stride-S reshape, select_mode="inverse".

    Follows xattn/src/Xattention.py:84-94: keys take token ``n*S+i`` into
    feature slab ``i``; queries take token ``m*S*kdb+(S-1-i)`` into slab ``i``
    (``kdb > 1`` keeps every kdb-th reshaped query row, the FIRST of each group).
    """
    rk = torch.cat([key_states[:, :, i::stride, :] for i in range(stride)], dim=-1)
    rq = torch.cat(
        [query_states[:, :, (stride - 1 - i) :: (stride * kdb), :] for i in range(stride)],
        dim=-1,
    )
    return rq, rk


def reshape_operands(query_states, key_states, stride, select_mode="inverse", perm=None, kdb=1):
    """The reshaped (query, key) pair of every ``select_mode`` of the torch
    branch, xattn/src/Xattention.py:72-135.  ``perm`` stands for the
    ``torch.randperm(stride)`` the reference draws for "random"; ``kdb`` enters
    the "inverse" reshape only (:88-93)."""
    S, d = stride, query_states.shape[-1]
    rk = torch.cat([key_states[:, :, i::S, :] for i in range(S)], dim=-1)
    if select_mode in ("inverse", ""):
        return reshape_inverse(query_states, key_states, stride, kdb)
    if kdb != 1:
        raise ValueError("kdb != 1 only makes sense with select_mode='inverse'")
    if select_mode == "random":
        rq = torch.cat([query_states[:, :, int(perm[i]) :: S, :] for i in range(S)], dim=-1)
        return rq, rk
    if select_mode == "slash":
        rq = torch.cat([query_states[:, :, i::S, :] for i in range(S)], dim=-1)
        return rq, rk
    rq = torch.cat([query_states[:, :, (S - 1 - i) :: S, :] for i in range(S)], dim=-1)
    if select_mode in ("double", "triple"):
        rk = rk + torch.cat([rk[..., d:], rk[..., :d]], dim=-1)
        if select_mode == "triple":
            rk = rk + torch.cat([rk[..., -d:], rk[..., :-d]], dim=-1)
        return rq, rk
    raise ValueError(select_mode)


def create_causal_mask(batch_size, head_num, block_size, block_num, divide_block_num, device="cpu"):
    """Additive mask of query block ``divide_block_num`` against all key blocks,
    xattn/src/utils.py:3-42 (the reference hard-codes ``device="cuda"``)."""
    divide_block_num += 1
    if divide_block_num < 1 or divide_block_num > block_num:
        raise ValueError(f"divide_block_num ({divide_block_num}) must be between 1 and block_num ({block_num}).")
    total = block_size * block_num
    mask = torch.zeros(block_size, total, device=device)
    if divide_block_num < block_num:
        mask[:, divide_block_num * block_size :] = NEG_INF
    start = (divide_block_num - 1) * block_size
    mask[:, start : start + block_size] = torch.triu(
        torch.full((block_size, block_size), NEG_INF, device=device), diagonal=1
    )
    return mask[None, None].expand(batch_size, head_num, block_size, total)


def antidiagonal_scores(query_states, key_states, stride):
    """score[m, n] = sum_i Q[m*S + S-1-i] . K[n*S + i]  (un-scaled).

    xattn/src/Xattention.py:182-185 applied to :func:`reshape_inverse`;
    identical to the pointer arithmetic of xattn/src/kernels.py:219-230.
    """
    rq, rk = reshape_inverse(query_states, key_states, stride)
    return torch.matmul(rq, rk.transpose(2, 3))


# --------------------------------------------------------------------------- #
# A5: threshold block selection
# --------------------------------------------------------------------------- #
def find_blocks_chunked(
    input_tensor,
    current_index,
    threshold,
    num_to_choose,
    decoding,
    mode="both",
    causal=True,
):
    """Per q-block row, keep blocks until their mass reaches ``threshold``.

    Restates the prefill branch of xattn/src/utils.py:87-191 including its
    incidental behaviours: fp64 arithmetic (:87), per-head tensor thresholds
    (:91-95), forced sink and diagonal columns (:99-106), the
    ``[0, forced_sum, others...]`` prefix that is one slot longer than the
    forced set when sink and diagonal coincide (:115-124), rewriting of the
    unselected ranks to column 0 before the scatter (:142, :164) and the
    clearing of columns past the chunk's last diagonal (:176-180).
    """
    assert threshold is None or num_to_choose is None
    if threshold is None:
        raise NotImplementedError("selection by block count is not implemented upstream")
    bsz, heads, rows, cols = input_tensor.shape
    if mode == "prefill" and decoding:
        return torch.ones_like(input_tensor, dtype=torch.bool)
    if mode == "decode" and not decoding:
        # xattn/src/utils.py:71-86, literally: the causal branch joins ROW slices along the column axis
        ones = torch.ones_like(input_tensor, dtype=torch.bool)
        if not causal:
            return ones
        return torch.cat(
            [ones[:, :, 0 : current_index + 1], torch.zeros_like(ones)[:, :, current_index + 1 :]], dim=-1
        )
    dev = input_tensor.device
    x = input_tensor.to(torch.float64)

    total = x.sum(dim=-1, keepdim=True)
    if isinstance(threshold, torch.Tensor):
        tau = threshold.to(torch.float64).to(dev)
        required = total * tau.reshape(1, -1, 1, 1).expand(bsz, heads, rows, 1)
    else:
        required = total * threshold

    def scatter_rows(mask, index):
        flat_mask = mask.view(bsz, heads * rows, cols)
        flat_index = index.view(bsz, heads * rows, cols)
        row_id = torch.arange(heads * rows, device=dev).unsqueeze(-1)
        flat_mask[:, row_id, flat_index] = True
        return flat_mask.view(bsz, heads, rows, cols)

    zero_col = torch.zeros((bsz, heads, rows, 1), dtype=torch.float64, device=dev)
    if causal:
        forced = torch.zeros_like(x, dtype=torch.bool)
        forced[..., 0] = True
        eye = torch.eye(rows, dtype=torch.bool, device=dev)
        forced[..., current_index : current_index + rows] = eye
        others_sorted, _ = torch.sort(x.masked_fill(forced, 0), dim=-1, descending=True)
        forced_sum = torch.where(forced, x, 0.0).sum(dim=-1, keepdim=True)
        ranked_values = torch.cat([zero_col, forced_sum, others_sorted[..., :-2]], dim=-1)
        _, order = torch.sort(
            torch.where(forced, 100000 * (1 + x), x), dim=-1, descending=True
        )
        mass_before = torch.cat([zero_col, ranked_values[..., :-1]], dim=-1).cumsum(dim=-1)
        keep = mass_before < required
        mask = scatter_rows(forced.clone(), torch.where(keep, order, 0))
        # columns after the last diagonal of this chunk never survive (:176-180)
        mask[..., current_index + rows :] = False
    else:
        values_sorted, order = torch.sort(x, dim=-1, descending=True)
        mass_before = torch.cat([zero_col, values_sorted[..., :-1]], dim=-1).cumsum(dim=-1)
        keep = mass_before < required
        mask = scatter_rows(
            torch.zeros_like(x, dtype=torch.bool), torch.where(keep, order, 0)
        )
    return mask


# --------------------------------------------------------------------------- #
# A2 / A4: per-chunk softmax + block sums (torch branch), and the estimate
# --------------------------------------------------------------------------- #
def estimate_chunk_block_sums(
    reshaped_query,
    reshaped_key,
    chunk_idx,
    *,
    head_dim,
    stride,
    norm,
    block_size,
    chunk_size,
    k_chunk_num,
    q_chunk_num,
    k_reshaped_num_to_pad,
    q_reshaped_num_to_pad,
    causal,
    pad0_quirk,
    out_dtype,
    softmax=True,
    kdb=1,
    triton_rows=False,
):
    """Block sums of softmax(antidiagonal scores) for one query chunk.

    Follows xattn/src/Xattention.py:174-252.  ``pad0_quirk=True`` keeps the
    literal behaviour of line 201: with no key padding the slice
    ``[..., -0:]`` covers every column, so each query chunk sees only the
    keys of its own chunk.  ``pad0_quirk=False`` skips that line when there is
    no padding, which is what the reference's Triton branch computes
    (xattn/src/kernels.py:42-66 sweeps from key column 0).

    ``kdb > 1`` (:174-181, :217-222, :245): the chunk holds ``rcs // kdb`` query
    rows; the causal mask is built for ``rcs`` rows and every kdb-th row of it,
    starting at ``kdb - 1``, is used - query row j (tokens of reshaped row
    ``j*kdb``) sees keys up to reshaped position ``j*kdb + kdb - 1``; the rows
    of the padded tail are the last ``q_reshaped_num_to_pad // kdb`` (a slice
    ``-0:`` when that is 0, i.e. then the whole chunk); a query block sums
    ``rbs // kdb`` rows.

    ``triton_rows=True`` replaces the torch branch's padded-row rule by the
    Triton branch's (xattn/src/kernels.py:70 with the ``real_q_len`` argument of
    xattn/src/Xattention.py:169): a row is zeroed when its position on the key
    axis is at or beyond the real (unpadded) reshaped key length, whatever the
    query padding; padded query rows that rule leaves alone carry the uniform
    softmax of an all-zero query.
    """
    bsz, heads = reshaped_query.shape[:2]
    rcs = chunk_size // stride
    rbs = block_size // stride
    offset_chunks = k_chunk_num - q_chunk_num
    cq = reshaped_query[:, :, (chunk_idx * rcs) // kdb : (chunk_idx * rcs + rcs) // kdb, :]
    w = torch.matmul(cq, reshaped_key.transpose(2, 3))
    w = w / math.sqrt(head_dim) / stride / norm
    last_padded = chunk_idx == q_chunk_num - 1 and q_reshaped_num_to_pad != 0
    if triton_rows:
        assert kdb == 1
        # key-axis position of this chunk's rows against the real reshaped key length
        pos = (chunk_idx + offset_chunks) * rcs + torch.arange(rcs, device=w.device)
        zero_rows = pos >= rcs * k_chunk_num - k_reshaped_num_to_pad
        last_padded = False
    if causal:
        cm = torch.zeros((bsz, heads, rcs, rcs * k_chunk_num), device=w.device)
        if k_reshaped_num_to_pad > 0 or pad0_quirk:
            cm[..., (-k_reshaped_num_to_pad):] = NEG_INF
        c0 = (chunk_idx + offset_chunks) * rcs
        c1 = c0 + rcs
        cm[..., c0:c1] = torch.triu(
            torch.full((rcs, rcs), NEG_INF, device=w.device), diagonal=1
        )
        if last_padded:
            cm[:, :, (-(q_reshaped_num_to_pad // kdb)):, :] = NEG_INF
        cm[..., c1:] = NEG_INF
        cm = cm[:, :, kdb - 1 :: kdb, :]
        w = w + cm
    if softmax:
        w = F.softmax(w, dim=-1, dtype=torch.float32).to(out_dtype)
    else:
        w = torch.exp(w).to(out_dtype)   # Xattention.py:231-234
    if last_padded:
        w[:, :, (-(q_reshaped_num_to_pad // kdb)):, :] = 0
    if triton_rows:
        w = torch.nan_to_num(w, nan=0.0)
        w[:, :, zero_rows, :] = 0
    sums = w.view(bsz, heads, rcs // rbs, rbs // kdb, -1, rbs).sum(dim=-1).sum(dim=-2)
    return sums


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
    use_triton=False,
    causal=True,
    kdb=1,
    keep_sink=False,
    keep_recent=False,
    pad0_quirk=True,
    perm=None,
):
    """(attn_sums, simple_masks), both ``[B, H, Nq_blocks_padded, Nk_blocks_padded]``.

    Restates xattn/src/Xattention.py:13-299 on whatever device the inputs live
    on (``perm``: the permutation "random" would draw).  ``use_triton`` is
    accepted for signature parity and ignored; which upstream branch is restated
    is chosen by ``pad0_quirk``: ``True`` = the torch branch literally,
    ``False`` = the Triton branch (keys of earlier chunks visible, and rows
    zeroed by their key-axis position against the real key length; the two
    row rules differ only when query and key padding differ).  ``kdb != 1``
    exists in the torch branch only (the reference raises with ``use_triton``).
    """
    triton_rows = not pad0_quirk
    if kdb != 1 and triton_rows:
        raise ValueError("use_triton and kdb cannot be used together")
    bsz, kv_heads, k_len, head_dim = key_states.shape
    _, heads, q_len, _ = query_states.shape
    assert heads == kv_heads

    k_pad = -k_len % chunk_size
    q_pad = -q_len % chunk_size
    k_chunk_num = (k_len + k_pad) // chunk_size
    q_chunk_num = (q_len + q_pad) // chunk_size
    k_block_num = (k_len + k_pad) // block_size
    q_block_num = (q_len + q_pad) // block_size
    assert k_chunk_num >= q_chunk_num
    pk = F.pad(key_states, (0, 0, 0, k_pad), value=0) if k_pad else key_states
    pq = F.pad(query_states, (0, 0, 0, q_pad), value=0) if q_pad else query_states
    rq, rk = reshape_operands(pq, pk, stride, select_mode, perm, kdb)
    blocks_per_chunk = chunk_size // block_size

    sums, masks = [], []
    for c in range(q_chunk_num):
        s = estimate_chunk_block_sums(
            rq,
            rk,
            c,
            head_dim=head_dim,
            stride=stride,
            norm=norm,
            block_size=block_size,
            chunk_size=chunk_size,
            k_chunk_num=k_chunk_num,
            q_chunk_num=q_chunk_num,
            k_reshaped_num_to_pad=k_pad // stride,
            q_reshaped_num_to_pad=q_pad // stride,
            causal=causal,
            pad0_quirk=pad0_quirk,
            out_dtype=pq.dtype,
            softmax=softmax,
            kdb=kdb,
            triton_rows=triton_rows,
        )
        m = find_blocks_chunked(
            s,
            k_block_num - q_block_num + c * blocks_per_chunk,
            threshold,
            None,
            decoding=False,
            mode="prefill",
            causal=causal,
        )
        sums.append(s)
        masks.append(m)
    attn_sums = torch.cat(sums, dim=-2)
    simple_masks = torch.cat(masks, dim=-2)

    if causal:
        tril = torch.tril(
            torch.ones(q_block_num, q_block_num, dtype=torch.bool, device=simple_masks.device)
        )
        tail = simple_masks[:, :, -q_block_num:, -q_block_num:]
        simple_masks[:, :, -q_block_num:, -q_block_num:] = tail & tril
    if keep_sink:
        simple_masks[:, :, 0, :] = True
    if keep_recent:
        eye = torch.eye(q_block_num, dtype=torch.bool, device=simple_masks.device)
        tail = simple_masks[:, :, -q_block_num:, -q_block_num:]
        simple_masks[:, :, -q_block_num:, -q_block_num:] = tail | eye
    return attn_sums, simple_masks


def default_chunk_size(k_len):
    """Operator's default chunk rule, xattn/src/Xattention.py:322-331."""
    p = 1 << (k_len - 1).bit_length()
    return int(max(min(max(2048, p), 128 * 1024 * 2048 // p), 2048))


# --------------------------------------------------------------------------- #
# A6: block-sparse attention as dense masked softmax attention
# --------------------------------------------------------------------------- #
def block_sparse_attention(
    query_states,
    key_states,
    value_states,
    block_mask,
    causal=True,
    block_size=128,
    softmax_scale=None,
    row_tile=1024,
):
    """softmax(Q K^T * scale + M) V in fp32, M = block mask expanded x block_size
    and (when ``causal``) the bottom-right-aligned token-causal mask.

    ``block_mask`` is ``[B, H, ceil(Lq/bs), ceil(Lk/bs)]`` bool.  K/V may carry
    fewer heads than Q (grouped-query attention); query head h reads KV head
    ``h // (H / H_kv)``.  A query row with no visible key yields zeros.
    Output is ``[B, H, Lq, d]`` in the input dtype.
    """
    bsz, heads, q_len, d = query_states.shape
    kv_heads, k_len = key_states.shape[1], key_states.shape[2]
    group = heads // kv_heads
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
    kf = key_states.float().repeat_interleave(group, dim=1)
    vf = value_states.float().repeat_interleave(group, dim=1)
    out = torch.empty((bsz, heads, q_len, d), dtype=torch.float32, device=query_states.device)
    kpos = torch.arange(k_len, device=query_states.device)
    for r0 in range(0, q_len, row_tile):
        r1 = min(q_len, r0 + row_tile)
        qpos = torch.arange(r0, r1, device=query_states.device)
        s = torch.matmul(query_states[:, :, r0:r1].float(), kf.transpose(2, 3)) * scale
        allow = block_mask[:, :, qpos // block_size][:, :, :, kpos // block_size]
        if causal:
            allow = allow & (kpos[None, :] <= qpos[:, None] + (k_len - q_len))
        s = s.masked_fill(~allow, NEG_INF)
        p = torch.softmax(s, dim=-1)
        p = torch.nan_to_num(p, nan=0.0)
        out[:, :, r0:r1] = torch.matmul(p, vf)
    return out.to(query_states.dtype)


def Xattention_prefill(
    query_states,
    key_states,
    value_states,
    stride,
    norm=1,
    threshold=0.8,
    block_size=128,
    use_triton=False,
    causal=True,
    kdb=1,
    chunk_size=None,
    keep_sink=False,
    keep_recent=False,
    pad0_quirk=True,
    return_mask=False,
):
    """Estimate -> block mask -> masked attention, xattn/src/Xattention.py:302-402."""
    bsz, heads, k_len, d = key_states.shape
    q_len = query_states.shape[2]
    assert block_size == 128 and bsz == 1
    q_block_num = (q_len + block_size - 1) // block_size
    k_block_num = (k_len + block_size - 1) // block_size
    if chunk_size is None:
        chunk_size = default_chunk_size(k_len)
    _, mask = xattn_estimate(
        query_states,
        key_states,
        block_size=block_size,
        stride=stride,
        norm=norm,
        threshold=threshold,
        select_mode="inverse",
        use_triton=use_triton,
        causal=causal,
        chunk_size=chunk_size,
        kdb=kdb,
        keep_sink=keep_sink,
        keep_recent=keep_recent,
        pad0_quirk=pad0_quirk,
    )
    mask = mask[:, :, :q_block_num, :k_block_num].contiguous()
    out = block_sparse_attention(
        query_states, key_states, value_states, mask, causal=causal, block_size=block_size
    )
    return (out, mask) if return_mask else out


# --------------------------------------------------------------------------- #
# decode step
# --------------------------------------------------------------------------- #
def single_decode_with_kv_cache(q, k, v, kv_layout="NHD", sm_scale=None):
    """One query token per head against the whole KV cache, fp32 throughout.

    The reference calls flashinfer.single_decode_with_kv_cache(q, k, v,
    kv_layout="HND") (xattn/src/load_llama.py:191-196) with q ``[H, d]`` and
    k, v ``[H_kv, L, d]``; query head h reads KV head ``h // (H / H_kv)``, the
    scale defaults to ``1/sqrt(d)``, no positional transform is applied.
    Returns ``[H, d]`` in q's dtype.
    """
    if kv_layout == "NHD":
        k, v = k.transpose(0, 1), v.transpose(0, 1)
    heads, dim = q.shape
    group = heads // k.shape[0]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(dim)
    out = torch.empty((heads, dim), dtype=torch.float32)
    for h in range(heads):
        kh = k[h // group].float()
        logits = (kh @ q[h].float()) * sm_scale
        out[h] = torch.softmax(logits, dim=0) @ v[h // group].float()
    return out.to(q.dtype)


# --------------------------------------------------------------------------- #
# threshold profiler
# --------------------------------------------------------------------------- #
def chunk_prefill_to_attn_sum(query_states, key_states, block_size=128):
    """True causal attention mass per block, ``[B, H, Nq, Nk]`` fp32.

    Follows xattn/threshold/profile_threshold/profile_threshold.py:15-57 with
    fp32 arithmetic: q-block by q-block, ``softmax(q k^T / sqrt(d))`` over the
    keys at or before each query (keys and query rows past the end excluded),
    summed over the block's rows and over each key block.  GQA by head sharing.
    """
    bsz, heads, q_len, d = query_states.shape
    kv_heads, k_len = key_states.shape[1], key_states.shape[2]
    assert q_len == k_len
    group = heads // kv_heads
    nb = (q_len + block_size - 1) // block_size
    k = key_states.float().repeat_interleave(group, 1)
    out = torch.zeros((bsz, heads, nb, nb), dtype=torch.float32)
    pos_k = torch.arange(nb * block_size)
    for i in range(nb):
        rows = torch.arange(i * block_size, min((i + 1) * block_size, q_len))
        w = torch.matmul(query_states[:, :, rows].float(), k.transpose(2, 3)) / math.sqrt(d)
        w = F.pad(w, (0, nb * block_size - k_len), value=NEG_INF)
        dead = (pos_k[None, :] > rows[:, None]) | (pos_k[None, :] >= k_len)
        w = w.masked_fill(dead, NEG_INF)
        p = F.softmax(w, dim=-1, dtype=torch.float32)
        out[:, :, i] = p.view(bsz, heads, len(rows), nb, block_size).sum(-1).sum(-2)
    return out


def profile_threshold_head(attn_sum, xattn_sum, coverage=0.9):
    """``[B, H]`` thresholds, profile_threshold.py:84-93 (``xattn_sum`` already
    cropped to ``attn_sum``'s shape and multiplied by the stride)."""
    vals, idx = torch.sort(attn_sum, dim=-1, descending=True, stable=True)
    cumsum = vals.cumsum(-1)
    need_len = (cumsum < coverage * cumsum[..., -1:]).sum(-1) + 1
    rank = torch.arange(vals.size(-1))
    selected = rank.view(1, 1, 1, -1) < need_len.unsqueeze(-1)
    x_sorted = xattn_sum.gather(-1, idx)
    miniblock = x_sorted.masked_fill(~selected, float("inf")).min(-1).values
    at_or_above = xattn_sum >= miniblock.unsqueeze(-1)
    return (xattn_sum * at_or_above).sum(-1).sum(-1) / (xattn_sum.sum(-1).sum(-1) + 1e-8)
