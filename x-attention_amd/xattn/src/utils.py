"""``find_blocks_chunked`` of ``xattn/src/utils.py`` (mit-han-lab/x-attention)
on the HIP block-selection kernel."""
import torch

from . import hip_backend as _hb

__all__ = ["find_blocks_chunked", "create_causal_mask"]


def create_causal_mask(batch_size, head_num, block_size, block_num, divide_block_num, device="cuda"):
    """Additive mask of one query block against ``block_num`` key blocks, the
    helper of xattn/src/utils.py:3-42 (the reference's threshold profiler builds
    its per-block softmax with it; the profiler here does that inside a kernel):
    ``[batch_size, head_num, block_size, block_size * block_num]``, zero where
    query row r of block ``divide_block_num`` may look (all earlier blocks, and
    columns <= r of its own block), ``-inf`` elsewhere.  A view expanded over
    batch and heads, like the reference's.  Host-side tensor code, no kernel."""
    own = divide_block_num + 1
    if own < 1 or own > block_num:
        raise ValueError(f"divide_block_num ({own}) must be between 1 and block_num ({block_num}).")
    cols = torch.arange(block_size * block_num, device=device)
    rows = torch.arange(block_size, device=device)
    visible = cols[None, :] <= rows[:, None] + divide_block_num * block_size
    mask = torch.zeros(block_size, block_size * block_num, device=device).masked_fill(~visible, float("-inf"))
    return mask[None, None].expand(batch_size, head_num, block_size, block_size * block_num)


def find_blocks_chunked(input_tensor, current_index, threshold, num_to_choose, decoding: bool, mode: str = "both",
                        causal=True):
    """Per q-block row, keep key blocks until their mass reaches ``threshold``.

    Contract of xattn/src/utils.py:44-191 for the prefill branch:
    ``input_tensor`` ``[1, H, rows, cols]`` block sums on the GPU, ``current_index``
    the column of row 0's diagonal, ``threshold`` a float or ``[H]`` tensor;
    returns a bool mask of the same shape.  One difference: when ``causal`` the
    kernel clears every column beyond each row's own diagonal (the reference
    clears only columns past the chunk's last diagonal here and the rest later,
    in xattn_estimate), and it takes block sums beyond the diagonal as zero.
    """
    assert threshold is None or num_to_choose is None
    if threshold is None:
        raise NotImplementedError("block num chunk prefill not impleted")
    if mode == "prefill" and decoding:
        return torch.ones_like(input_tensor, dtype=torch.bool)
    if mode == "decode" and not decoding:
        # xattn/src/utils.py:71-86: no selection in this mode.  Non-causal: everything is kept.  Causal: the
        # reference returns the first current_index + 1 ROWS of an all-true mask joined, along the column
        # axis, to the remaining rows of an all-false one - which only has a shape when both parts have
        # equally many rows (rows == 2 * (current_index + 1)); torch raises otherwise, as it does there.
        keep = torch.ones_like(input_tensor, dtype=torch.bool)
        if not causal:
            return keep
        return torch.cat([keep[:, :, : current_index + 1], ~keep[:, :, current_index + 1:]], dim=-1)
    if not input_tensor.is_cuda:
        raise _hb.XattnHipError("input_tensor must live on a ROCm device (no CPU fallback exists)")
    bsz, heads, rows, cols = input_tensor.shape
    assert bsz == 1
    lib = _hb.lib()
    dev = input_tensor.device
    sums = input_tensor[0].to(torch.float32).contiguous()
    if isinstance(threshold, torch.Tensor):
        tau = threshold.detach().to(torch.float64).reshape(-1)
        tau = (tau.expand(heads) if tau.numel() == 1 else tau).contiguous().to(dev)
    else:
        tau = torch.full((heads,), float(threshold), dtype=torch.float64, device=dev)
    mask = torch.empty((heads, rows, cols), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _hb.check(
            lib.xattn_select_blocks(
                sums.data_ptr(), tau.data_ptr(), mask.data_ptr(), None, None, 0,
                heads, rows, cols, 0, rows, int(current_index), int(bool(causal)), 0, 0,
                cols, rows * 128, int(current_index) * 128, rows, 0, 0, torch.cuda.current_stream(dev).cuda_stream,
            ),
            "xattn_select_blocks",
        )
    return mask.view(torch.bool).unsqueeze(0)
