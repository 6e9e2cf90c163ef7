"""``find_blocks_chunked`` of ``xattn/src/utils.py`` (mit-han-lab/x-attention)
on the HIP block-selection kernel."""
import torch

from . import hip_backend as _hb

__all__ = ["find_blocks_chunked"]


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
        raise NotImplementedError("decode-mode masks are outside the prefill path")
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
