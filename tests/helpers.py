"""Shared helpers of the GPU parity tests (HIP path vs the CPU oracle)."""
import torch

OUT_MAX_ABS = 2e-2   # bf16 attention output, max-abs tolerance of the parity contract
OUT_MEAN_ABS = 5e-3  # ... and mean-abs


def lists_from_mask(mask):
    """bool [H, Nq, Nk] -> (col_idx int32 [H, Nq, Nk], col_cnt int32 [H, Nq]), ascending columns."""
    H, nq, nk = mask.shape
    order = torch.argsort((~mask).to(torch.int8), dim=-1, stable=True).to(torch.int32)
    cnt = mask.sum(-1).to(torch.int32)
    return order.contiguous(), cnt.contiguous()

from oracle.parity import TAU_BAND, head_mask_parity, mask_mismatch_report  # noqa: E402,F401
