"""GPU: the call shapes of the Qwen2-VL and HunyuanVideo integrations against
the oracle composed the same way."""
import pytest
import torch

from helpers import OUT_MAX_ABS, OUT_MEAN_ABS, lists_from_mask, mask_mismatch_report
from oracle import xattn_oracle as O

pytestmark = pytest.mark.gpu


def _close(out, want):
    err = (out.float().cpu() - want.float()).abs()
    assert err.max().item() <= OUT_MAX_ABS and err.mean().item() <= OUT_MEAN_ABS, (err.max(), err.mean())


def test_valid_padded_attention():
    from xattn.src.integrations import valid_padded_attention
    from xattn.src.Xattention import default_chunk_size, xattn_estimate
    from xattn.synthetic import WORKLOADS, make_inputs

    H, valid, total = 4, 1500, 1756                      # 256 padding tokens
    q, k, v = make_inputs(WORKLOADS[4], device="cpu", seed=2, L=total, heads=H, kv_heads=H)
    cu = torch.tensor([0, valid, total], dtype=torch.int32)
    out = valid_padded_attention(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), stride=8, threshold=0.9)
    assert out.shape == (1, H, total, 128)
    # valid part: oracle attention under the mask the estimator picks for these tensors (non-causal)
    qa, ka, va = q[:, :, :valid], k[:, :, :valid], v[:, :, :valid]
    _, mask = xattn_estimate(qa.cuda(), ka.cuda(), 128, 8, threshold=0.9, chunk_size=default_chunk_size(valid),
                             causal=False)
    nb = (valid + 127) // 128
    want_sums, want_mask = O.xattn_estimate(qa.float(), ka.float(), 128, 8, threshold=0.9,
                                            chunk_size=default_chunk_size(valid), causal=False)
    nbad, outside = mask_mismatch_report(want_sums[0], mask[0], want_mask[0], 0.9, False, 0,
                                         default_chunk_size(valid) // 128)
    assert outside == 0, (nbad, outside)
    mask = mask[:, :, :nb, :nb].cpu()
    _close(out[:, :, :valid], O.block_sparse_attention(qa.float(), ka.float(), va.float(), mask, causal=False))
    # padding part: dense among itself
    qb, kb, vb = q[:, :, valid:], k[:, :, valid:], v[:, :, valid:]
    _close(out[:, :, valid:], O.block_sparse_attention(qb.float(), kb.float(), vb.float(),
                                                      torch.ones(1, H, 2, 2, dtype=torch.bool), causal=False))
    # threshold 1: dense on the valid part too
    dense = valid_padded_attention(q.cuda(), k.cuda(), v.cuda(), cu, cu, stride=8, threshold=1.0)
    _close(dense[:, :, :valid], O.block_sparse_attention(qa.float(), ka.float(), va.float(),
                                                         torch.ones(1, H, nb, nb, dtype=torch.bool), causal=False))


def test_prefill_or_decode():
    from xattn.src.integrations import prefill_or_decode
    from xattn.src.Xattention import Xattention_prefill
    from xattn.synthetic import WORKLOADS, make_inputs

    q, k, v = make_inputs(WORKLOADS[3], device="cuda", seed=1, L=2048, heads=28, kv_heads=4)
    sparse = prefill_or_decode(q, k, v, stride=16, threshold=0.9)
    assert torch.equal(sparse, Xattention_prefill(q, k, v, 16, threshold=0.9))
    dense = prefill_or_decode(q, k, v, sparse=False)
    _close(dense, O.block_sparse_attention(q.cpu().float(), k.cpu().float(), v.cpu().float(),
                                           torch.ones(1, 28, 16, 16, dtype=torch.bool), causal=True))
    step = prefill_or_decode(q[:, :, -1:], k, v)
    assert step.shape == (1, 28, 1, 128)
    assert (step[0, :, 0].float() - dense[0, :, -1].float()).abs().max().item() <= 1e-2
