"""GPU: the keyword forms in which the reference's own scripts call the
operator (demo/example.py:12, eval/LongBench/pred.py:131-141,
eval/efficiency/attention_speedup.py:87) run unchanged against this package."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_reference_call_forms():
    from xattn.src.Xattention import Xattention_prefill

    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn((1, 32, 1024, 128), device="cuda", generator=g).bfloat16() for _ in range(3))
    # demo/example.py
    out = Xattention_prefill(query_states=q, key_states=k, value_states=v, stride=16, block_size=128,
                             use_triton=True, chunk_size=2048)
    assert out.shape == (1, 32, 1024, 128) and out.dtype == torch.bfloat16 and torch.isfinite(out.float()).all()
    # eval/efficiency/attention_speedup.py
    a = Xattention_prefill(q, k, v, stride=16, threshold=0.9, use_triton=True)
    b = Xattention_prefill(q, k, v, stride=8, threshold=torch.full((32,), 0.9), use_triton=True)
    assert a.shape == b.shape == out.shape
    # eval/LongBench/pred.py: positional stride, per-head thresholds on the device, keep flags
    c = Xattention_prefill(q, k, v, 8, norm=1, threshold=torch.rand(32, device="cuda") * 0.5 + 0.4,
                           use_triton=True, keep_sink=True, keep_recent=True)
    assert torch.isfinite(c.float()).all()
    # transposed [B, L, H, d] views, as the model forwards pass them
    qt = q.transpose(1, 2).contiguous().transpose(1, 2)
    assert torch.equal(Xattention_prefill(qt, k, v, stride=16, threshold=0.9, use_triton=True), a)
