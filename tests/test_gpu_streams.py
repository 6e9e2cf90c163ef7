"""GPU: entry points are stream-ordered and keep no shared state - two operator
calls issued on two HIP streams (default priority) overlap freely and give the
results of the same calls made one after the other."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_two_streams_give_serial_results():
    from xattn.src.Xattention import Xattention_prefill
    from xattn.src.decode import single_decode_with_kv_cache
    from xattn.synthetic import WORKLOADS, make_inputs

    a = make_inputs(WORKLOADS[1], device="cuda", seed=1, L=8192, heads=8, kv_heads=2)
    b = make_inputs(WORKLOADS[1], device="cuda", seed=2, L=6000, heads=8, kv_heads=2)
    want_a = Xattention_prefill(*a, 8, threshold=0.9)
    want_b = Xattention_prefill(*b, 16, threshold=0.8)
    want_da = single_decode_with_kv_cache(a[0][0, :, -1], a[1][0], a[2][0], "HND")
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for _ in range(3):
        with torch.cuda.stream(s1):
            got_a = Xattention_prefill(*a, 8, threshold=0.9)
            got_da = single_decode_with_kv_cache(a[0][0, :, -1], a[1][0], a[2][0], "HND")
        with torch.cuda.stream(s2):
            got_b = Xattention_prefill(*b, 16, threshold=0.8)
        s1.synchronize()
        s2.synchronize()
        assert torch.equal(got_a, want_a) and torch.equal(got_b, want_b) and torch.equal(got_da, want_da)
