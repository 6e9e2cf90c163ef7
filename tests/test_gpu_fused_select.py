"""GPU: the fused normalise-and-select pass (xattn_estimate_select, block sums kept in LDS) gives exactly the
lists and masks of the two-kernel path (xattn_estimate_block_sums, then xattn_select_blocks), whose results the
other test files check against the oracle.  Bit equality, not a tolerance: both passes share their arithmetic."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(q, k, stride, tau, chunk, **kw):
    from xattn.src.Xattention import estimate_and_select

    a = estimate_and_select(q, k, stride, tau, chunk, want_sums=True, **kw)
    b = estimate_and_select(q, k, stride, tau, chunk, want_sums=False, **kw)
    torch.cuda.synchronize()
    assert b["sums"] is None
    return a, b


def _assert_same(a, b, ctx):
    assert torch.equal(a["mask"], b["mask"]), ctx
    assert torch.equal(a["col_cnt"], b["col_cnt"]), ctx
    # entries beyond a row's count are unspecified
    n = a["col_idx"].shape[-1]
    live = torch.arange(n, device=a["col_idx"].device)[None, None, :] < a["col_cnt"][..., None]
    assert torch.equal(a["col_idx"][live], b["col_idx"][live]), ctx


CASES = [
    # heads, kv, q_len, k_len, stride, chunk, causal, use_triton
    (4, 2, 1024, 1024, 8, 512, True, True),
    (4, 4, 1000, 1000, 16, 256, True, True),
    (3, 1, 777, 1500, 4, 256, True, True),
    (8, 2, 2048, 2048, 16, 2048, True, False),
    (2, 2, 900, 900, 8, 128, False, True),
    (5, 5, 640, 1920, 16, 128, True, False),
    (2, 1, 4096, 4096, 4, 1024, True, True),
    (6, 2, 300, 300, 8, 2048, False, False),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("keep", [(False, False), (True, True)])
def test_fused_pass_equals_the_two_kernel_path(case, keep):
    H, Hkv, Lq, Lk, S, C, causal, use_triton = case
    g = torch.Generator(device="cpu").manual_seed(1000 + H * 7 + Lq)
    q = (torch.randn(1, H, Lq, 128, generator=g) * 1.5).bfloat16().cuda()
    k = (torch.randn(1, Hkv, Lk, 128, generator=g) * 1.5).bfloat16().cuda()
    tau = torch.linspace(0.5, 0.95, H, dtype=torch.float64)
    a, b = _both(q, k, S, tau, C, causal=causal, use_triton=use_triton, keep_sink=keep[0], keep_recent=keep[1])
    _assert_same(a, b, case)


@pytest.mark.parametrize("mode", ["slash", "double"])
def test_fused_pass_with_other_reshapes_and_without_softmax(mode):
    from xattn.src.Xattention import slab_pairs_for

    g = torch.Generator(device="cpu").manual_seed(5)
    q = torch.randn(1, 4, 1536, 128, generator=g).bfloat16().cuda()
    k = torch.randn(1, 2, 1536, 128, generator=g).bfloat16().cuda()
    for softmax in (True, False):
        a, b = _both(q, k, 8, 0.8, 512, causal=True, use_triton=False, slab_pairs=slab_pairs_for(mode, 8), softmax=softmax)
        _assert_same(a, b, (mode, softmax))


@pytest.mark.parametrize("workload", [1, 2])
def test_fused_pass_at_the_benchmark_sizes(workload):
    from xattn.synthetic import WORKLOADS, make_inputs

    w = WORKLOADS[workload]
    q, k, _ = make_inputs(w, device="cuda", seed=0, L=w.L, dtype=torch.bfloat16)
    a, b = _both(q, k, w.stride, w.threshold, w.chunk_size, causal=True, want_mask=False)
    assert torch.equal(a["col_cnt"], b["col_cnt"])
    n = a["col_idx"].shape[-1]
    for h in range(w.heads):     # head by head: the comparison mask of all heads at once would take 4 GiB
        live = torch.arange(n, device="cuda")[None, :] < a["col_cnt"][h][:, None]
        assert torch.equal(a["col_idx"][h][live], b["col_idx"][h][live]), h


def test_operator_runs_the_fused_pass_and_matches_lists_from_block_sums():
    """Xattention_prefill (fused pass inside) against block-sparse attention over the two-kernel path's lists."""
    from xattn.src.Xattention import Xattention_prefill, block_sparse_attention, estimate_and_select

    g = torch.Generator(device="cpu").manual_seed(9)
    q = torch.randn(1, 8, 3000, 128, generator=g).bfloat16().cuda()
    k = torch.randn(1, 2, 3000, 128, generator=g).bfloat16().cuda()
    v = torch.randn(1, 2, 3000, 128, generator=g).bfloat16().cuda()
    out = Xattention_prefill(q, k, v, 8, threshold=0.9, chunk_size=1024)
    r = estimate_and_select(q, k, 8, 0.9, 1024, causal=True, want_mask=False)
    ref = block_sparse_attention(q, k, v, r["col_idx"], r["col_cnt"], causal=True)
    torch.cuda.synchronize()
    assert torch.equal(out, ref)
