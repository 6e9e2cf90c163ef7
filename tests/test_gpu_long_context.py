"""GPU: the operator works through long sequences in groups of query chunks on
buffers of one group - same result whatever the grouping, and a bounded
amount of memory beside inputs and output at a million tokens."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("causal", [True, False])
def test_grouping_does_not_change_the_result(monkeypatch, causal):
    import xattn.src.Xattention as X
    from xattn.synthetic import WORKLOADS, make_inputs

    w = WORKLOADS[1]
    q, k, v = make_inputs(w, device="cuda", seed=2, L=16384 + 300, heads=8, kv_heads=2)
    kw = dict(threshold=0.9, chunk_size=2048, causal=causal)
    whole = X.Xattention_prefill(q, k, v, 8, **kw)
    r = X.estimate_and_select(q, k, 8, 0.9, 2048, causal=causal)
    nb = (q.shape[2] + 127) // 128
    ref = X.block_sparse_attention(q, k, v, r["col_idx"], r["col_cnt"], causal=causal)
    assert torch.equal(whole, ref)
    for limit in (150_000, 450_000, 800_000):           # one chunk per group, three, five (of nine)
        monkeypatch.setattr(X, "GROUP_LIMIT", limit)
        plan = X._Plan(q, k, 8, 0.9, 2048, causal, 1, True, False, False, 128, True, False, want_mask=False,
                       group_limit=limit)
        assert len(plan.groups()) > 1
        assert torch.equal(X.Xattention_prefill(q, k, v, 8, **kw), whole), limit
    # a query chunk against a longer cache, grouped
    out = X.Xattention_prefill(q[:, :, -6000:], k, v, 8, **kw)
    monkeypatch.setattr(X, "GROUP_LIMIT", 2 << 30)
    assert torch.equal(X.Xattention_prefill(q[:, :, -6000:], k, v, 8, **kw), out)


def test_window_arguments_are_checked():
    from xattn.src import hip_backend as hb

    lib = hb.lib()
    s = torch.zeros(2, 4, 16, device="cuda")
    tau = torch.full((2,), 0.9, dtype=torch.float64, device="cuda")
    cnt = torch.zeros(2, 4, dtype=torch.int32, device="cuda")
    idx = torch.zeros(2, 4, 16, dtype=torch.int32, device="cuda")
    args = lambda r0, r1, w0, wr: lib.xattn_select_blocks(
        s.data_ptr(), tau.data_ptr(), None, idx.data_ptr(), cnt.data_ptr(), 16, 2, 16, 16, r0, r1, 0, 1, 0, 0, 16,
        2048, 0, 16, w0, wr, None)
    assert args(4, 8, 4, 4) == 0                       # rows 4..7 of 16 in a 4-row window: fine, and no mask wanted
    assert args(4, 9, 4, 4) == -4 and args(3, 8, 4, 4) == -4
    assert lib.xattn_select_blocks(s.data_ptr(), tau.data_ptr(), None, None, None, 16, 2, 16, 16, 0, 4, 0, 1, 0, 0, 16,
                                   2048, 0, 16, 0, 4, None) == -1     # neither mask nor lists: nothing to write
    torch.cuda.synchronize()


def test_a_million_tokens_within_eight_gib_beside_inputs_and_output():
    """L = 1 048 576, 32 query / 8 KV heads (the shape whose block sums alone are 8.6 GB when
    held whole): peak allocation of the operator <= inputs + output + 8 GiB."""
    import xattn.src.Xattention as X
    from xattn.synthetic import WORKLOADS, make_inputs

    w = WORKLOADS[2]
    L = 1 << 20
    q, k, v = make_inputs(w, device="cuda", seed=0, L=L)
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    out = X.Xattention_prefill(q, k, v, 16, threshold=0.9)
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - base
    out_bytes = out.numel() * 2
    print(f"1M tokens: peak beside the inputs {peak / 2**30:.2f} GiB of which output {out_bytes / 2**30:.2f} GiB", flush=True)
    assert peak <= out_bytes + (8 << 30)
    assert out.shape == (1, 32, L, 128)
    # spot checks instead of a full scan of 8 GiB: finite, and the first q-block (which attends only itself)
    # equals dense attention of that block
    sample = out[0, :, ::4099].float()
    assert torch.isfinite(sample).all()
    first = X.block_sparse_attention(q[:, :, :128], k[:, :, :128], v[:, :, :128], causal=True)
    assert torch.equal(out[:, :, :128], first)
