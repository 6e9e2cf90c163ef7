"""GPU: the decode step, the block-sparse attention launch and the whole
prefill operator are capturable in a HIP graph (nothing is allocated or
synchronised inside the entry points, and the operator never reads back):
every replay, with new contents in the same buffers and eager work in
between, must reproduce the eager result bit for bit."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_decode_step_replays_from_a_graph():
    from xattn.src import hip_backend as hb
    from xattn.src.decode import single_decode_with_kv_cache

    H, Hkv, L = 32, 8, 5000
    g = torch.Generator(device="cuda").manual_seed(0)
    q = torch.randn(H, 128, device="cuda", generator=g).bfloat16()
    k = torch.randn(Hkv, L, 128, device="cuda", generator=g).bfloat16()
    v = torch.randn(Hkv, L, 128, device="cuda", generator=g).bfloat16()
    ws = torch.empty(hb.lib().xattn_decode_workspace_bytes(H, Hkv, L), dtype=torch.uint8, device="cuda")
    out = torch.empty(H, 128, dtype=torch.bfloat16, device="cuda")
    single_decode_with_kv_cache(q, k, v, "HND", out=out, workspace=ws)      # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        single_decode_with_kv_cache(q, k, v, "HND", out=out, workspace=ws)
    for i in range(4):
        q.copy_(torch.randn(H, 128, device="cuda", generator=g).bfloat16())
        k[:, i * 100:(i + 1) * 100].mul_(-1.5)                                # eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = single_decode_with_kv_cache(q, k, v, "HND")
        torch.cuda.synchronize()
        assert torch.equal(got, want), i


def test_block_sparse_attention_replays_from_a_graph():
    from xattn.src.Xattention import block_sparse_attention, estimate_and_select
    from xattn.synthetic import WORKLOADS, make_inputs

    q, k, v = make_inputs(WORKLOADS[1], device="cuda", seed=2, L=4096, heads=8, kv_heads=2)
    r = estimate_and_select(q, k, 8, 0.9, 2048)
    out = torch.empty(1, 4096, 8, 128, dtype=torch.bfloat16, device="cuda")
    block_sparse_attention(q, k, v, r["col_idx"], r["col_cnt"], out=out)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        block_sparse_attention(q, k, v, r["col_idx"], r["col_cnt"], out=out)
    for i in range(3):
        v.mul_(0.5 + i)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = block_sparse_attention(q, k, v, r["col_idx"], r["col_cnt"])
        torch.cuda.synchronize()
        assert torch.equal(got.transpose(1, 2), want), i


def test_whole_operator_replays_from_a_graph():
    """estimate -> select -> attention captured as one graph (temporaries from the
    capture's memory pool): the selection changes with the inputs from replay
    to replay, and every replay equals the eager call."""
    from xattn.src.Xattention import Xattention_prefill
    from xattn.synthetic import WORKLOADS, make_inputs

    w = WORKLOADS[1]
    q, k, v = make_inputs(w, device="cuda", seed=3, L=4096 + 200, heads=8, kv_heads=2)
    kw = dict(threshold=0.9, chunk_size=2048)
    Xattention_prefill(q, k, v, 8, **kw)                                      # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = Xattention_prefill(q, k, v, 8, **kw)
    for i in range(3):
        q2, k2, v2 = make_inputs(w, device="cuda", seed=10 + i, L=4096 + 200, heads=8, kv_heads=2)
        q.copy_(q2), k.copy_(k2), v.copy_(v2)                                 # eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = Xattention_prefill(q, k, v, 8, **kw)
        torch.cuda.synchronize()
        assert torch.equal(got, want), i
