"""GPU: the allocation-free decode entry point (xattn_decode_fwd_static) gives
the very output of xattn_decode_fwd, on two calls in a row of which the second
is smaller, and is refused beyond the size of its built-in scratch array."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(lib, hb, q, k, v):
    heads, kv_heads, kv_len = q.shape[0], k.shape[0], k.shape[1]
    stream = torch.cuda.current_stream().cuda_stream
    scale = 1.0 / math.sqrt(128)
    ws = torch.empty(lib.xattn_decode_workspace_bytes(heads, kv_heads, kv_len), dtype=torch.uint8, device="cuda")
    a = torch.full((heads, 128), float("nan"), dtype=torch.bfloat16, device="cuda")
    b = torch.full((heads, 128), float("nan"), dtype=torch.bfloat16, device="cuda")
    hb.check(lib.xattn_decode_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), a.data_ptr(), ws.data_ptr(), ws.numel(),
                                  heads, kv_heads, kv_len, 128, q.stride(0), k.stride(0), k.stride(1), v.stride(0),
                                  v.stride(1), a.stride(0), scale, stream), "xattn_decode_fwd")
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    hb.check(lib.xattn_decode_fwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), b.data_ptr(), heads, kv_heads,
                                         kv_len, 128, q.stride(0), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
                                         b.stride(0), scale, stream), "xattn_decode_fwd_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return a, b


def test_static_decode_equals_workspace_decode_twice_second_smaller():
    from oracle import xattn_oracle as O
    from xattn.src import hip_backend as hb

    lib = hb.lib()
    g = torch.Generator().manual_seed(0)
    for heads, kv_heads, kv_len in ((32, 8, 40000), (8, 2, 3001)):       # the second call is the smaller one
        print(f"static decode: heads {heads}/{kv_heads}, kv_len {kv_len}", flush=True)
        q = torch.randn(heads, 128, generator=g).bfloat16().cuda()
        k = torch.randn(kv_heads, kv_len, 128, generator=g).bfloat16().cuda()
        v = torch.randn(kv_heads, kv_len, 128, generator=g).bfloat16().cuda()
        a, b = _both(lib, hb, q, k, v)
        assert torch.isfinite(b.float()).all()
        assert torch.equal(a, b)
        want = O.single_decode_with_kv_cache(q.cpu().float(), k.cpu().float(), v.cpu().float(), kv_layout="HND")
        assert (b.float().cpu() - want).abs().max().item() <= 2e-2


def test_static_decode_through_the_python_wrapper_and_its_limit():
    from xattn.src import hip_backend as hb
    from xattn.src.decode import single_decode_with_kv_cache

    lib = hb.lib()
    g = torch.Generator().manual_seed(1)
    q = torch.randn(16, 128, generator=g).bfloat16().cuda()
    k = torch.randn(5000, 4, 128, generator=g).bfloat16().cuda()
    v = torch.randn(5000, 4, 128, generator=g).bfloat16().cuda()
    out = torch.empty(16, 128, dtype=torch.bfloat16, device="cuda")
    got = single_decode_with_kv_cache(q, k, v, out=out, static_scratch=True)
    assert got is out
    assert torch.equal(out, single_decode_with_kv_cache(q, k, v))
    # 512 KV heads x 32 query heads each need more (range, head) pairs than the array holds
    big = lib.xattn_decode_fwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), 512 * 32, 512, 64, 128,
                                      128, 128 * 64, 128, 128 * 64, 128, 128, 0.1, None)
    assert big == -7 and b"workspace" in lib.xattn_error_string(big)
    assert lib.xattn_decode_fwd_static(None, k.data_ptr(), v.data_ptr(), out.data_ptr(), 16, 4, 5000, 128,
                                       128, 128, 512, 128, 512, 128, 0.1, None) == -1


def test_static_decode_replays_from_a_graph():
    """What the entry point is for: a capture refuses allocations (hipMalloc inside a capturing stream is an
    error), so a graph that holds the static form and replays correctly shows that it allocates nothing -
    which the allocator statistics above cannot (they only see torch's own allocator)."""
    from xattn.src.decode import single_decode_with_kv_cache

    H, Hkv, L = 32, 8, 6000
    g = torch.Generator(device="cuda").manual_seed(3)
    q = torch.randn(H, 128, device="cuda", generator=g).bfloat16()
    k = torch.randn(Hkv, L, 128, device="cuda", generator=g).bfloat16()
    v = torch.randn(Hkv, L, 128, device="cuda", generator=g).bfloat16()
    out = torch.empty(H, 128, dtype=torch.bfloat16, device="cuda")
    single_decode_with_kv_cache(q, k, v, "HND", out=out, static_scratch=True)   # the symbol lookup happens here
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        single_decode_with_kv_cache(q, k, v, "HND", out=out, static_scratch=True)
    for i in range(3):
        q.copy_(torch.randn(H, 128, device="cuda", generator=g).bfloat16())
        v[:, i * 50:(i + 1) * 50].mul_(2.0)                                      # eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = single_decode_with_kv_cache(q, k, v, "HND")                       # the workspace form, eager
        torch.cuda.synchronize()
        assert torch.equal(got, want), i
