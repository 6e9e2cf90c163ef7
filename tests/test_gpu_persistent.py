"""GPU: the persistent (ticket-queue) launch of the block-sparse attention kernel
computes exactly what the one-workgroup-per-unit launch computes, leaves its
ticket counters at zero, and matches the oracle."""
import pytest
import torch

from helpers import OUT_MAX_ABS, OUT_MEAN_ABS, lists_from_mask
from oracle import xattn_oracle as O

pytestmark = pytest.mark.gpu


def _inputs(H, Hkv, Lq, Lk, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(1, H, Lq, 128, generator=g).bfloat16().cuda()
    k = torch.randn(1, Hkv, Lk, 128, generator=g).bfloat16().cuda()
    v = torch.randn(1, Hkv, Lk, 128, generator=g).bfloat16().cuda()
    return q, k, v


def _mask(H, nq, nk, causal, density, seed, heavy_head=None):
    g = torch.Generator().manual_seed(seed)
    m = torch.rand(H, nq, nk, generator=g) < density
    if heavy_head is not None:
        m[heavy_head] = torch.rand(nq, nk, generator=g) < 0.6       # one head with long lists, like real workloads
    off = nk - nq
    ar_q, ar_k = torch.arange(nq), torch.arange(nk)
    if causal:
        m &= ar_k[None, :] <= ar_q[:, None] + off
        m[:, ar_q, ar_q + off] = True
    m[:, :, 0] = True
    m[0, 3] = False                  # a unit without any block
    m[1, 5] = False
    m[1, 5, 0] = True                # a unit with exactly one block
    return m


def _queues_are_zero():
    import xattn.src.Xattention as X

    torch.cuda.synchronize()
    return all(int(t.abs().sum()) == 0 for t in X._queues.values())


@pytest.mark.parametrize("H,Hkv,Lq,Lk,causal", [
    (8, 2, 16384, 16384, True),       # 4 query heads per KV head
    (28, 4, 8192, 8192, True),        # 7 per KV head: gaps in the ticket map
    (8, 8, 6000, 6000, False),        # ragged, non-causal
    (8, 2, 4096, 20480, True),        # chunk of queries against a longer cache
    (71, 1, 2048, 2048, True),        # more than 64 query heads on one KV head
])
def test_persistent_equals_plain_launch(H, Hkv, Lq, Lk, causal):
    from xattn.src.Xattention import block_sparse_attention

    q, k, v = _inputs(H, Hkv, Lq, Lk, 1)
    nq, nk = (Lq + 127) // 128, (Lk + 127) // 128
    mask = _mask(H, nq, nk, causal, 0.06, 2, heavy_head=H - 1)
    idx, cnt = lists_from_mask(mask)
    idx, cnt = idx.cuda(), cnt.cuda()
    plain = block_sparse_attention(q, k, v, idx, cnt, causal=causal, persistent=False)
    for _ in range(2):               # twice: the second launch finds the counters the first one left
        pers = block_sparse_attention(q, k, v, idx, cnt, causal=causal, persistent=True)
        assert torch.equal(pers, plain)
        assert _queues_are_zero()
    assert (pers[0, 0, 3 * 128 : 4 * 128].float() == 0).all()
    # against the oracle on a few query blocks (all keys)
    for h, qb in [(0, 0), (1, 5), (H - 1, nq - 1), (H // 2, nq // 2)]:
        r0, r1 = qb * 128, min(Lq, qb * 128 + 128)
        kv = h // (H // Hkv)
        want = O.block_sparse_attention(q[:, h:h + 1, r0:r1].float().cpu(), k[:, kv:kv + 1].float().cpu(),
                                        v[:, kv:kv + 1].float().cpu(), mask[h:h + 1, qb:qb + 1][None],
                                        causal=False) if not causal else None
        if causal:
            # bottom-right aligned causal mask for this block of rows: give the oracle the whole row range up to r1
            want = O.block_sparse_attention(q[:, h:h + 1, :r1].float().cpu(), k[:, kv:kv + 1, :r1 + Lk - Lq].float().cpu(),
                                            v[:, kv:kv + 1, :r1 + Lk - Lq].float().cpu(),
                                            mask[h:h + 1, :qb + 1, :(r1 + Lk - Lq + 127) // 128][None], causal=True)[:, :, r0:r1]
        err = (pers[:, h:h + 1, r0:r1].float().cpu() - want).abs()
        assert err.max().item() <= OUT_MAX_ABS and err.mean().item() <= OUT_MEAN_ABS, (h, qb)


def test_persistent_launch_over_a_q_block_range_and_on_a_side_stream():
    from xattn.src.Xattention import block_sparse_attention

    H, Hkv, L = 16, 4, 16384
    q, k, v = _inputs(H, Hkv, L, L, 3)
    nb = L // 128
    idx, cnt = lists_from_mask(_mask(H, nb, nb, True, 0.05, 4))
    idx, cnt = idx.cuda(), cnt.cuda()
    whole = block_sparse_attention(q, k, v, idx, cnt, causal=True, persistent=False)
    out = torch.zeros((1, L, H, 128), dtype=torch.bfloat16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    block_sparse_attention(q, k, v, idx, cnt, causal=True, out=out, q_blocks=(0, 48))
    block_sparse_attention(q, k, v, idx, cnt, causal=True, out=out, q_blocks=(48, nb), stream=side)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert torch.equal(out.transpose(1, 2), whole)
    assert _queues_are_zero()


def test_operator_uses_the_persistent_launch_and_matches_the_plain_one():
    import xattn.src.Xattention as X
    from xattn.synthetic import WORKLOADS, make_inputs

    w = WORKLOADS[1]
    q, k, v = make_inputs(w, device="cuda", seed=0, L=16384)
    r = X.estimate_and_select(q, k, w.stride, w.threshold, 4096, causal=True)
    a = X.block_sparse_attention(q, k, v, r["col_idx"], r["col_cnt"], causal=True, persistent=False)
    b = X.Xattention_prefill(q, k, v, w.stride, threshold=w.threshold, chunk_size=4096)
    assert torch.equal(a, b)
    assert _queues_are_zero()
