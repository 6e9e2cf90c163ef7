"""GPU parity over a seeded sweep of random operator configurations (strides,
chunk sizes, head groupings, ragged lengths, k_len > q_len, causal or not,
keep flags, scalar and per-head thresholds): block sums, masks and outputs of
the HIP path against the oracle on identical inputs."""
import random

import pytest
import torch

from helpers import OUT_MAX_ABS, OUT_MEAN_ABS, lists_from_mask, mask_mismatch_report
from oracle import xattn_oracle as O

pytestmark = pytest.mark.gpu


def _cases(n, seed):
    rng = random.Random(seed)
    out = []
    for i in range(n):
        S = rng.choice([4, 8, 16])
        C = rng.choice([256, 512, 1024, 2048])
        heads, kv = rng.choice([(4, 4), (4, 2), (8, 2), (6, 3), (4, 1), (7, 1)])
        causal = rng.random() < 0.7
        Lq = rng.randint(1, 24) * 100 + rng.choice([0, 28, 1, 127])
        extra = rng.choice([0, 0, 0, 128, 384, 1024]) if causal else 0     # key blocks ahead of the queries
        Lk = Lq + extra
        if extra and Lq % 128:
            Lq -= Lq % 128                                                # cached prefixes come in whole blocks
            Lk = Lq + extra
        tau = rng.choice([0.9, 0.8, 0.95, 0.5, "per_head"])
        out.append(dict(S=S, C=C, H=heads, Hkv=kv, causal=causal, Lq=max(Lq, 128 if extra else 1), Lk=max(Lk, 1),
                        tau=tau, keep_sink=rng.random() < 0.2, keep_recent=rng.random() < 0.2,
                        use_triton=rng.random() < 0.7, seed=1000 + i))
    return out


@pytest.mark.parametrize("c", _cases(72, 7), ids=lambda c: f"S{c['S']}C{c['C']}H{c['H']}x{c['Hkv']}q{c['Lq']}k{c['Lk']}{'c' if c['causal'] else 'n'}")
def test_random_configuration(c):
    from xattn.src.Xattention import Xattention_prefill, block_sparse_attention, xattn_estimate
    from xattn.synthetic import WORKLOADS, make_inputs

    H, Hkv, Lq, Lk, S, C = c["H"], c["Hkv"], c["Lq"], c["Lk"], c["S"], c["C"]
    q_all, k, v = make_inputs(WORKLOADS[1], device="cpu", seed=c["seed"], L=Lk, heads=H, kv_heads=Hkv)
    q = q_all[:, :, Lk - Lq:].contiguous()
    g = torch.Generator().manual_seed(c["seed"])
    tau = torch.rand(H, generator=g) * 0.6 + 0.35 if c["tau"] == "per_head" else c["tau"]
    group = H // Hkv
    kw = dict(threshold=tau, chunk_size=C, causal=c["causal"], keep_sink=c["keep_sink"], keep_recent=c["keep_recent"])

    want_sums, want_mask = O.xattn_estimate(q.float(), k.repeat_interleave(group, 1).float(), 128, S,
                                            pad0_quirk=not c["use_triton"], **kw)
    tau_dev = tau.cuda() if isinstance(tau, torch.Tensor) else tau
    sums, mask = xattn_estimate(q.cuda(), k.cuda(), 128, S, use_triton=c["use_triton"],
                                **{**kw, "threshold": tau_dev})
    assert mask.shape == want_mask.shape
    assert torch.allclose(sums.float().cpu(), want_sums, rtol=1e-2, atol=2e-3)          # bf16 result of the operator
    # (blocks the keep flags force are set on both sides and cannot mismatch themselves)
    nq_p, nk_p = mask.shape[2], mask.shape[3]
    nbad, outside = mask_mismatch_report(want_sums[0], mask[0], want_mask[0], tau, c["causal"], nk_p - nq_p, C // 128,
                                         keep_recent=c["keep_recent"])
    assert outside == 0, (nbad, outside)

    nq, nk = (Lq + 127) // 128, (Lk + 127) // 128
    m = mask[0, :, :nq, :nk].cpu()
    idx, cnt = lists_from_mask(m)
    out = block_sparse_attention(q.cuda(), k.cuda(), v.cuda(), idx.cuda(), cnt.cuda(), causal=c["causal"])
    # fp32 oracle output: rows that attend a single key reproduce |v| up to 4-5, where one bf16 step is 0.03
    want = O.block_sparse_attention(q.float(), k.float(), v.float(), m[None], causal=c["causal"])
    err = (out.float().cpu() - want.float()).abs()
    assert err.max().item() <= OUT_MAX_ABS and err.mean().item() <= OUT_MEAN_ABS
    full = Xattention_prefill(q.cuda(), k.cuda(), v.cuda(), S, use_triton=c["use_triton"], **{**kw, "threshold": tau_dev})
    assert torch.equal(full, out)           # the operator is these two steps


def _wide_cases(n, seed):
    """Wider ranges than above: chunk sizes down to one block, head groupings up to 16:2 and 9:1, lengths that
    are no multiple of anything, cached prefixes of any length (the q-blocks then straddle key blocks), the three
    input generators, thresholds from 0 to 1, query-row subsampling and norm on the torch branch, and inputs that
    live in [L, H, d] memory."""
    rng = random.Random(seed)
    out = []
    for i in range(n):
        S = rng.choice([4, 8, 16])
        C = rng.choice([128, 256, 384, 512, 1024, 2048, 4096])
        H, Hkv = rng.choice([(4, 4), (4, 2), (8, 2), (6, 3), (4, 1), (7, 1), (16, 2), (12, 4), (1, 1), (3, 3), (10, 2), (9, 1)])
        causal = rng.random() < 0.7
        Lq = rng.randint(1, 3000)
        extra = rng.choice([0, 0, 1, 77, 128, 300, 1000, rng.randint(1, 2000)]) if causal else rng.choice([0, 0, 50, 700])
        Lk = Lq + extra
        if causal and Lk <= 128 and C == 128:
            Lq, Lk = Lq + 128, Lk + 128          # a single key block: the reference itself raises (scatter shape)
        use_triton = rng.random() < 0.6
        kdb = 1 if use_triton else rng.choice([1, 1, 2, 4])
        if (128 // S) % kdb:
            kdb = 1
        out.append(dict(S=S, C=C, H=H, Hkv=Hkv, causal=causal, Lq=Lq, Lk=Lk, wl=rng.choice([1, 1, 1, 3, 4]),
                        tau=rng.choice([0.9, 0.8, 0.95, 0.5, 0.99, 0.999, 1.0, 0.0, 0.3, "per_head", "per_head"]),
                        use_triton=use_triton, kdb=kdb, norm=rng.choice([1, 1, 1, 2, 0.5]),
                        keep_sink=rng.random() < 0.2, keep_recent=rng.random() < 0.2,
                        nhd=rng.random() < 0.5, seed=5000 + i))
    return out


@pytest.mark.parametrize("c", _wide_cases(96, 11), ids=lambda c: f"S{c['S']}C{c['C']}H{c['H']}x{c['Hkv']}q{c['Lq']}k{c['Lk']}{'c' if c['causal'] else 'n'}{'t' if c['use_triton'] else 'p'}d{c['kdb']}")
def test_random_configuration_wide(c):
    from xattn.src.Xattention import Xattention_prefill, block_sparse_attention, xattn_estimate
    from xattn.synthetic import WORKLOADS, make_inputs

    H, Hkv, Lq, Lk, S, C = c["H"], c["Hkv"], c["Lq"], c["Lk"], c["S"], c["C"]
    q_all, k, v = make_inputs(WORKLOADS[c["wl"]], device="cpu", seed=c["seed"], L=Lk, heads=H, kv_heads=Hkv)
    q = q_all[:, :, Lk - Lq:].contiguous()
    g = torch.Generator().manual_seed(c["seed"])
    tau = torch.rand(H, generator=g) * 0.7 + 0.3 if c["tau"] == "per_head" else c["tau"]
    kw = dict(threshold=tau, chunk_size=C, causal=c["causal"], keep_sink=c["keep_sink"], keep_recent=c["keep_recent"],
              norm=c["norm"], kdb=c["kdb"])
    want_sums, want_mask = O.xattn_estimate(q.float(), k.repeat_interleave(H // Hkv, 1).float(), 128, S,
                                            pad0_quirk=not c["use_triton"], **kw)

    def dev(t):
        t = t.cuda()
        return t.transpose(1, 2).contiguous().transpose(1, 2) if c["nhd"] else t      # [B, L, H, d] memory

    qd, kd, vd = dev(q), dev(k), dev(v)
    kw["threshold"] = tau.cuda() if isinstance(tau, torch.Tensor) else tau
    sums, mask = xattn_estimate(qd, kd, 128, S, use_triton=c["use_triton"], **kw)
    assert mask.shape == want_mask.shape
    assert torch.allclose(sums.float().cpu(), want_sums, rtol=1e-2, atol=2e-3)
    nq_p, nk_p = mask.shape[2], mask.shape[3]
    nbad, outside = mask_mismatch_report(want_sums[0], mask[0], want_mask[0], tau, c["causal"], nk_p - nq_p, C // 128,
                                         keep_recent=c["keep_recent"])
    assert outside == 0, (nbad, outside)
    nq, nk = (Lq + 127) // 128, (Lk + 127) // 128
    m = mask[0, :, :nq, :nk].cpu()
    idx, cnt = lists_from_mask(m)
    out = block_sparse_attention(qd, kd, vd, idx.cuda(), cnt.cuda(), causal=c["causal"])
    want = O.block_sparse_attention(q.float(), k.float(), v.float(), m[None], causal=c["causal"])
    err = (out.float().cpu() - want.float()).abs()
    # one bf16 step of the stored output where it is larger than the absolute tolerance (|out| > 2.56)
    assert bool((err <= torch.clamp(want.float().abs() * 2.0 ** -7, min=OUT_MAX_ABS)).all())
    assert err.mean().item() <= OUT_MEAN_ABS
    assert torch.equal(Xattention_prefill(qd, kd, vd, S, use_triton=c["use_triton"], **kw), out)
