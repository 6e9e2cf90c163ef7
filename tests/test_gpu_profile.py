"""GPU parity of the threshold profiler: xattn_block_mass and
xattn_threshold_rows (through the C ABI) vs the CPU oracle, and the profiler
run over a small random-weight Llama."""
import pytest
import torch

from oracle import xattn_oracle as O

pytestmark = pytest.mark.gpu

MASS_ATOL, MASS_RTOL = 2e-3, 1e-3     # block masses are sums of up to 16384 fp32 probabilities
THR_ATOL = 1e-4                       # thresholds from identical inputs


@pytest.mark.parametrize("shape", [(4, 2, 1024), (4, 4, 300), (8, 2, 1000), (2, 1, 128), (3, 1, 2500)])
def test_block_mass_matches_oracle(shape):
    from xattn.synthetic import WORKLOADS, make_inputs
    from xattn.threshold.profile_threshold.profile_threshold import chunk_prefill_to_attn_sum

    H, Hkv, L = shape
    q, k, _ = make_inputs(WORKLOADS[1], device="cpu", seed=4, L=L, heads=H, kv_heads=Hkv)
    got = chunk_prefill_to_attn_sum(q.cuda(), k.cuda(), 128).cpu()
    want = O.chunk_prefill_to_attn_sum(q, k, 128)
    assert got.shape == want.shape and got.dtype == torch.float32
    assert torch.allclose(got, want, atol=MASS_ATOL, rtol=MASS_RTOL), (got - want).abs().max()
    nb = (L + 127) // 128
    rows = torch.tensor([min(128, L - i * 128) for i in range(nb)], dtype=torch.float32)
    assert torch.allclose(got.sum(-1), rows.expand(1, H, nb), atol=1e-2)
    assert (got.triu(1) == 0).all()


def test_block_mass_takes_strided_views():
    from xattn.threshold.profile_threshold.profile_threshold import chunk_prefill_to_attn_sum

    g = torch.Generator().manual_seed(5)
    q = torch.randn(1, 700, 4, 128, generator=g).bfloat16()
    k = torch.randn(1, 700, 2, 128, generator=g).bfloat16()
    got = chunk_prefill_to_attn_sum(q.cuda().transpose(1, 2), k.cuda().transpose(1, 2), 128).cpu()
    want = O.chunk_prefill_to_attn_sum(q.transpose(1, 2), k.transpose(1, 2), 128)
    assert torch.allclose(got, want, atol=MASS_ATOL, rtol=MASS_RTOL)


@pytest.mark.parametrize("coverage", [0.9, 0.5, 0.99])
def test_threshold_rows_match_oracle(coverage):
    from xattn.threshold.profile_threshold.profile_threshold import profile_threshold_head

    g = torch.Generator().manual_seed(6)
    H, nq, nk = 5, 37, 37
    attn = (torch.rand(1, H, nq, nk, generator=g) ** 4).tril().contiguous()
    attn[0, 0, 3] = 0                                   # a row without mass
    x_pad = torch.zeros(1, H, 48, 64)                   # the estimator's padded layout
    x_pad[:, :, :nq, :nk] = (attn + 0.1 * torch.rand(1, H, nq, nk, generator=g)).tril()
    got = profile_threshold_head(attn.cuda(), x_pad.cuda(), coverage).cpu()
    want = O.profile_threshold_head(attn, x_pad[:, :, :nq, :nk], coverage)
    assert got.shape == (1, H)
    assert torch.allclose(got, want, atol=THR_ATOL), (got, want)


def test_threshold_rows_wide_row():
    from xattn.threshold.profile_threshold.profile_threshold import profile_threshold_head

    g = torch.Generator().manual_seed(7)
    attn = torch.rand(1, 2, 3, 1500, generator=g).contiguous()   # diffuse rows: hundreds of blocks taken
    x = attn * (0.5 + torch.rand(1, 2, 3, 1500, generator=g))
    got = profile_threshold_head(attn.cuda(), x.cuda(), 0.9).cpu()
    assert torch.allclose(got, O.profile_threshold_head(attn, x, 0.9), atol=1e-3)


def test_profile_model_on_small_llama():
    transformers = pytest.importorskip("transformers")
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaForCausalLM
    from xattn.threshold.profile_threshold import profile_threshold as PT

    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=512, hidden_size=512, intermediate_size=1024, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=2, head_dim=128, max_position_embeddings=8192)
    model = LlamaForCausalLM(cfg).to(torch.bfloat16).cuda().eval()
    seen = []
    real = PT.xattn_prefill_profile

    def spy(self, q, k, v, block_size, stride, **kw):
        seen.append((self.layer_idx, q.detach().cpu(), k.detach().cpu(), stride))
        return real(self, q, k, v, block_size, stride, **kw)

    PT_forward_globals = PT.forward_profile.__globals__
    old = PT_forward_globals["xattn_prefill_profile"]
    PT_forward_globals["xattn_prefill_profile"] = spy
    try:
        gen = torch.Generator().manual_seed(1)
        texts = [torch.randint(0, 512, (1, n), generator=gen) for n in (1536, 900)]
        table = PT.profile_model(model, PT.ProfileConfig(stride=8), texts)
    finally:
        PT_forward_globals["xattn_prefill_profile"] = old
    assert table.shape == (2, 4) and ((table > 0) & (table <= 1)).all()
    # the same table from the oracle, fed with the tensors the layers saw
    from xattn.src.Xattention import default_chunk_size

    per_text = []
    for t in range(2):
        rows = []
        for layer, q, k, stride in seen[2 * t: 2 * t + 2]:
            attn = O.chunk_prefill_to_attn_sum(q, k, 128)
            nb = attn.shape[-1]
            sums, _ = O.xattn_estimate(q.float(), k.repeat_interleave(2, 1).float(), 128, stride, threshold=1.0,
                                       chunk_size=16384, pad0_quirk=False)
            rows.append(O.profile_threshold_head(attn, sums[:, :, :nb, :nb] * stride))
        per_text.append(torch.cat(rows, 0))
    want = torch.stack(per_text).max(0)[0]
    assert torch.allclose(table.cpu(), want, atol=2e-2), (table, want)
