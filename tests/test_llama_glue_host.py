"""Host-side checks of the Llama glue (no GPU): configuration rules and that
patching binds the forward to every attention layer."""
import pytest
import torch

transformers = pytest.importorskip("transformers")


def test_config_rules():
    from xattn.src.load_llama import FastPrefillConfig

    c = FastPrefillConfig(threshold=0.9)
    assert c.stride == 16 and c.metric == "xattn" and c.layer_threshold(5) == 0.9
    t = torch.rand(3, 4)
    c = FastPrefillConfig(threshold=t, stride=8)
    assert torch.equal(c.layer_threshold(2), t[2])
    with pytest.raises(ValueError):
        FastPrefillConfig(threshold=0.9, stride=5)
    with pytest.raises(NotImplementedError):
        FastPrefillConfig(threshold=0.9, metric="minfer")
    with pytest.raises(ValueError):
        FastPrefillConfig(threshold=torch.rand(4))


def test_default_thresholds_come_from_the_profiled_tables(tmp_path, monkeypatch):
    """``FastPrefillConfig()`` with no threshold (the reference's default construction,
    xattn/src/load_llama.py:249-266) reads ``llama_fuse_<stride>``: from the JSON file the
    profiler writes, or from a module of plain lists put in place of the loader."""
    import sys
    import types

    from xattn.src.load_llama import FastPrefillConfig
    from xattn.threshold import llama_threshold

    monkeypatch.setenv("XATTN_THRESHOLD_TABLES", str(tmp_path / "none.json"))
    with pytest.raises(ValueError, match="llama_threshold"):
        FastPrefillConfig()                         # no tables anywhere: the error names where they are looked for
    g = torch.Generator().manual_seed(0)
    t16, t8 = torch.rand(32, 32, generator=g), torch.rand(32, 32, generator=g)
    path = str(tmp_path / "tables.json")
    llama_threshold.write_tables(path, llama_fuse_16=t16)
    llama_threshold.write_tables(path, llama_fuse_8=t8.tolist())       # added to the same file
    monkeypatch.setenv("XATTN_THRESHOLD_TABLES", path)
    c = FastPrefillConfig()
    assert c.stride == 16 and c.threshold.shape == (32, 32) and torch.allclose(c.threshold, t16)
    assert torch.allclose(FastPrefillConfig(stride=8).layer_threshold(12), t8[12])
    with pytest.raises(ValueError, match="llama_fuse_4"):
        FastPrefillConfig(stride=4)                 # that stride was never profiled
    with pytest.raises(ValueError):
        llama_threshold.write_tables(path, llama_fuse_32=t8)
    # the reference's module form: plain module-level lists under the same import path
    stub = types.ModuleType("xattn.threshold.llama_threshold")
    stub.llama_fuse_16 = [[0.5] * 4] * 3
    monkeypatch.setitem(sys.modules, "xattn.threshold.llama_threshold", stub)
    import xattn.threshold as pkg

    monkeypatch.setattr(pkg, "llama_threshold", stub, raising=False)
    c = FastPrefillConfig()
    assert c.threshold.shape == (3, 4) and float(c.layer_threshold(2)[1]) == 0.5


def test_patch_binds_every_layer_and_checks_head_dim():
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaForCausalLM
    from xattn.src.load_llama import FastPrefillConfig, forward_eval, patch_model

    kw = dict(vocab_size=64, hidden_size=256, intermediate_size=256, num_hidden_layers=3, num_key_value_heads=1)
    model = LlamaForCausalLM(LlamaConfig(num_attention_heads=2, head_dim=128, **kw))
    cfg = FastPrefillConfig(threshold=0.8)
    patch_model(model, cfg)
    for layer in model.model.layers:
        assert layer.self_attn.forward.__func__ is forward_eval
        assert layer.self_attn.fastprefillconfig is cfg
    # CPU tensors never reach a kernel: the operator refuses them
    with pytest.raises(Exception), torch.no_grad():
        model(torch.zeros(1, 8, dtype=torch.long))
    small = LlamaForCausalLM(LlamaConfig(num_attention_heads=4, head_dim=64, **kw))
    with pytest.raises(ValueError):
        patch_model(small, cfg)


def test_rotary_matches_model_code():
    from transformers.models.llama import modeling_llama as m
    from xattn.src.load_llama import apply_rotary_pos_emb

    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(1, 4, 10, 128, generator=g), torch.randn(1, 2, 10, 128, generator=g)
    ang = torch.randn(1, 10, 128, generator=g)
    a = apply_rotary_pos_emb(q, k, ang.cos(), ang.sin())
    b = m.apply_rotary_pos_emb(q, k, ang.cos(), ang.sin())
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


@pytest.mark.parametrize("mode", [torch.no_grad, torch.inference_mode])
def test_static_cache_branch_on_the_host(monkeypatch, mode):
    """The preallocated-cache branch of the forward (how much of the cache is filled) with the attention kernels
    replaced by torch reference attention, so that it runs without a GPU: under ``torch.inference_mode()``
    tensors carry no version counter, and the positions may come as ``cache_position`` or ``position_ids``."""
    import copy

    import torch.nn.functional as F
    from transformers import LlamaConfig, StaticCache
    from transformers.models.llama.modeling_llama import LlamaForCausalLM

    from xattn.src import load_llama
    from xattn.src.load_llama import FastPrefillConfig, patch_model

    def attention(q, k, v, causal=True, **kw):
        rep = q.shape[1] // k.shape[1]
        k, v = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
        lq, lk = q.shape[2], k.shape[2]
        mask = torch.ones(lq, lk, dtype=torch.bool).tril(lk - lq)
        return F.scaled_dot_product_attention(q, k, v, attn_mask=mask)

    def decode(q, k, v, kv_layout="HND", **kw):
        return attention(q[None, :, None, :], k[None], v[None])[0, :, 0]

    monkeypatch.setattr(load_llama, "block_sparse_attention", attention)
    monkeypatch.setattr(load_llama, "single_decode_with_kv_cache", decode)
    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=128, hidden_size=256, intermediate_size=256, num_hidden_layers=2, num_attention_heads=2,
                      num_key_value_heads=1, head_dim=128, max_position_embeddings=512, attn_implementation="eager")
    stock = LlamaForCausalLM(cfg).eval()
    ours = patch_model(copy.deepcopy(stock), FastPrefillConfig(threshold=0.9, metric="full"))
    ids = torch.randint(0, 128, (1, 40), generator=torch.Generator().manual_seed(1))
    with mode():
        a = stock(ids, use_cache=True)
        cache = StaticCache(config=ours.config, max_cache_len=64)
        b = ours(ids, past_key_values=cache, use_cache=True)
        assert torch.allclose(b.logits, a.logits, atol=1e-4, rtol=1e-4)
        nxt = a.logits[:, -1:].argmax(-1)
        for step in range(2):
            a = stock(nxt, past_key_values=a.past_key_values, use_cache=True)
            b = ours(nxt, past_key_values=cache, use_cache=True)
            assert torch.allclose(b.logits, a.logits, atol=1e-4, rtol=1e-4), step
            nxt = a.logits[:, -1:].argmax(-1)
    # positions through position_ids only (an attention layer called without cache_position)
    layer = ours.model.layers[0].self_attn
    with mode():
        cache2 = StaticCache(config=ours.config, max_cache_len=64)
        h = torch.randn(1, 10, 256)
        pos = torch.arange(10)[None]
        cos, sin = ours.model.rotary_emb(h, pos)
        out = layer(h, position_embeddings=(cos, sin), past_key_values=cache2, position_ids=pos)[0]
        assert out.shape == (1, 10, 256) and torch.isfinite(out).all()
