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
