"""Configuration, registry, weight loading errors and the random-weights mode (no GPU)."""
import json

import pytest
import torch
from safetensors.torch import save_file

from tessweave_engine_amd.models.qwen2 import Qwen2Config
from tessweave_engine_amd.config import (ConfigError, EngineConfig, build_model, config_from_dict,
                                         read_model_config, register_architecture, registered_architectures,
                                         unregister_architecture)
from tessweave_engine_amd.weights import (WeightError, random_tensors, read_tensors, write_model_folder)
from tiny_configs import TINY_A, TINY_B

BASE = dict(model_type="qwen2", vocab_size=128, hidden_size=32, intermediate_size=64, num_hidden_layers=2,
            num_attention_heads=4, max_position_embeddings=128)


def test_defaults_follow_the_reference():
    c = config_from_dict(BASE)
    assert isinstance(c, Qwen2Config)
    assert (c.num_key_value_heads, c.head_dim) == (4, 8)                  # kv heads default to heads, head_dim to H/heads
    assert (c.rms_norm_eps, c.rope_theta, c.tie_word_embeddings) == (1e-6, 10000.0, False)
    assert c.attention_bias is True                                       # qwen2: q/k/v biases always on
    assert config_from_dict({**BASE, "attention_bias": False}).attention_bias is True
    assert c.eos_token_ids == ()
    assert config_from_dict({**BASE, "eos_token_id": 7}).eos_token_ids == (7,)
    assert config_from_dict({**BASE, "eos_token_id": [7, 9]}).eos_token_ids == (7, 9)
    assert c.kv_bytes_per_token(4) == 2 * 2 * 4 * 8 * 4
    # KV bytes vector of the reference's docs: L24, Hk2, D64 -> 24 KiB per token in fp32
    big = config_from_dict({**BASE, "hidden_size": 896, "num_attention_heads": 14, "num_key_value_heads": 2,
                            "num_hidden_layers": 24})
    assert big.head_dim == 64 and big.kv_bytes_per_token(4) == 24 * 1024
    # to_dict round trip
    assert config_from_dict(c.to_dict()) == c
    for name, cfg in (("A", TINY_A), ("B", TINY_B)):
        t = config_from_dict(cfg)
        assert t.hidden_size == t.num_attention_heads * t.head_dim, name


@pytest.mark.parametrize("override", [
    {"model_type": "gemma4"}, {"use_sliding_window": True}, {"rope_scaling": {"rope_type": "yarn"}},
    {"quantization_config": {"bits": 4}}, {"auto_map": {"AutoModel": "run_me.py"}}, {"hidden_act": "gelu"},
    {"mlp_bias": True}, {"num_experts": 8}, {"num_local_experts": 2}, {"num_key_value_heads": 3},
    {"head_dim": 16}, {"hidden_size": 30}, {"vocab_size": 0}, {"num_hidden_layers": 0}, {"rms_norm_eps": 0.0}])
def test_unsupported_semantics_rejected(override):
    with pytest.raises(ValueError):
        config_from_dict({**BASE, "architectures": ["Qwen2ForCausalLM"], **override})


def test_accepted_variants_and_missing_keys():
    config_from_dict({**BASE, "rope_scaling": {"rope_type": "default"}})
    config_from_dict({**BASE, "sliding_window": 4096, "max_window_layers": 28})       # ignored while the flag is off
    with pytest.raises(ConfigError):
        config_from_dict({k: v for k, v in BASE.items() if k != "intermediate_size"})
    with pytest.raises(ConfigError):
        config_from_dict({**BASE, "architectures": ["LlamaForCausalLM"], "model_type": "llama"})


def test_registry_and_generation_config(tmp_path):
    assert "Qwen2ForCausalLM" in registered_architectures()
    (tmp_path / "config.json").write_text(json.dumps({**BASE, "architectures": ["Qwen2ForCausalLM"], "eos_token_id": 3}))
    assert read_model_config(tmp_path).eos_token_ids == (3,)
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [5, 6]}))
    assert read_model_config(tmp_path).eos_token_ids == (5, 6)
    with pytest.raises(ConfigError):
        read_model_config(tmp_path / "nowhere")

    class Other:
        @classmethod
        def from_dict(cls, d):
            return "parsed"
    register_architecture("OtherForCausalLM", "other", Other, lambda c: "built")
    try:
        assert config_from_dict({"architectures": ["OtherForCausalLM"]}) == "parsed"
        assert config_from_dict({"model_type": "other"}) == "parsed"
        with pytest.raises(ValueError):
            register_architecture("OtherForCausalLM", "other", Other, lambda c: None)
    finally:
        unregister_architecture("OtherForCausalLM")


def test_engine_config_validation():
    c = EngineConfig()
    assert (c.block_size, c.kv_blocks, c.max_context, c.max_active, c.max_queue, c.prefill_chunk,
            c.min_prefill_chunk, c.target_step_ms, c.prefix_cache) == (16, 256, 2048, 4, 32, 256, 16, 50.0, True)
    assert c.step_token_budget == 4 + 256
    for bad in (dict(block_size=0), dict(kv_blocks=-1), dict(prefill_chunk=8, min_prefill_chunk=16),
                dict(target_step_ms=0), dict(dtype="float16"), dict(max_step_tokens=3, max_active=4)):
        with pytest.raises(ValueError):
            EngineConfig(**bad)


# ---------------------------------------------------------------------------------------
def specs_for(cfg):
    return build_model(config_from_dict(cfg)).tensor_specs()


def test_tensor_names_are_the_checkpoints():
    names = {s.name for s in specs_for(TINY_B) if s.optional_alias_of is None}
    assert len(names) == 12 * 3 + 3
    for key in ("model.embed_tokens.weight", "model.norm.weight", "lm_head.weight",
                "model.layers.2.self_attn.q_proj.bias", "model.layers.0.self_attn.o_proj.weight",
                "model.layers.1.mlp.gate_proj.weight", "model.layers.1.post_attention_layernorm.weight"):
        assert key in names
    assert not any("o_proj.bias" in n or "mlp" in n and "bias" in n for n in names)
    tied = {s.name for s in specs_for(TINY_A) if s.optional_alias_of is None}
    assert "lm_head.weight" not in tied and len(tied) == 12 * 2 + 2


def test_random_weights_round_trip_and_precisions(tmp_path):
    cfg = config_from_dict(TINY_B)
    write_model_folder(tmp_path, cfg, seed=1)
    assert read_model_config(tmp_path) == cfg
    specs = specs_for(TINY_B)
    drawn = random_tensors(specs, 1)
    again = random_tensors(list(reversed(specs)), 1)                 # by name: the order does not matter
    other = random_tensors(specs, 2)
    for dtype in (torch.bfloat16, torch.float32):
        loaded = read_tensors(tmp_path, specs, dtype, "cpu")
        for s in specs:
            t = loaded[s.name]
            assert tuple(t.shape) == s.shape
            assert t.dtype == (dtype if s.role == "matrix" else torch.float32)       # vectors are held in 32-bit
            torch.testing.assert_close(t.float(), drawn[s.name].float(), atol=0, rtol=0)
            torch.testing.assert_close(drawn[s.name], again[s.name], atol=0, rtol=0)
    assert not torch.equal(drawn["model.norm.weight"], other["model.norm.weight"])
    w = drawn["model.layers.0.mlp.up_proj.weight"].float()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    n = drawn["model.layers.1.input_layernorm.weight"].float()
    assert abs(float(n.mean()) - 1.0) < 0.01                          # norm weights are 1 + N(0, 0.02)
    # a tensor stored in 32-bit keeps every bit when it is a vector
    write_model_folder(tmp_path / "f32", cfg, seed=1, store_dtype="float32")
    kept = read_tensors(tmp_path / "f32", specs, torch.bfloat16, "cpu")
    raw = random_tensors(specs, 1, store_dtype=torch.float32)
    torch.testing.assert_close(kept["model.norm.weight"], raw["model.norm.weight"], atol=0, rtol=0)
    assert kept["model.norm.weight"].dtype == torch.float32 and kept["lm_head.weight"].dtype == torch.bfloat16


def test_one_error_lists_everything_wrong(tmp_path):
    cfg = config_from_dict(TINY_B)
    specs = specs_for(TINY_B)
    tensors = random_tensors(specs, 0)
    del tensors["model.layers.1.mlp.down_proj.weight"], tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.o_proj.bias"] = torch.zeros(192)
    tensors["surprise.weight"] = torch.zeros(2)
    tensors["lm_head.weight"] = torch.zeros(389, 100, dtype=torch.bfloat16)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)       # skipped, as in the reference
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    save_file(tensors, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightError) as info:
        read_tensors(tmp_path, specs, torch.float32, "cpu")
    e = info.value
    assert e.missing == ["model.layers.1.mlp.down_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.o_proj.bias", "surprise.weight"]
    assert [w[0] for w in e.wrong_shape] == ["lm_head.weight"]
    text = str(e)
    for piece in ("model.norm.weight", "surprise.weight", "[389, 100]", "[389, 192]"):
        assert piece in text


def test_tied_head_sharded_index_and_unsafe_names(tmp_path):
    cfg = config_from_dict(TINY_A)
    specs = specs_for(TINY_A)
    tensors = random_tensors(specs, 0)
    names = sorted(tensors)
    a = {k: tensors[k] for k in names[:10]}
    b = {k: tensors[k] for k in names[10:]}
    b["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()      # present although tied: skipped
    save_file(a, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file(b, str(tmp_path / "model-00002-of-00002.safetensors"))
    index = {"weight_map": {**{k: "model-00001-of-00002.safetensors" for k in a},
                            **{k: "model-00002-of-00002.safetensors" for k in b}}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    loaded = read_tensors(tmp_path, specs, torch.float32, "cpu")
    assert sorted(loaded) == names
    # a tensor in two shards is a duplicate
    save_file({**b, names[0]: tensors[names[0]]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightError) as info:
        read_tensors(tmp_path, specs, torch.float32, "cpu")
    assert info.value.duplicate == [names[0]]
    # shard names cannot leave the folder
    for bad in ("../evil.safetensors", "sub/model.safetensors", "model.bin"):
        (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"x": bad}}))
        with pytest.raises(WeightError):
            read_tensors(tmp_path, specs, torch.float32, "cpu")
    # untied model without lm_head.weight: missing
    cfg_b, specs_b = config_from_dict(TINY_B), specs_for(TINY_B)
    tb = random_tensors(specs_b, 0)
    del tb["lm_head.weight"]
    folder = tmp_path / "untied"
    folder.mkdir()
    save_file(tb, str(folder / "model.safetensors"))
    with pytest.raises(WeightError) as info:
        read_tensors(folder, specs_b, torch.float32, "cpu")
    assert info.value.missing == ["lm_head.weight"]


def test_cache_bytes_per_token_vector_of_the_reference():
    """Qwen2.5-0.5B (24 layers, 2 key/value heads of 64): 24 KiB a token in 32-bit, 12 KiB in 16-bit
    (the reference's docs/ARCHITECTURE.md:64 and flow_engine/config.py:64-65), from the
    configuration class and from the cache layout of the model built for it."""
    from tessweave_engine_amd.config import build_model, config_from_dict
    cfg = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", num_hidden_layers=24, hidden_size=896,
               num_attention_heads=14, num_key_value_heads=2, intermediate_size=4864, vocab_size=151936,
               max_position_embeddings=32768)
    config = config_from_dict(cfg)
    assert config.head_dim == 64
    assert config.kv_bytes_per_token(4) == 24 * 1024 and config.kv_bytes_per_token(2) == 12 * 1024
    layout = build_model(config).cache_layout()
    assert layout.bytes_per_token(4) == 24 * 1024 and layout.bytes_per_token(2) == 12 * 1024
