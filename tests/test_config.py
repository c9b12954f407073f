"""Configuration and registry: keys, defaults and rejections as the reference's
reader has them (/root/reference/crates/nnis-model/src/safetensors_loader.rs:136-229,
tests :1024-1049; /root/reference/crates/nnis-model/src/config.rs:205-259)."""

import json

import pytest

import nnis_amd.models  # noqa: F401 (registers the architecture)
from configs import TINY_A, TINY_B, TINY_C
from nnis_amd.config import LlamaConfig, lookup_architecture, read_config_json, register_architecture, spec_from_config
from nnis_amd.errors import InvalidInput, Unsupported

SMOLLM2 = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 49152, "hidden_size": 576,
    "intermediate_size": 1536, "num_hidden_layers": 30, "num_attention_heads": 9, "num_key_value_heads": 3,
    "max_position_embeddings": 8192, "rms_norm_eps": 1e-5, "rope_theta": 100000, "hidden_act": "silu",
    "tie_word_embeddings": True, "torch_dtype": "bfloat16", "eos_token_id": 0, "bos_token_id": 0,
    "attention_bias": False, "rope_scaling": None, "rope_interleaved": False, "use_cache": True,
}


def test_smollm2_shape():
    cfg = LlamaConfig.from_dict(SMOLLM2)
    assert (cfg.head_dim, cfg.num_key_value_heads, cfg.eos_token_ids, cfg.torch_dtype) == (64, 3, (0,), "bfloat16")
    assert cfg.kv_width == 192 and cfg.q_width == 576 and cfg.group_size == 3
    assert cfg.attention_topology() == "GQA"
    assert LlamaConfig.from_dict(cfg.to_dict()) == cfg


def test_defaults_and_optional_keys():
    raw = dict(SMOLLM2)
    del raw["num_key_value_heads"], raw["tie_word_embeddings"], raw["eos_token_id"]
    cfg = LlamaConfig.from_dict(raw)
    assert cfg.num_key_value_heads == 9 and cfg.tie_word_embeddings is False and cfg.eos_token_ids == ()
    assert cfg.attention_topology() == "MHA"
    assert LlamaConfig.from_dict(TINY_B).attention_topology() == "MQA"
    c = LlamaConfig.from_dict(TINY_C)
    assert c.head_dim == 64 and c.q_width == 384 and c.eos_token_ids == (5, 9)


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "rms_norm_eps", "rope_theta", "torch_dtype", "hidden_act",
                                 "max_position_embeddings", "num_hidden_layers", "intermediate_size"])
def test_required_keys_are_named(key):
    raw = dict(SMOLLM2)
    del raw[key]
    with pytest.raises(InvalidInput, match=key):
        LlamaConfig.from_dict(raw)


@pytest.mark.parametrize("change, error", [
    ({"torch_dtype": "float16"}, Unsupported),
    ({"architectures": ["MistralForCausalLM"], "model_type": "mistral"}, Unsupported),
    ({"model_type": "mistral"}, Unsupported),
    ({"hidden_act": "gelu"}, Unsupported),
    ({"attention_bias": True}, Unsupported),
    ({"mlp_bias": True}, Unsupported),
    ({"rope_scaling": {"type": "linear", "factor": 2.0}}, Unsupported),
    ({"rope_interleaved": True}, Unsupported),
    ({"vocab_size": 0}, InvalidInput),
    ({"num_attention_heads": 7}, InvalidInput),
    ({"num_key_value_heads": 4}, InvalidInput),
    ({"head_dim": 33}, InvalidInput),
    ({"rms_norm_eps": 0.0}, InvalidInput),
    ({"rope_theta": float("inf")}, InvalidInput),
    ({"eos_token_id": 49152}, InvalidInput),
    ({"eos_token_id": "x"}, InvalidInput),
    ({"hidden_size": "576"}, InvalidInput),
])
def test_rejections(change, error):
    raw = dict(SMOLLM2)
    raw.update(change)
    with pytest.raises(error):
        LlamaConfig.from_dict(raw)


def test_registry_maps_name_to_model(tmp_path):
    assert lookup_architecture(TINY_A).name == "LlamaForCausalLM"
    cfg, spec = spec_from_config(TINY_A)
    assert spec.architecture == "LlamaForCausalLM" and len(spec.layers) == 2 and len(spec.schedule) == 2
    assert spec.layers[1]["mixer"]["kv_heads"] == 2 and spec.layers[0]["norm1"]["eps"] == 1e-5
    assert spec.head["tied_to"] == "model.embed_tokens.weight"
    assert spec_from_config(TINY_B)[1].head["tied_to"] is None
    with pytest.raises(Unsupported, match="NoSuchModel"):
        lookup_architecture({"architectures": ["NoSuchModel"], "model_type": "x"})
    with pytest.raises(InvalidInput):
        lookup_architecture({"architectures": []})
    with pytest.raises(InvalidInput):
        register_architecture("LlamaForCausalLM", LlamaConfig, lambda c: None)
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    assert read_config_json(str(tmp_path))["hidden_size"] == 64
    with pytest.raises(InvalidInput):
        read_config_json(str(tmp_path / "missing"))


def test_no_size_stands_in_code():
    """Two configurations that differ in every size give descriptions that
    differ in every size."""
    a, b = spec_from_config(TINY_A)[1], spec_from_config(TINY_B)[1]
    for key in ("width", "heads", "kv_heads", "head_dim"):
        assert a.layers[0]["mixer"][key] != b.layers[0]["mixer"][key]
    assert a.layers[0]["feed_forward"]["inner"] != b.layers[0]["feed_forward"]["inner"]
    assert a.layers[0]["norm1"]["eps"] != b.layers[0]["norm1"]["eps"]
    assert a.positions["rope"]["theta"] != b.positions["rope"]["theta"]
    assert a.vocab_size != b.vocab_size and a.max_positions != b.max_positions


def test_presets_and_the_capability_record():
    """The named shapes read back as configurations, and the two checkpoints
    the reference pins give its capability records letter for letter
    (/root/reference/crates/nnis-model/src/exact_checkpoint_spec.rs:10-30,219-259)."""
    from nnis_amd.config import preset, preset_names

    assert {"smollm2-135m", "smollm2-1.7b", "tinyllama-1.1b", "llama-8b", "tiny-a", "tiny-b"} <= set(preset_names())
    big = LlamaConfig.from_dict(preset("llama-8b"))
    assert (big.head_dim, big.num_attention_heads // big.num_key_value_heads) == (128, 4)
    small = LlamaConfig.from_dict(preset("smollm2-135m"))
    assert small.capability_record() == ("NNIS-DECODER-CAPABILITY-V1\nattention=grouped_query\nrope=llama_rotate_half_unscaled\n"
                                         "mlp=swiglu_silu\nweight_dtype=bf16\nq_heads=9\nkv_heads=3\nhead_dim=64\n")
    tiny = LlamaConfig.from_dict(preset("tinyllama-1.1b"))
    assert tiny.capability_record() == ("NNIS-DECODER-CAPABILITY-V1\nattention=grouped_query\nrope=llama_rotate_half_unscaled\n"
                                        "mlp=swiglu_silu\nweight_dtype=bf16\nq_heads=32\nkv_heads=4\nhead_dim=64\n")
    assert tiny.kv_width == 256 and tiny.eos_token_ids == (2,) and small.eos_token_ids == (0,)
    wide = LlamaConfig.from_dict(preset("smollm2-1.7b"))
    assert "attention=multi_head" in wide.capability_record()
    assert "attention=multi_query" in LlamaConfig.from_dict(preset("tiny-b")).capability_record()
    # the record a caller plans by: parameter counts of the published sizes, bytes of cache a token
    described = small.describe()
    assert described["parameters"] == 134_515_008 and described["weight_bytes"] == 2 * 134_515_008
    assert described["cache_bytes_per_token"] == {"bfloat16": 23_040, "float32": 46_080}
    assert described["attention"] == "GQA" and described["group_size"] == 3 and described["tied_head"]
    assert tiny.describe()["parameters"] == 1_100_048_384
    # overrides replace keys and leave the preset as it was
    assert preset("smollm2-135m", num_hidden_layers=2)["num_hidden_layers"] == 2
    assert preset("smollm2-135m")["num_hidden_layers"] == 30
    with pytest.raises(InvalidInput, match="unknown preset"):
        preset("llama-70b")
