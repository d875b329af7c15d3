"""Configuration and registry: keys, defaults and refusals."""
import copy
import math

import pytest

import tiny_configs as tc
from fllm_amd.config import ConfigError, LlamaConfig
from fllm_amd.registry import model_spec_from_config, resolve_architecture, supported_model_types


def test_llama_is_registered():
    assert "llama" in supported_model_types()
    assert resolve_architecture(tc.TINY_A).model_type == "llama"


def test_sizes_come_from_config_keys():
    c = LlamaConfig.from_dict(tc.TINY_B)
    assert (c.hidden_size, c.num_layers, c.num_heads, c.num_kv_heads, c.head_dim) == (160, 3, 5, 1, 32)
    assert (c.intermediate_size, c.vocab_size, c.max_position) == (432, 512, 256)
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0 and c.tie_word_embeddings
    s = c.rope_scaling
    assert (s.kind, s.factor, s.low_freq_factor, s.high_freq_factor, s.original_max_position) == ("llama3", 8.0, 1.0, 4.0, 64)


def test_defaults_follow_the_reference():
    """plan.rs:1078-1082 (kv heads, context), :1096 (head_dim), :1222-1236 (eps), :1325-1338 (theta),
    convert.rs:321-324 (tied)."""
    c = LlamaConfig.from_dict({"model_type": "llama", "hidden_size": 64, "num_attention_heads": 4,
                               "num_hidden_layers": 2, "intermediate_size": 128})
    assert c.num_kv_heads == 4 and c.head_dim == 16 and c.rms_norm_eps == 1e-6 and c.rope_theta == 10000.0
    assert c.max_position == 40960 and c.vocab_size == 32000 and not c.tie_word_embeddings
    assert c.rope_scaling.kind == "none" and c.layer_windows == (None, None)


def test_round_trip():
    for cfg in tc.CONFIGS.values():
        c = LlamaConfig.from_dict(cfg)
        assert LlamaConfig.from_dict(c.to_dict()) == c


def test_rope_parameters_form():
    cfg = copy.deepcopy(tc.TINY_B)
    scaling = cfg.pop("rope_scaling")
    theta = cfg.pop("rope_theta")
    cfg["rope_parameters"] = dict(scaling, rope_theta=theta)
    assert LlamaConfig.from_dict(cfg) == LlamaConfig.from_dict(tc.TINY_B)
    cfg["rope_parameters"] = {"full_attention": dict(scaling, rope_theta=theta)}
    assert LlamaConfig.from_dict(cfg) == LlamaConfig.from_dict(tc.TINY_B)


def test_yarn_longrope_and_dynamic_keys():
    """plan.rs:1433-1477, :1507-1548, :1339-1343."""
    f = LlamaConfig.from_dict(tc.TINY_F).rope_scaling
    assert (f.kind, f.factor, f.original_max_position, f.beta_fast, f.beta_slow) == ("yarn", 4.0, 64, 16.0, 2.0)
    assert f.extrapolation == 1.0 and f.truncate and f.attention is None
    cfg = copy.deepcopy(tc.TINY_F)
    cfg["rope_scaling"].update(mscale=1.0, mscale_all_dim=0.5, truncate=False, extrapolation_factor=0.5)
    del cfg["rope_scaling"]["original_max_position_embeddings"]
    cfg["original_max_position_embeddings"] = 32                       # the model's own key stands in
    y = LlamaConfig.from_dict(cfg).rope_scaling
    assert y.original_max_position == 32 and not y.truncate and y.extrapolation == 0.5
    assert abs(y.attention - (1 + 0.1 * math.log(4.0)) / (1 + 0.05 * math.log(4.0))) < 1e-12
    cfg["rope_scaling"]["attention_factor"] = 1.5                      # goes before the pair
    assert LlamaConfig.from_dict(cfg).rope_scaling.attention == 1.5
    g = LlamaConfig.from_dict(tc.TINY_G)
    assert g.rope_dims == 24 and g.rope_scaling.kind == "longrope" and len(g.rope_scaling.long_factor) == 12
    assert abs(g.rope_scaling.attention - math.sqrt(1 + math.log(160 / 48) / math.log(48))) < 1e-12
    cfg = copy.deepcopy(tc.TINY_G)
    del cfg["rope_scaling"]["original_max_position_embeddings"]        # then the model's context is the original one
    s = LlamaConfig.from_dict(cfg).rope_scaling
    assert s.original_max_position == 160 and s.attention == 1.0
    cfg = dict(tc.TINY_A, rope_scaling={"rope_type": "dynamic", "alpha": 4.0})
    d = LlamaConfig.from_dict(cfg)
    assert d.rope_scaling.kind == "none" and abs(d.rope_theta - 10000.0 * 4.0 ** (16 / 14)) < 1e-6


def test_windows():
    c = LlamaConfig.from_dict(tc.TINY_C)
    assert c.layer_windows == (24, None, 24, None) and c.rope_dims == 24
    cfg = dict(tc.TINY_C)
    del cfg["layer_types"]
    assert LlamaConfig.from_dict(cfg).layer_windows == (24, 24, 24, 24)
    cfg["use_sliding_window"] = False
    assert LlamaConfig.from_dict(cfg).layer_windows == (None,) * 4


@pytest.mark.parametrize("change,text", [
    ({"model_type": None}, "requires model_type"),
    ({"model_type": "gpt2"}, "unsupported model_type"),
    ({"architectures": ["MistralForCausalLM"]}, "does not match architectures"),
    ({"hidden_size": None}, "requires valid hidden_size"),
    ({"num_attention_heads": "4"}, "requires valid num_attention_heads"),
    ({"num_hidden_layers": None}, "requires valid num_hidden_layers"),
    ({"intermediate_size": -3}, "requires valid intermediate_size"),
    ({"num_key_value_heads": 3}, "not a multiple"),
    ({"head_dim": None, "hidden_size": 66}, "invalid or inconsistent model dimensions"),
    ({"num_hidden_layers": 0}, "invalid or inconsistent model dimensions"),
    ({"hidden_act": "gelu"}, "unsupported activation"),
    ({"rms_norm_eps": float("inf")}, "invalid rms_norm_eps"),
    ({"rms_norm_eps": 0.0}, "invalid rms_norm_eps"),
    ({"rope_scaling": {"rope_type": "llama3", "original_max_position_embeddings": 64}}, "requires factor"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0}}, "requires original_max_position_embeddings"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 8.0}}, "yarn rope_scaling requires original_max_position_embeddings"),
    ({"rope_scaling": {"rope_type": "yarn", "original_max_position_embeddings": 64}}, "yarn rope_scaling requires factor"),
    ({"rope_scaling": {"rope_type": "longrope", "long_factor": [1.0] * 8}}, "longrope scaling requires short_factor"),
    ({"rope_scaling": {"rope_type": "su", "short_factor": [1.0] * 8, "long_factor": [1.0] * 7}}, "longrope factors must have 8 entries"),
    ({"rope_scaling": {"rope_type": "dynamic", "factor": 2.0}}, 'unsupported rope scaling type "dynamic"'),
    ({"rope_scaling": {"rope_type": "proportional", "factor": 2.0}}, "unsupported rope_scaling type"),
    ({"rope_scaling": {"type": "linear"}}, "linear rope_scaling requires factor"),
    ({"head_dim": 15}, "even head and rotary dimensions"),
    ({"quantization_config": {"bits": 4}}, "quantized"),
])
def test_refusals(change, text):
    cfg = dict(tc.TINY_A)
    for k, v in change.items():
        if v is None:
            cfg.pop(k, None)
        else:
            cfg[k] = v
    with pytest.raises(ConfigError, match=text):
        model_spec_from_config(cfg)


def test_spec_describes_every_layer():
    _, spec = model_spec_from_config(tc.TINY_C)
    assert len(spec.layers) == 4 and [e.layer for e in spec.run_order] == [0, 1, 2, 3]
    assert [l.mixer["window"] for l in spec.layers] == [24, None, 24, None]
    m = spec.layers[0].mixer
    assert (m["num_heads"], m["num_kv_heads"], m["head_dim"]) == (6, 3, 48)
    assert m["position"]["dims"] == 24 and m["position"]["scaling"] == "linear"
    assert spec.head.tensors["weight"] == "lm_head.weight"
    _, tied = model_spec_from_config(tc.TINY_B)
    assert tied.head.tensors["weight"] == "model.embed_tokens.weight"


def test_generation_defaults_of_a_model_folder(tmp_path):
    """rust/engine/src/server/gencfg.rs:93-135, and its test at :165-190: the five sampling keys count whether or not
    do_sample is set; values no sampler can use are dropped; `vllm` means none; a file named outright must be there."""
    import json
    from fllm_amd.config.files import generation_defaults, generation_eos_ids
    folder = tmp_path / "model"
    folder.mkdir()
    assert generation_defaults("auto", str(folder)) == ({}, "none in the model")
    (folder / "generation_config.json").write_text(json.dumps(
        {"do_sample": False, "temperature": 0.6000004, "top_p": 0.9, "top_k": 0, "min_p": 1.5, "repetition_penalty": 1.1,
         "eos_token_id": [128001, 128008, 128009], "max_length": 20}))
    got, origin = generation_defaults("auto", str(folder))
    assert got == {"temperature": 0.6, "top_p": 0.9, "top_k": 0, "repetition_penalty": 1.1} and origin.endswith("generation_config.json")
    assert generation_defaults("vllm", str(folder))[0] == {}
    assert generation_defaults(str(folder), None)[0] == got and generation_defaults(str(folder / "generation_config.json"), None)[0] == got
    assert generation_eos_ids(str(folder)) == (128001, 128008, 128009)
    with pytest.raises(ConfigError, match="cannot read generation defaults"):
        generation_defaults(str(tmp_path / "nothing.json"), None)
    (folder / "generation_config.json").write_text("{ not json")
    assert generation_defaults("auto", str(folder)) == ({}, "none in the model") and generation_eos_ids(str(folder)) == ()
    with pytest.raises(ConfigError, match="cannot read generation defaults"):
        generation_defaults(str(folder), None)
    (folder / "generation_config.json").write_text(json.dumps({"temperature": float("nan"), "top_k": -1, "top_p": True, "eos_token_id": 2}))
    assert generation_defaults("auto", str(folder))[0] == {} and generation_eos_ids(str(folder)) == (2,)
