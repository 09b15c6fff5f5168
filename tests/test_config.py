"""Configuration: required keys, defaults, checks, registry (no GPU)."""
import copy
import json

import pytest

from rbitnet_amd.config import LlamaConfig, load_config, registered_architectures
from rbitnet_amd.errors import ConfigError

from helpers import TINY_A, TINY_B


def test_defaults_follow_the_reference():
    # config.rs:56 (kv heads = heads), :94-97 (theta 1e4), :99-102 (eps 1e-5), :104-107 (context 2048)
    cfg = LlamaConfig.from_dict({"hidden_size": 64, "num_hidden_layers": 1, "num_attention_heads": 4,
                                 "intermediate_size": 100, "vocab_size": 50})
    assert cfg.num_key_value_heads == 4 and cfg.head_dim == 16
    assert cfg.rope_theta == 10000.0 and cfg.rms_norm_eps == 1e-5 and cfg.max_position_embeddings == 2048
    assert cfg.rope_scaling is None and not cfg.tie_word_embeddings
    # the pairing of the rotation: not said -> "half", the layout of weights stored under a
    # config.json's own names; GGUF spellings in the weight file -> the reference's adjacent pairs
    assert cfg.rope_style is None and cfg.effective_rope_style == "half"
    assert cfg.to_spec().layers[0].mixer["position"]["style"] == "half"
    hf = cfg.with_tensor_names(["model.layers.0.self_attn.q_proj.weight", "model.embed_tokens.weight"])
    assert hf.effective_rope_style == "half"
    gguf = cfg.with_tensor_names(["blk.0.attn_q.weight", "token_embd.weight"])
    assert gguf.effective_rope_style == "interleaved" and "rope_style" in gguf.to_dict()
    said = LlamaConfig.from_dict({"hidden_size": 64, "num_hidden_layers": 1, "num_attention_heads": 4,
                                  "intermediate_size": 100, "vocab_size": 50, "rope_style": "half"})
    assert said.with_tensor_names(["blk.0.attn_q.weight"]).effective_rope_style == "half"      # the key wins
    assert "rope_style" not in cfg.to_dict()


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads", "intermediate_size",
                                 "vocab_size"])
def test_missing_required_key_is_named(key):
    d = copy.deepcopy(TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=f"missing {key}"):
        LlamaConfig.from_dict(d)


def test_gguf_spellings_are_accepted():
    cfg = LlamaConfig.from_dict({"llama.embedding_length": 64, "llama.block_count": 2, "llama.attention.head_count": 4,
                                 "llama.attention.head_count_kv": 2, "llama.feed_forward_length": 172,
                                 "llama.vocab_size": 256, "llama.rope.freq_base": 5000.0,
                                 "llama.attention.layer_norm_rms_epsilon": 1e-6, "llama.context_length": 99})
    assert (cfg.hidden_size, cfg.num_key_value_heads, cfg.rope_theta, cfg.rms_norm_eps,
            cfg.max_position_embeddings) == (64, 2, 5000.0, 1e-6, 99)


@pytest.mark.parametrize("patch,msg", [
    ({"num_key_value_heads": 3}, "num_attention_heads / num_key_value_heads"),      # config.rs:57-61
    ({"num_key_value_heads": 0}, "num_attention_heads / num_key_value_heads"),
    ({"hidden_size": 66}, "not divisible"),                                          # config.rs:62-67
    ({"hidden_size": 60, "num_attention_heads": 4, "num_key_value_heads": 4}, "head_dim"),   # 15 is odd, :68-72
    ({"head_dim": 7}, "head_dim"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"rope_style": "spiral"}, "rope_style"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "rope_type"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 4.0, "high_freq_factor": 1.0,
                       "original_max_position_embeddings": 32}}, "high_freq_factor"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0}}, "low_freq_factor"),
    ({"vocab_size": 2.5}, "vocab_size"),
    ({"vocab_size": -3}, "vocab_size"),
    ({"rope_theta": "big"}, "rope_theta"),
])
def test_invalid_values(patch, msg):
    d = copy.deepcopy(TINY_A)
    d.update(patch)
    with pytest.raises(ConfigError, match=msg):
        LlamaConfig.from_dict(d)


def test_integral_floats_and_eos_lists():
    d = copy.deepcopy(TINY_B)
    d["vocab_size"] = 384.0
    d["eos_token_id"] = [7, 9]
    cfg = LlamaConfig.from_dict(d)
    assert cfg.vocab_size == 384 and cfg.eos_token_ids == [7, 9]
    assert cfg.rope_scaling.factor == 8.0 and cfg.rope_scaling.original_max_position_embeddings == 32


def test_registry_and_spec():
    assert "LlamaForCausalLM" in registered_architectures()
    cfg, spec = load_config(TINY_B)
    assert isinstance(cfg, LlamaConfig)
    assert spec.head_name is None and spec.stop_token_ids == [7]          # tied, EOS
    assert len(spec.layers) == 3 and spec.schedule == [0, 1, 2]
    m = spec.layers[1].mixer
    assert m.kind == "attention" and m["num_kv_heads"] == 1 and m["head_dim"] == 24
    assert m["position"].kind == "rope" and m["position"]["scaling"]["factor"] == 8.0
    assert spec.layers[0].norm1["eps"] == 1e-6 and spec.layers[0].feed_forward["intermediate_size"] == 256
    d = copy.deepcopy(TINY_A)
    d["architectures"] = ["MambaForCausalLM"]
    with pytest.raises(ConfigError, match="unknown architecture.*LlamaForCausalLM"):
        load_config(d)
    with pytest.raises(ConfigError, match="names no architecture"):
        load_config({"hidden_size": 8})


def test_round_trip_through_to_dict():
    cfg, _ = load_config(TINY_B)
    again = LlamaConfig.from_dict(json.loads(json.dumps(cfg.to_dict())))
    assert again == cfg


def test_no_size_is_a_constant_in_the_spec():
    """Every size in the spec comes from the configuration: change each and see it move."""
    base = load_config(TINY_A)[1]
    for key, probe in [("hidden_size", lambda s: s.hidden_size), ("vocab_size", lambda s: s.vocab_size),
                       ("intermediate_size", lambda s: s.layers[0].feed_forward["intermediate_size"]),
                       ("rms_norm_eps", lambda s: s.final_norm["eps"]),
                       ("rope_theta", lambda s: s.layers[0].mixer["position"]["theta"]),
                       ("max_position_embeddings", lambda s: s.max_positions)]:
        d = copy.deepcopy(TINY_A)
        d[key] = d[key] * 2
        assert probe(load_config(d)[1]) == 2 * probe(base), key
