"""Configuration and registry: every key read and checked, each refusal by name (method of
/root/reference/tests/arch_minimax_m3.cpp:140-193: remove each key in turn, match the refusal text)."""

import copy
import json

import pytest

from helpers import TINY_A, TINY_B
from llmx_amd import ConfigError, MiniMaxM3Config
from llmx_amd.models import architectures, read_config, assemble, register_architecture, unregister_architecture


def as_json(cfg_dict):
    return MiniMaxM3Config(**cfg_dict).to_json()


def test_round_trip_and_every_value():
    for tiny in (TINY_A, TINY_B):
        j = as_json(tiny)
        cfg = read_config(json.loads(json.dumps(j)))
        for key, value in tiny.items():
            assert getattr(cfg, key) == value, key
        assert cfg.q_width == tiny["num_attention_heads"] * tiny["head_dim"]
    assert "MiniMaxM3ForCausalLM" in architectures()


REQUIRED = ["vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads", "head_dim", "rms_norm_eps",
            "num_local_experts", "num_experts_per_tok", "intermediate_size", "routed_scaling_factor", "norm_topk_prob",
            "tie_word_embeddings", "max_position_embeddings"]


@pytest.mark.parametrize("key", REQUIRED)
def test_each_missing_key_is_refused_by_name(key):
    j = as_json(TINY_A)
    del j[key]
    with pytest.raises(ConfigError, match=f"missing key {key}"):
        read_config(j)


def test_rope_keys():
    j = as_json(TINY_A)
    del j["rope_parameters"]
    with pytest.raises(ConfigError, match="missing key rope_parameters.rope_theta"):
        read_config(j)
    j["rope_theta"] = 10000.0                       # the flat spelling is read too
    assert read_config(j).rope_theta == 10000.0
    j = as_json(TINY_A)
    del j["rotary_dim"]
    with pytest.raises(ConfigError, match="missing key rotary_dim"):
        read_config(j)
    j["rope_parameters"]["partial_rotary_factor"] = 0.5   # rotary width from the factor: 16 * 0.5
    assert read_config(j).rotary_dim == 8
    j["rotary_dim"] = 12                            # the two spellings must agree
    with pytest.raises(ConfigError, match="unsupported value for rotary_dim"):
        read_config(j)
    j = as_json(TINY_A)
    j["rope_parameters"]["rope_type"] = "yarn"
    with pytest.raises(ConfigError, match="unsupported value for rope_parameters.rope_type"):
        read_config(j)


@pytest.mark.parametrize("key,value", [("sliding_window", 128), ("hidden_act", "gelu"), ("scoring_func", "softmax"), ("swiglu_limit", 7.0),
                                       ("shared_intermediate_size", 32), ("rope_scaling", {"type": "yarn"}), ("use_qk_norm", False),
                                       ("attention_bias", True), ("n_group", 4)])
def test_options_computed_one_way_only_are_held(key, value):
    j = as_json(TINY_A)
    j[key] = value
    with pytest.raises(ConfigError, match=f"unsupported value for {key}"):
        read_config(j)


def test_unknown_key_is_refused_by_name_and_harmless_ones_pass():
    j = as_json(TINY_A)
    j["index_topk_blocks"] = 3
    with pytest.raises(ConfigError, match="key index_topk_blocks is not one this engine reads"):
        read_config(j)
    j = as_json(TINY_A)
    j.update(torch_dtype="bfloat16", transformers_version="5.0", num_mtp_modules=3, pad_token_id=0)
    read_config(j)


@pytest.mark.parametrize("change,text", [
    (dict(num_key_value_heads=3), "num_key_value_heads"), (dict(rotary_dim=7), "rotary_dim"), (dict(rotary_dim=18), "rotary_dim"),
    (dict(num_experts_per_tok=9), "num_experts_per_tok"), (dict(vocab_size=0), "vocab_size"), (dict(hidden_size=-4), "hidden_size"),
    (dict(rms_norm_eps=0.0), "rms_norm_eps"), (dict(norm_topk_prob="yes"), "norm_topk_prob"), (dict(head_dim=16.5), "head_dim"),
    (dict(eos_token_id=256), "eos_token_id")])
def test_values_out_of_range(change, text):
    j = as_json(TINY_A)
    j.update(change)
    with pytest.raises(ConfigError, match=f"unsupported value for {text}"):
        read_config(j)


def test_architecture_lookup():
    j = as_json(TINY_A)
    j["architectures"] = ["SomethingElseForCausalLM"]
    with pytest.raises(ConfigError, match="unsupported architecture 'SomethingElseForCausalLM'"):
        read_config(j)
    del j["architectures"]
    with pytest.raises(ConfigError, match="missing key architectures"):
        read_config(j)


def test_model_spec_is_data():
    """The configuration decides every size; the run order is a list that can name a layer twice or share a cache."""
    from llmx_amd.parts.spec import RunEntry
    spec = assemble(MiniMaxM3Config(**TINY_B))
    assert len(spec.blocks) == 3 and [e.layer for e in spec.run_order] == [0, 1, 2]
    b = spec.blocks[1]
    assert b.mixer.params["heads"] == 8 and b.mixer.params["kv_heads"] == 1 and b.mixer.params["head_dim"] == 24
    assert b.mixer.params["position"].params == {"rotary_dim": 24, "theta": 1e6, "head_dim": 24}
    assert b.ffn.params["experts"] == 16 and b.ffn.params["top_k"] == 4 and b.ffn.params["normalize"] is False and b.ffn.params["scale"] == 2.5
    assert b.mixer_norm.params["eps"] == 1e-5 and b.mixer.prefix == "model.layers.1.self_attn."
    spec.run_order = [RunEntry(0, 0), RunEntry(1, 1), RunEntry(1, 2), RunEntry(2, 1, writes=False)]
    spec.check()
    spec.run_order = [RunEntry(0, 0), RunEntry(1, 0)]
    with pytest.raises(ValueError, match="two entries write cache 0"):
        spec.check()
    spec.run_order = [RunEntry(0, 1, writes=False)]
    with pytest.raises(ValueError, match="before any entry writes"):
        spec.check()
    spec.run_order = [RunEntry(5, 0)]
    with pytest.raises(ValueError, match="names layer 5"):
        spec.check()
