"""Configuration reading, the architecture registry and engine options (no GPU)."""
import json

import pytest

from dinfer_amd.config import ConfigError, EngineOptions, get_architecture, known_architectures, load_config
from dinfer_amd.config.qwen3 import Qwen3Config
from tiny_configs import CONFIGS

BASE = CONFIGS["B"][0]


def test_reads_every_key_and_ignores_unknown_ones():
    c = Qwen3Config.from_dict({**BASE, "torch_dtype": "bfloat16", "bos_token_id": 1, "something_new": [1, 2]})
    assert (c.vocab_size, c.hidden_size, c.intermediate_size, c.num_hidden_layers) == (512, 96, 224, 3)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (8, 2, 32)
    assert c.rms_norm_eps == 1e-5 and c.rope_theta == 1e6 and c.max_position_embeddings == 256
    assert c.tie_word_embeddings is False and c.eos_token_ids == (3, 5)
    # derived sizes as the reference computes them (config.rs:66-77); head_dim is not hidden / heads
    assert (c.q_size, c.kv_size, c.group_size) == (256, 64, 4)


def test_defaults():
    d = {k: v for k, v in BASE.items() if k not in ("tie_word_embeddings", "attention_bias", "hidden_act", "eos_token_id")}
    c = Qwen3Config.from_dict(d)
    assert c.tie_word_embeddings is False and c.attention_bias is False and c.hidden_act == "silu"
    assert c.use_sliding_window is False and c.sliding_window is None and c.eos_token_ids == ()


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "num_key_value_heads", "head_dim", "rms_norm_eps",
                                 "rope_theta", "max_position_embeddings"])
def test_required_keys_are_named_when_missing(key):
    d = dict(BASE)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(d)


@pytest.mark.parametrize("patch,needle", [
    ({"hidden_act": "gelu"}, "gelu"), ({"attention_bias": True}, "attention_bias"),
    ({"num_attention_heads": 7}, "7"), ({"head_dim": 33}, "33"), ({"vocab_size": 0}, "vocab_size"),
    ({"rope_scaling": {"type": "yarn", "factor": 4.0}}, "rope_scaling"), ({"hidden_size": "96"}, "hidden_size"),
    ({"rms_norm_eps": True}, "rms_norm_eps"), ({"eos_token_id": "2"}, "eos_token_id"),
    ({"use_sliding_window": True}, "sliding_window"),
    ({"use_sliding_window": True, "sliding_window": 8}, "max_window_layers"),
    ({"use_sliding_window": True, "sliding_window": 8, "max_window_layers": 9}, "max_window_layers"),
])
def test_rejections_name_the_offender(patch, needle):
    with pytest.raises(ConfigError, match=needle):
        Qwen3Config.from_dict({**BASE, **patch})


def test_eos_number_or_list_and_null_rope_scaling():
    assert Qwen3Config.from_dict({**BASE, "eos_token_id": 151645}).eos_token_ids == (151645,)
    assert Qwen3Config.from_dict({**BASE, "eos_token_id": [1, 2]}).eos_token_ids == (1, 2)
    assert Qwen3Config.from_dict({**BASE, "rope_scaling": None}).rope_scaling_present is False


def test_window_layers():
    c = Qwen3Config.from_dict(CONFIGS["C"][0])
    assert [c.layer_window(i) for i in range(5)] == [None, None, 24, 24, 24]
    assert Qwen3Config.from_dict(BASE).layer_window(2) is None


def test_layer_types_must_say_what_the_window_keys_say():
    """Newer config.json files list each layer's kind; the list is read and a file whose list and keys disagree is refused."""
    win = CONFIGS["C"][0]                                   # 5 layers, the window from layer 2 on
    ok = ["full_attention"] * 2 + ["sliding_attention"] * 3
    assert Qwen3Config.from_dict({**win, "layer_types": ok}).layer_types == tuple(ok)
    assert Qwen3Config.from_dict({**BASE, "layer_types": ["full_attention"] * BASE["num_hidden_layers"]}).layer_window(0) is None
    for bad, needle in ((["full_attention"] * 5, "layer 2"), (ok[:4], "lists 4"), (ok[:4] + ["chunked"], "chunked"),
                        ("full_attention", "layer_types")):
        with pytest.raises(ConfigError, match=needle):
            Qwen3Config.from_dict({**win, "layer_types": bad})
    with pytest.raises(ConfigError, match="layer 0"):       # a list that asks for windows the keys switch off
        Qwen3Config.from_dict({**BASE, "layer_types": ["sliding_attention"] * BASE["num_hidden_layers"]})


def test_round_trip_through_config_json(tmp_path):
    for name, (cfg, _) in CONFIGS.items():
        c = Qwen3Config.from_dict(cfg)
        (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
        arch, c2 = load_config(tmp_path)
        assert arch.name == "Qwen3ForCausalLM" and c2 == c


def test_registry():
    assert "Qwen3ForCausalLM" in known_architectures()
    assert get_architecture("Qwen3ForCausalLM").config_class is Qwen3Config
    with pytest.raises(ConfigError, match="Qwen3ForCausalLM"):  # the error lists what is known
        get_architecture("LlamaForCausalLM")


def test_load_config_errors(tmp_path):
    with pytest.raises(ConfigError, match="does not exist"):
        load_config(tmp_path)
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        load_config(tmp_path)
    (tmp_path / "config.json").write_text(json.dumps({k: v for k, v in BASE.items() if k != "architectures"}))
    with pytest.raises(ConfigError, match="architectures"):
        load_config(tmp_path)


def test_spec_follows_the_configuration_layer_by_layer():
    """Every size of the model spec comes from the configuration; the window makes two kinds of layers."""
    arch = get_architecture("Qwen3ForCausalLM")
    for name, (cfg, _) in CONFIGS.items():
        c = Qwen3Config.from_dict(cfg)
        spec = arch.build_spec(c)
        assert len(spec.layers) == c.num_hidden_layers == len(spec.run)
        assert spec.vocab_size == c.vocab_size and spec.tie_embeddings == c.tie_word_embeddings
        for i, l in enumerate(spec.layers):
            p = l.mixer.params
            assert (p["heads"], p["kv_heads"], p["head_dim"]) == (c.num_attention_heads, c.num_key_value_heads, c.head_dim)
            assert p["window"] == c.layer_window(i) and p["position"].params["theta"] == c.rope_theta
            assert l.norm.params["eps"] == c.rms_norm_eps and l.feed_forward.params["intermediate"] == c.intermediate_size
            assert l.prefix == f"model.layers.{i}."


def test_engine_options_check():
    EngineOptions().check()
    for bad in (dict(dtype="float16"), dict(block_size=0), dict(num_blocks=0), dict(gpu_memory_utilization=1.5),
                dict(max_num_seqs=-1)):
        with pytest.raises(ValueError):
            EngineOptions(**bad).check()
