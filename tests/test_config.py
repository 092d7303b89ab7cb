"""Configuration and registry (vectors re-expressed from crates/qwen3-spec/src/lib.rs:209-449 and
infer/src/model_registry.rs:271-467)."""
import json

import pytest

import arle_amd.models  # noqa: F401  registers Qwen3ForCausalLM
from arle_amd.config import ConfigError, Qwen3Config, detect_architecture, load_model_config
from arle_amd.config.base import read_stop_token_ids

BASE = dict(hidden_size=2048, intermediate_size=5632, num_hidden_layers=24, num_attention_heads=32,
            num_key_value_heads=8, head_dim=128, vocab_size=151936, rms_norm_eps=1e-6, rope_theta=1e6,
            tie_word_embeddings=True, max_position_embeddings=32768)


def test_parse_and_tied_head_name():
    c = Qwen3Config.from_dict(BASE)
    assert (c.hidden_size, c.num_key_value_heads, c.head_dim) == (2048, 8, 128)
    assert c.q_width == 4096 and c.kv_width == 1024  # q width is independent of hidden_size
    assert c.lm_head_tensor_name() == "model.embed_tokens.weight"
    assert Qwen3Config.from_dict(dict(BASE, tie_word_embeddings=False)).lm_head_tensor_name() == "lm_head.weight"


def test_aliases():
    raw = {k: v for k, v in BASE.items() if k not in ("num_key_value_heads", "max_position_embeddings")}
    raw.update(num_kv_heads=4, context_length=4096)
    c = Qwen3Config.from_dict(raw)
    assert c.num_key_value_heads == 4 and c.max_position_embeddings == 4096


def test_layer_tensor_names():
    n = Qwen3Config.layer_tensor_names(7)
    assert n["q_proj"] == "model.layers.7.self_attn.q_proj.weight"
    assert n["k_norm"] == "model.layers.7.self_attn.k_norm.weight"
    assert n["down_proj"] == "model.layers.7.mlp.down_proj.weight"
    assert n["post_attention_layernorm"] == "model.layers.7.post_attention_layernorm.weight"


@pytest.mark.parametrize("missing", sorted(BASE))
def test_every_key_is_required(missing):
    raw = {k: v for k, v in BASE.items() if k != missing}
    with pytest.raises(ConfigError, match=missing):
        Qwen3Config.from_dict(raw)


@pytest.mark.parametrize("patch,msg", [
    (dict(head_dim=127, num_attention_heads=6, num_key_value_heads=2), "even"),
    (dict(num_attention_heads=6, num_key_value_heads=4), "divisible"),
    (dict(num_key_value_heads=0), "non-zero"),
    (dict(max_position_embeddings=0), "max_position_embeddings"),
    (dict(hidden_size="big"), "hidden_size"),
    (dict(tie_word_embeddings=1), "tie_word_embeddings"),
    (dict(num_hidden_layers=10 ** 12), "num_hidden_layers"),      # a damaged file must not start a model of 10^12 layers
    (dict(vocab_size=2 ** 31), "vocab_size"),
    (dict(num_attention_heads=2 ** 26, num_key_value_heads=2 ** 26), "q_width"),
])
def test_invalid_configs(patch, msg):
    with pytest.raises(ConfigError, match=msg):
        Qwen3Config.from_dict(dict(BASE, **patch))


def test_round_trip_and_unknown_keys_ignored():
    c = Qwen3Config.from_dict(dict(BASE, some_future_key=[1, 2], rope_scaling=None))
    assert Qwen3Config.from_dict(c.to_dict()) == c


def test_registry():
    assert detect_architecture({"architectures": ["Other", "Qwen3ForCausalLM"]}).name == "Qwen3ForCausalLM"
    with pytest.raises(ConfigError, match="NoSuchModel"):
        detect_architecture({"architectures": ["NoSuchModel"]})
    with pytest.raises(ConfigError, match="no `architectures`"):
        detect_architecture({})


def test_model_folder_and_stop_ids(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(dict(BASE, architectures=["Qwen3ForCausalLM"],
                                                          eos_token_id=151645, bos_token_id=151643)))
    arch, config, stops = load_model_config(str(tmp_path))
    assert arch.name == "Qwen3ForCausalLM" and config.eos_token_id == 151645 and stops == (151645,)
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [151645, 151643]}))
    assert read_stop_token_ids(str(tmp_path), 151645) == (151645, 151643)
    assert read_stop_token_ids(str(tmp_path / "nowhere"), None) == ()
    with pytest.raises(ConfigError, match="failed to load config"):
        load_model_config(str(tmp_path / "nowhere"))
