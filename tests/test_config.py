"""Configuration and registry (CPU)."""
import json
import os

import pytest

from conftest import TINY_A, TINY_B, TINY_W
from pulse_infer_amd.config import (ConfigError, Qwen3Config, config_from_dict, load_config, lookup_architecture,
                                    register_architecture, registered_architectures, unregister_architecture)

# the keys the reference requires (src/model/qwen3/config.cpp:250-325), torch_dtype apart (a string, tested below)
REQUIRED = ["head_dim", "hidden_size", "intermediate_size", "max_position_embeddings", "num_attention_heads",
            "num_hidden_layers", "num_key_value_heads", "rms_norm_eps", "rope_theta", "tie_word_embeddings",
            "vocab_size"]


def test_reads_every_size_from_the_keys():
    a, b = Qwen3Config.from_dict(TINY_A), Qwen3Config.from_dict(TINY_B)
    for key in REQUIRED + ["num_key_value_heads", "tie_word_embeddings"]:
        assert getattr(a, key) == TINY_A[key] and getattr(b, key) == TINY_B[key]
        assert getattr(a, key) != getattr(b, key), f"the tiny configurations should differ in {key}"


@pytest.mark.parametrize("key", REQUIRED + ["torch_dtype"])
def test_missing_required_key_is_named(key):
    data = dict(TINY_A)
    del data[key]
    with pytest.raises(ConfigError, match=f"'{key}'"):
        Qwen3Config.from_dict(data, "cfg.json")


def test_wrong_type_is_named():
    with pytest.raises(ConfigError, match="'hidden_size'"):
        Qwen3Config.from_dict(dict(TINY_A, hidden_size="64"))
    with pytest.raises(ConfigError, match="'tie_word_embeddings'"):
        Qwen3Config.from_dict(dict(TINY_A, tie_word_embeddings=1))


def test_head_dim_is_free_of_hidden_size():
    cfg = Qwen3Config.from_dict(TINY_B)
    assert cfg.num_attention_heads * cfg.head_dim != cfg.hidden_size


def test_validation():
    with pytest.raises(ConfigError, match="shared out evenly"):
        Qwen3Config.from_dict(dict(TINY_A, num_attention_heads=5))
    with pytest.raises(ConfigError, match="sizes must be positive"):
        Qwen3Config.from_dict(dict(TINY_A, vocab_size=0))
    with pytest.raises(ConfigError, match="even"):
        Qwen3Config.from_dict(dict(TINY_A, head_dim=15))
    for key, value in (("attention_bias", True), ("hidden_act", "gelu"), ("rope_scaling", {"rope_type": "yarn"})):
        with pytest.raises(ConfigError, match=key):
            Qwen3Config.from_dict(dict(TINY_A, **{key: value}))
    # the reference attends to all keys whatever config.json says: window keys are refused, not interpreted
    with pytest.raises(ConfigError, match="use_sliding_window"):
        Qwen3Config.from_dict(dict(TINY_A, use_sliding_window=True, sliding_window=24, max_window_layers=1))
    with pytest.raises(ConfigError, match="layer_types"):
        Qwen3Config.from_dict(dict(TINY_A, layer_types=["full_attention", "sliding_attention"]))
    Qwen3Config.from_dict(dict(TINY_A, layer_types=["full_attention"] * 2, sliding_window=4096, max_window_layers=2))


def test_eos_int_or_list_and_generation_override(tmp_path):
    assert Qwen3Config.from_dict(dict(TINY_A, eos_token_id=7)).eos_token_ids == [7]
    assert Qwen3Config.from_dict(dict(TINY_A, eos_token_id=[7, 9])).eos_token_ids == [7, 9]
    assert Qwen3Config.from_dict(TINY_A).eos_token_ids == []
    with pytest.raises(ConfigError, match="eos_token_id"):
        Qwen3Config.from_dict(dict(TINY_A, eos_token_id="x"))
    (tmp_path / "config.json").write_text(json.dumps(dict(TINY_A, eos_token_id=3)))
    (tmp_path / "generation_config.json").write_text(json.dumps(
        {"eos_token_id": [5, 6], "temperature": 0.6, "top_k": 20, "top_p": 0.95}))
    cfg = load_config(str(tmp_path))
    assert cfg.eos_token_ids == [5, 6] and cfg.top_k == 20
    assert abs(cfg.temperature - 0.6) < 1e-12 and abs(cfg.top_p - 0.95) < 1e-12
    # a file path stands for its folder
    assert load_config(str(tmp_path / "config.json")).eos_token_ids == [5, 6]


def test_qwen3_0_6b_values(tmp_path):
    """The values the reference's config demo asserts (demo/qwen3_config_demo.cpp:73-86), as a fixture written here."""
    (tmp_path / "config.json").write_text(json.dumps(dict(
        architectures=["Qwen3ForCausalLM"], hidden_size=1024, intermediate_size=3072, num_hidden_layers=28,
        num_attention_heads=16, num_key_value_heads=8, head_dim=128, max_position_embeddings=40960,
        vocab_size=151936, rms_norm_eps=1e-6, rope_theta=1000000, tie_word_embeddings=True,
        torch_dtype="bfloat16", eos_token_id=151645, max_window_layers=28, sliding_window=None,
        use_sliding_window=False, rope_scaling=None)))
    (tmp_path / "generation_config.json").write_text(json.dumps(
        {"eos_token_id": [151645, 151643], "temperature": 0.6, "top_k": 20, "top_p": 0.95}))
    cfg = load_config(str(tmp_path))
    assert (cfg.hidden_size, cfg.intermediate_size, cfg.num_hidden_layers) == (1024, 3072, 28)
    assert (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == (16, 8, 128)
    assert (cfg.max_position_embeddings, cfg.vocab_size, cfg.torch_dtype) == (40960, 151936, "bfloat16")
    assert cfg.eos_token_ids == [151645, 151643] and cfg.top_k == 20
    assert all(cfg.layer_window(i) is None for i in range(28))


def test_windows_per_layer_are_an_option_of_the_engine():
    from conftest import OVERRIDES
    cfg = Qwen3Config.from_dict(TINY_W)
    assert all(cfg.layer_window(i) is None for i in range(4))
    cfg.apply_overrides(OVERRIDES["W"])
    assert [cfg.layer_window(i) for i in range(4)] == [None, None, 24, 24]
    assert [l.mixer.params["window"] for l in cfg.model_spec().layers] == [None, None, 24, 24]
    assert "layer_windows" not in cfg.to_dict()                   # no key of config.json
    cfg.apply_overrides({"layer_windows": [8, 0, None, 3]})
    assert [cfg.layer_window(i) for i in range(4)] == [8, None, None, 3]
    for bad in ([24], [None, None, -1, 24], [None, None, "24", 24], [None, None, True, 24]):
        with pytest.raises(ConfigError, match="layer_windows"):
            Qwen3Config.from_dict(TINY_W).apply_overrides({"layer_windows": bad})
    assert Qwen3Config.engine_options["layer_windows"]["type"]("0,0,24,24") == [None, None, 24, 24]


def test_model_spec_carries_no_size_of_its_own():
    for data in (TINY_A, TINY_B):
        cfg = Qwen3Config.from_dict(data)
        spec = cfg.model_spec()
        assert len(spec.layers) == data["num_hidden_layers"] and len(spec.order) == len(spec.layers)
        m = spec.layers[0].mixer.params
        assert (m["num_heads"], m["num_kv_heads"], m["head_dim"]) == (
            data["num_attention_heads"], data["num_key_value_heads"], data["head_dim"])
        assert m["scale"] == data["head_dim"] ** -0.5 and m["qk_norm_eps"] == data["rms_norm_eps"]
        assert spec.positions["rope"].params["theta"] == data["rope_theta"]
        assert spec.layers[0].ffn.params["intermediate_size"] == data["intermediate_size"]
        assert spec.head.params["tied"] == data["tie_word_embeddings"]


def test_round_trip_through_to_dict():
    cfg = Qwen3Config.from_dict(dict(TINY_W, eos_token_id=[1, 2]))
    again = Qwen3Config.from_dict(cfg.to_dict())
    assert again == cfg


def test_registry(tmp_path):
    assert "Qwen3ForCausalLM" in registered_architectures()
    assert lookup_architecture("Qwen3ForCausalLM").config_class is Qwen3Config
    with pytest.raises(ConfigError, match="unknown architecture 'NopeForCausalLM'.*Qwen3ForCausalLM"):
        config_from_dict(dict(TINY_A, architectures=["NopeForCausalLM"]))
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict({k: v for k, v in TINY_A.items() if k != "architectures"})
    with pytest.raises(ValueError, match="already registered"):
        register_architecture("Qwen3ForCausalLM", Qwen3Config)

    class Other(Qwen3Config):
        pass

    register_architecture("OtherForCausalLM", Other)
    try:
        (tmp_path / "config.json").write_text(json.dumps(dict(TINY_A, architectures=["OtherForCausalLM"])))
        assert isinstance(load_config(str(tmp_path)), Other)
    finally:
        unregister_architecture("OtherForCausalLM")
    with pytest.raises(ConfigError, match="there is no file"):
        load_config(str(tmp_path / "nowhere"))


def test_rope_pairing_is_an_option_of_the_engine():
    from pulse_infer_amd.config import ConfigError, Qwen3Config
    from conftest import TINY_A

    cfg = Qwen3Config.from_dict(TINY_A)
    assert cfg.rope_pairing == "interleaved"   # what the reference computes (rope_kernel.cu:100-126)
    assert cfg.model_spec().positions["rope"].params["pairing"] == "interleaved"
    cfg.rope_pairing = "half"
    cfg.validate()
    assert cfg.model_spec().positions["rope"].params["pairing"] == "half"
    assert "rope_pairing" not in cfg.to_dict()
    cfg.rope_pairing = "pairs"
    with pytest.raises(ConfigError):
        cfg.validate()


def test_config_json_may_hold_comments(tmp_path):
    """The reference parses config.json with comments allowed (src/model/qwen3/config.cpp:52)."""
    text = json.dumps(TINY_B, indent=1)
    text = text.replace('"hidden_size"', '// the width\n "hidden_size"', 1)
    text = text.replace('"vocab_size"', '/* tokens:\n   all of them */ "vocab_size"', 1)
    text = text.replace('"qwen3",', '"qwen3", // not "/*" a comment inside', 1)
    (tmp_path / "config.json").write_text(text)
    cfg = load_config(str(tmp_path))
    assert cfg.hidden_size == TINY_B["hidden_size"] and cfg.vocab_size == TINY_B["vocab_size"]
    (tmp_path / "config.json").write_text('{"a": "x // y", /* c */ "b": 1} trailing')
    with pytest.raises(ConfigError, match="not valid JSON"):
        load_config(str(tmp_path))
