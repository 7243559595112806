"""Configuration and registry (no GPU)."""

import copy

import pytest

from flyweight_amd.config import (ConfigError, Lfm2Config, ScheduleEntry, config_from_dict,
                                  register_architecture, registered_architectures)
from helpers import TINY_A, TINY_B


def test_reads_every_key_of_both_tiny_configurations():
    a, b = config_from_dict(TINY_A), config_from_dict(TINY_B)
    assert isinstance(a, Lfm2Config)
    assert (a.head_dim, a.ff_dim, a.full_attn_idxs, a.conv_bias, a.tie_word_embeddings) == (16, 160, (1, 3), False, True)
    assert (b.head_dim, b.ff_dim, b.full_attn_idxs, b.conv_bias, b.tie_word_embeddings) == (32, 384, (0, 4), True, False)
    assert (a.norm_eps, b.norm_eps, a.rope_theta, b.rope_theta) == (1e-5, 1e-6, 1e4, 1e6)
    assert (a.conv_L_cache, b.conv_L_cache) == (3, 4)


# the five (intermediate_size -> effective width) points the target shapes give
@pytest.mark.parametrize("inter,auto,mult,multiple,expected", [
    (12288, True, 1.0, 256, 8192), (6656, True, 1.0, 256, 4608), (10752, True, 1.0, 256, 7168),
    (384, True, 1.5, 64, 384), (160, False, None, None, 160)])
def test_feed_forward_width_rule(inter, auto, mult, multiple, expected):
    data = dict(TINY_A, intermediate_size=inter, block_auto_adjust_ff_dim=auto)
    if mult is not None:
        data.update(block_ffn_dim_multiplier=mult, block_multiple_of=multiple)
    assert config_from_dict(data).ff_dim == expected


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "num_key_value_heads", "intermediate_size", "max_position_embeddings"])
def test_missing_key_is_named(key):
    data = dict(TINY_A)
    del data[key]
    with pytest.raises(ConfigError, match=key):
        config_from_dict(data)


def test_documented_defaults_and_the_original_key_spellings():
    """Keys that may be absent get their documented defaults; the architecture's original
    spellings (block_ff_dim for the width, tie_embedding) are read as the generic ones are."""
    from flyweight_amd.config.lfm2 import DEFAULTS
    assert DEFAULTS == {"norm_eps": 1e-5, "rope_theta": 1000000.0, "conv_L_cache": 3}
    data = {k: v for k, v in TINY_B.items() if k not in ("norm_eps", "rope_theta", "conv_L_cache", "conv_bias",
                                                         "tie_word_embeddings", "block_auto_adjust_ff_dim")}
    config = config_from_dict(data)
    assert (config.norm_eps, config.rope_theta, config.conv_L_cache) == (1e-5, 1000000.0, 3)
    assert (config.conv_bias, config.tie_word_embeddings, config.block_auto_adjust_ff_dim) == (False, True, False)
    assert config.ff_dim == TINY_B["intermediate_size"]         # no adjustment unless asked for
    original = dict(TINY_B, block_ff_dim=TINY_B["intermediate_size"], tie_embedding=False)
    del original["intermediate_size"], original["tie_word_embeddings"]
    assert config_from_dict(original) == config_from_dict(TINY_B)
    assert config_from_dict(dict(TINY_B, block_ff_dim=TINY_B["intermediate_size"])) == config_from_dict(TINY_B)
    with pytest.raises(ConfigError, match="disagree"):
        config_from_dict(dict(TINY_B, block_ff_dim=TINY_B["intermediate_size"] + 64))
    with pytest.raises(ConfigError, match="block_ff_dim"):
        config_from_dict({k: v for k, v in TINY_B.items() if k != "intermediate_size"})


def test_layer_kinds_from_either_key_and_their_agreement():
    data = dict(TINY_A)
    del data["layer_types"]
    with pytest.raises(ConfigError, match="layer_types"):
        config_from_dict(data)
    data["full_attn_idxs"] = [1, 3]
    assert config_from_dict(data).layer_types == ("conv", "full_attention", "conv", "full_attention")
    both = dict(TINY_A, full_attn_idxs=[1, 3])
    assert config_from_dict(both).full_attn_idxs == (1, 3)
    with pytest.raises(ConfigError, match="disagree"):
        config_from_dict(dict(TINY_A, full_attn_idxs=[0, 3]))
    with pytest.raises(ConfigError, match="sliding"):
        config_from_dict(dict(TINY_A, layer_types=["conv", "sliding", "conv", "full_attention"]))
    with pytest.raises(ConfigError, match="num_hidden_layers"):
        config_from_dict(dict(TINY_A, layer_types=["conv", "full_attention"]))
    with pytest.raises(ConfigError, match="outside"):
        config_from_dict(dict(TINY_A, layer_types=None, full_attn_idxs=[7]))


@pytest.mark.parametrize("patch,match", [
    (dict(hidden_size=66), "multiple of num_attention_heads"),
    (dict(num_key_value_heads=3), "multiple of"),
    (dict(conv_L_cache=1), "conv_L_cache"),
    (dict(norm_eps=0.0), "norm_eps"),
    (dict(rope_theta=-1.0), "rope_theta"),
    (dict(vocab_size=0), "vocab_size"),
    (dict(hidden_size=20, num_attention_heads=4, num_key_value_heads=2), "even"),
    (dict(block_auto_adjust_ff_dim=True), "block_multiple_of"),
    (dict(conv_bias="yes"), "conv_bias"),
    (dict(tie_word_embeddings=True, tie_embedding=False), "disagree"),
])
def test_validation(patch, match):
    with pytest.raises(ConfigError, match=match):
        config_from_dict(dict(TINY_A, **patch))


def test_registry_refuses_unknown_names_and_lists_known_ones():
    with pytest.raises(ConfigError) as error:
        config_from_dict(dict(TINY_A, architectures=["NoSuchModel"], model_type="nosuch"))
    assert "NoSuchModel" in str(error.value) and "Lfm2ForCausalLM" in str(error.value)
    assert "Lfm2ForCausalLM" in registered_architectures() and "lfm2" in registered_architectures()
    # model_type alone is enough
    data = dict(TINY_A)
    del data["architectures"]
    assert isinstance(config_from_dict(data), Lfm2Config)
    class Other(Lfm2Config):
        pass
    with pytest.raises(ValueError, match="already registered"):
        register_architecture("Lfm2ForCausalLM", Other)
    with pytest.raises(TypeError):
        register_architecture("Other", dict)                    # not a configuration class


def test_model_spec_carries_every_size_as_a_parameter():
    spec = config_from_dict(TINY_B).model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["gqa_attention", "short_conv", "short_conv", "short_conv",
                                                           "gqa_attention", "short_conv"]
    attention = spec.layers[0].mixer
    assert (attention["num_heads"], attention["num_kv_heads"], attention["head_dim"]) == (3, 1, 32)
    assert attention["position"]["theta"] == 1e6 and attention["qk_norm_eps"] == 1e-6
    assert spec.layers[1].mixer["kernel_size"] == 4 and spec.layers[1].mixer["bias"] is True
    assert spec.layers[1].ffn["intermediate_size"] == 384
    assert spec.lm_head_name == "lm_head.weight" and config_from_dict(TINY_A).model_spec().lm_head_name is None
    assert [(e.layer, e.cache) for e in spec.schedule] == [(i, i) for i in range(6)]


def test_schedule_is_data_and_is_checked():
    import dataclasses
    spec = config_from_dict(TINY_A).model_spec()
    # a layer named twice, the second time reading the first's cache
    twice = dataclasses.replace(spec, schedule=spec.schedule + (ScheduleEntry(1, cache=1, writes_cache=False),))
    twice.validate()
    with pytest.raises(ConfigError, match="only one may write"):
        dataclasses.replace(spec, schedule=spec.schedule + (ScheduleEntry(1, cache=1),)).validate()
    with pytest.raises(ConfigError, match="before anything wrote"):
        dataclasses.replace(spec, schedule=(ScheduleEntry(1, cache=9, writes_cache=False),) + spec.schedule).validate()
    with pytest.raises(ConfigError, match="names layer"):
        dataclasses.replace(spec, schedule=(ScheduleEntry(11, cache=0),)).validate()


def test_round_trip_through_config_json(tmp_path):
    config = config_from_dict(TINY_B)
    config.save(str(tmp_path))
    from flyweight_amd.config import load_config
    assert load_config(str(tmp_path)) == config
    with pytest.raises(ConfigError, match="no config.json"):
        load_config(str(tmp_path / "nothing"))


# ----- the engine's own JSON reader -------------------------------------------------------------
def test_json_reader_values_and_what_it_refuses():
    import json
    from flyweight_amd.config import json_reader
    text = r'{"a": [1, -2, 3.5e2, true, false, null], "b": {"c": "x\n\u00e9\ud83d\ude00 \" \/"}, "n": 18446744073709551615, "f": 0.1}'
    assert json.loads(text)["b"]["c"] == 'x\n\u00e9\U0001f600 " /'
    value = json_reader.parse(text)
    assert value == json.loads(text)
    assert value["n"] == 2 ** 64 - 1 and isinstance(value["n"], int)       # offsets beyond 2^53 survive
    assert value["f"].literal == "0.1" and value["a"][2].literal == "3.5e2" and isinstance(value["a"][0], int)
    assert json_reader.parse(b"  [ ]  ") == [] and json_reader.parse("{}") == {}
    for bad, offset, what in (('{"a": 1} x', 9, "follows"), ('{"a": 1,}', 8, "key"), ("[1 2]", 3, "','"), ('{"a" 1}', 5, "':'"),
                              ('"abc', 0, "not closed"), ("01", 0, "leading zero"), ("[1.]", 1, "behind its point"),
                              ('{"a": 1, "a": 2}', 9, "twice"), ("tru", 0, "expected a value"), ("", 0, "ends here"),
                              ('"\\x"', 1, "escape"), ('"\\u+1a2"', 3, "four hexadecimal"), ('"\\u1_2a"', 3, "four hexadecimal"),
                              ('"\\u 1a2"', 3, "four hexadecimal"), ('"a\\ud800"', 2, "surrogate"), ('"\\udc00\\ud800"', 1, "surrogate"),
                              ('"\\ud83dx"', 1, "surrogate"), ("[" + "9" * 65 + "]", 1, "more than 64 digits")):
        with pytest.raises(json_reader.JsonError, match=what) as caught:
            json_reader.parse(bad)
        assert caught.value.offset == offset, (bad, caught.value.offset)
    assert json_reader.parse("-" + "9" * 64) == -int("9" * 64)
    deep = "[" * 64 + "]" * 64
    assert json_reader.parse(deep) is not None
    with pytest.raises(json_reader.JsonError, match="deeper than 64"):
        json_reader.parse("[" * 65 + "]" * 65)
    with pytest.raises(json_reader.JsonError, match="deeper"):
        json_reader.parse("[" * 100000)            # no recursion error, whatever the depth


def test_config_errors_carry_the_byte_offset(tmp_path):
    from flyweight_amd.config import load_config
    folder = tmp_path / "m"
    folder.mkdir()
    (folder / "config.json").write_text('{"architectures": ["Lfm2ForCausalLM"], "vocab_size": 12,, }')
    with pytest.raises(ConfigError, match="byte 56: expected a key"):
        load_config(str(folder))
