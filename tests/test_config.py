"""Configuration parsing and the architecture registry (CPU)."""

import json

import pytest

from tinyserve_llm_amd import models
from tinyserve_llm_amd.config import ConfigError, LlamaConfig
from tinyserve_llm_amd.models.registry import read_config, resolve

# Llama 3.2 1B's config.json values as the reference's own test lists them (tests/test_llama.py:114-136)
HUB_1B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": 2048, "intermediate_size": 8192,
    "num_hidden_layers": 16, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
    "vocab_size": 128256, "max_position_embeddings": 131072, "rms_norm_eps": 1e-05, "rope_theta": 500000.0,
    "rope_scaling": {"factor": 32.0, "high_freq_factor": 4.0, "low_freq_factor": 1.0,
                     "original_max_position_embeddings": 8192, "rope_type": "llama3"},
    "tie_word_embeddings": True, "torch_dtype": "bfloat16", "hidden_act": "silu", "attention_bias": False,
    "mlp_bias": False, "eos_token_id": [128001, 128008, 128009],
}


def test_hub_style_config():
    c = LlamaConfig.from_dict(HUB_1B)
    assert (c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == \
        (2048, 16, 32, 8, 64)
    assert c.rope_theta == 500000.0 and c.rope_scaling.factor == 32.0
    assert c.rope_scaling.original_max_position_embeddings == 8192
    assert c.tie_word_embeddings and c.eos_token_id == 128001, "the first of several end tokens"
    assert (c.q_size, c.kv_size, c.group_size) == (2048, 512, 4)


def test_rope_parameters_spelling_and_legacy_type_key():
    raw = {k: v for k, v in HUB_1B.items() if k not in ("rope_theta", "rope_scaling")}
    raw["rope_parameters"] = {"rope_type": "llama3", "rope_theta": 500000.0, **{
        k: v for k, v in HUB_1B["rope_scaling"].items() if k != "rope_type"}}
    assert LlamaConfig.from_dict(raw) == LlamaConfig.from_dict(HUB_1B)
    legacy = dict(HUB_1B, rope_scaling={**{k: v for k, v in HUB_1B["rope_scaling"].items() if k != "rope_type"},
                                        "type": "llama3"})
    assert LlamaConfig.from_dict(legacy) == LlamaConfig.from_dict(HUB_1B)


def test_defaults():
    raw = {"vocab_size": 100, "hidden_size": 48, "intermediate_size": 64, "num_hidden_layers": 1,
           "num_attention_heads": 3, "max_position_embeddings": 32, "rms_norm_eps": 1e-6}
    c = LlamaConfig.from_dict(raw)
    assert c.head_dim == 16 and c.num_key_value_heads == 3, "head_dim = hidden / heads; no grouping"
    assert c.rope_theta == 10000.0 and c.rope_scaling is None and not c.tie_word_embeddings and c.eos_token_id == -1
    c = LlamaConfig.from_dict(dict(raw, rope_scaling={"rope_type": "default"}, head_dim=None))
    assert c.rope_scaling is None and c.head_dim == 16
    c = LlamaConfig.from_dict(dict(raw, rope_scaling={"rope_type": "llama3", "factor": 2.0, "low_freq_factor": 1.0,
                                                      "high_freq_factor": 4.0}))
    assert c.rope_scaling.original_max_position_embeddings == 32, "defaults to the table length"


@pytest.mark.parametrize("change, match", [
    ({"hidden_act": "gelu"}, "hidden_act"), ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"), ({"num_key_value_heads": 5}, "multiple"), ({"head_dim": 7}, "even"),
    ({"vocab_size": None}, "vocab_size"), ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
])
def test_unusable_configs_name_the_key(change, match):
    with pytest.raises(ConfigError, match=match):
        LlamaConfig.from_dict(dict(HUB_1B, **change))


def test_other_rope_types_are_refused():
    with pytest.raises(NotImplementedError, match="yarn"):
        LlamaConfig.from_dict(dict(HUB_1B, rope_scaling={"rope_type": "yarn", "factor": 2.0}))


def test_round_trip_through_a_folder(tmp_path):
    c = LlamaConfig.from_dict(HUB_1B)
    c.save(str(tmp_path))
    arch, again = read_config(str(tmp_path))
    assert arch.name == "LlamaForCausalLM" and again == c
    raw = json.loads((tmp_path / "config.json").read_text())
    assert raw["rope_scaling"]["rope_type"] == "llama3" and raw["architectures"] == ["LlamaForCausalLM"]


def test_registry_resolves_by_architecture_then_model_type():
    assert resolve({"architectures": ["LlamaForCausalLM"]}).name == "LlamaForCausalLM"
    assert resolve({"model_type": "llama"}).name == "LlamaForCausalLM"
    assert resolve({"architectures": ["SomethingElse"], "model_type": "llama"}).name == "LlamaForCausalLM"
    with pytest.raises(NotImplementedError, match="is not supported; have"):
        resolve({"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3"})
    assert "LlamaForCausalLM" in models.ARCHITECTURES


def test_spec_holds_every_size_from_the_config():
    c = LlamaConfig.from_dict(HUB_1B)
    spec = models.ARCHITECTURES["LlamaForCausalLM"].build_spec(c)
    assert len(spec.layers) == 16 and [r.layer for r in spec.order] == list(range(16))
    att = spec.layers[0].mixer.args
    assert (att["num_heads"], att["num_kv_heads"], att["head_dim"], att["hidden_size"]) == (32, 8, 64, 2048)
    assert spec.layers[0].feed_forward.args["intermediate_size"] == 8192
    assert spec.final_norm.args == {"hidden_size": 2048, "eps": 1e-05}
    assert spec.position_encodings["rope"].args["scaling"]["factor"] == 32.0
    assert "lm_head.weight" not in spec.checkpoint and spec.optional == ("lm_head.weight",)
    d = spec.checkpoint["model.layers.3.self_attn.v_proj.weight"]
    assert (d.param, d.row, d.rows) == ("layers.3.mixer.qkv", 2048 + 512, 512)


def test_an_architecture_is_found_by_its_configurations_type_and_written_from_its_fields(tmp_path):
    """A configuration class needs `from_dict` only: the registry finds the architecture of a typed
    configuration by the class `config_from_dict` belongs to and writes config.json from the
    fields, adding the keys by which the folder is resolved again."""
    import json
    from dataclasses import dataclass

    from tinyserve_llm_amd.models import registry

    @dataclass(frozen=True)
    class Small:
        width: int
        depth: int = 2

        @classmethod
        def from_dict(cls, raw):
            return cls(int(raw["width"]), int(raw.get("depth", 2)))

    arch = registry.Architecture("SmallForCausalLM", ("small",), Small.from_dict, lambda c: None)
    assert arch.owns(Small(8)) and not arch.owns(object())
    assert arch.to_dict(Small(8, 3)) == dict(width=8, depth=3, architectures=["SmallForCausalLM"], model_type="small")
    registry.register_architecture(arch)
    try:
        assert registry.architecture_of(Small(8)) is arch
        registry.write_config(str(tmp_path), Small(8, 5))
        with open(tmp_path / "config.json") as f:
            assert json.load(f)["depth"] == 5
        found, config = registry.read_config(str(tmp_path))
        assert found is arch and config == Small(8, 5)
    finally:
        del registry.ARCHITECTURES["SmallForCausalLM"]
    import pytest as _pytest
    with _pytest.raises(NotImplementedError, match="Small"):
        registry.architecture_of(Small(8))
    # the Llama configuration goes out in the Hub's spelling, by its own writer
    from tests.helpers import TINY_B
    llama = registry.architecture_of(TINY_B)
    assert llama.name == "LlamaForCausalLM" and llama.to_dict(TINY_B)["rope_scaling"]["rope_type"] == "llama3"
    assert llama.config_from_dict(llama.to_dict(TINY_B)) == TINY_B
