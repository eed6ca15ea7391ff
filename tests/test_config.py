"""Configuration: typed reading of config.json keys, geometry refusals, the registry."""
import copy
import json

import pytest

from tiny import TINY_A, TINY_B, TINY_C
from xyntetik_runner_amd.config import (ConfigError, LlamaConfig, config_from_dict, get_architecture,
                                        known_architectures, load_config, register_architecture,
                                        unregister_architecture)


def test_reads_every_key_of_tiny_configs():
    a = LlamaConfig.from_dict(TINY_A)
    assert (a.num_hidden_layers, a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim,
            a.intermediate_size, a.vocab_size) == (2, 64, 4, 2, 16, 176, 256)
    assert a.rope_scaling is None and a.rms_norm_eps == 1e-5 and not a.tie_word_embeddings
    b = LlamaConfig.from_dict(TINY_B)
    assert b.rope_scaling.rope_type == "llama3" and b.rope_scaling.factor == 8.0
    assert b.rope_scaling.original_max_position_embeddings == 32
    assert b.tie_word_embeddings and b.rms_norm_eps == 1e-6 and b.rope_theta == 500000.0
    c = LlamaConfig.from_dict(TINY_C)
    assert c.q_size == 288 and c.hidden_size == 72 and c.attention_bias and c.mlp_bias
    assert c.rope_scaling.rope_type == "linear"


def test_defaults_follow_the_reference():
    raw = {"architectures": ["LlamaForCausalLM"], "num_hidden_layers": 1, "hidden_size": 32,
           "num_attention_heads": 4, "intermediate_size": 64, "vocab_size": 100}
    c = LlamaConfig.from_dict(raw)
    assert c.num_key_value_heads == 4          # default = heads
    assert c.head_dim == 8                     # default = E / H
    assert c.max_position_embeddings == 2048
    assert c.rms_norm_eps == 1e-5 and c.rope_theta == 10000.0
    assert not c.tie_word_embeddings and c.rope_scaling is None


def test_round_trip_through_to_dict():
    for raw in (TINY_A, TINY_B, TINY_C):
        c = LlamaConfig.from_dict(raw)
        assert LlamaConfig.from_dict(c.to_dict()) == c


@pytest.mark.parametrize("key,value,needle", [
    ("num_attention_heads", 5, "multiple"),            # heads % kv_heads
    ("num_key_value_heads", 8, "num_key_value_heads"), # kv > heads
    ("head_dim", 0, "head_dim"),
    ("head_dim", 15, "even"),
    ("hidden_size", -3, "hidden_size"),
    ("num_hidden_layers", 0, "num_hidden_layers"),
    ("vocab_size", "many", "vocab_size"),
    ("rms_norm_eps", float("nan"), "rms_norm_eps"),
    ("rms_norm_eps", -1.0, "rms_norm_eps"),
    ("rope_theta", 0.0, "rope_theta"),
    ("tie_word_embeddings", "yes", "tie_word_embeddings"),
    ("hidden_act", "gelu", "hidden_act"),
    ("intermediate_size", True, "intermediate_size"),
])
def test_bad_values_are_named(key, value, needle):
    raw = copy.deepcopy(TINY_A)
    raw[key] = value
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict(raw)
    assert needle in str(e.value)


def test_missing_required_key():
    for key in ("num_hidden_layers", "hidden_size", "num_attention_heads", "intermediate_size", "vocab_size"):
        raw = copy.deepcopy(TINY_A)
        del raw[key]
        with pytest.raises(ConfigError) as e:
            LlamaConfig.from_dict(raw)
        assert key in str(e.value)


def test_rope_scaling_refusals():
    raw = copy.deepcopy(TINY_B)
    raw["rope_scaling"]["rope_type"] = "yarn"
    with pytest.raises(ConfigError):
        LlamaConfig.from_dict(raw)
    raw = copy.deepcopy(TINY_B)
    raw["rope_scaling"]["high_freq_factor"] = 0.5       # must exceed low
    with pytest.raises(ConfigError):
        LlamaConfig.from_dict(raw)
    raw = copy.deepcopy(TINY_B)
    del raw["rope_scaling"]["factor"]
    with pytest.raises(ConfigError):
        LlamaConfig.from_dict(raw)
    raw = copy.deepcopy(TINY_B)
    raw["rope_scaling"] = {"type": "default"}
    assert LlamaConfig.from_dict(raw).rope_scaling is None


def test_unknown_architecture_lists_known(tmp_path):
    raw = copy.deepcopy(TINY_A)
    raw["architectures"] = ["MysteryForCausalLM"]
    with pytest.raises(ConfigError) as e:
        config_from_dict(raw)
    assert "MysteryForCausalLM" in str(e.value) and "LlamaForCausalLM" in str(e.value)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    with pytest.raises(ConfigError):
        load_config(str(tmp_path))
    with pytest.raises(ConfigError):
        load_config(str(tmp_path / "nowhere"))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError):
        load_config(str(tmp_path))


def test_registry_register_and_build():
    assert "LlamaForCausalLM" in known_architectures()
    arch, cfg = config_from_dict(TINY_B)
    spec = arch.build_spec(cfg)
    assert len(spec.layers) == 3 and [s.layer for s in spec.order] == [0, 1, 2]
    assert spec.head.params["tied"] is True
    assert spec.layers[1].mixer.params["num_kv_heads"] == 1
    assert spec.layers[0].mixer.params["position"].params["scaling"]["rope_type"] == "llama3"
    with pytest.raises(ValueError):
        register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, lambda c: None)
    register_architecture("OtherLM", LlamaConfig.from_dict, arch.build_spec)
    try:
        assert get_architecture("OtherLM").name == "OtherLM"
    finally:
        unregister_architecture("OtherLM")


def test_no_size_stands_in_code():
    """Two configurations that differ in every size give specs that differ in every size."""
    sa = config_from_dict(TINY_A)[0].build_spec(config_from_dict(TINY_A)[1])
    sb = config_from_dict(TINY_B)[0].build_spec(config_from_dict(TINY_B)[1])
    pa, pb = sa.layers[0].mixer.params, sb.layers[0].mixer.params
    for k in ("hidden_size", "num_heads", "num_kv_heads", "head_dim"):
        assert pa[k] != pb[k]
    assert sa.layers[0].feed_forward.params["intermediate_size"] != sb.layers[0].feed_forward.params["intermediate_size"]
    assert sa.layers[0].norms["mixer_norm"].params["eps"] != sb.layers[0].norms["mixer_norm"].params["eps"]
    assert sa.vocab_size != sb.vocab_size and len(sa.layers) != len(sb.layers)


def test_sizes_the_kernels_do_not_take_are_refused_when_the_model_is_built():
    """A head size beyond what the attention and rotation kernels take is an error at load,
    not at the first step (the reference refuses bad geometry at load too,
    src/model.c:2295-2329)."""
    from xyntetik_runner_amd.engine.model import Model
    raw = dict(TINY_A, head_dim=272, num_attention_heads=2, num_key_value_heads=1)
    arch, cfg = config_from_dict(raw)
    with pytest.raises(ValueError, match="head size 272"):
        Model(arch.build_spec(cfg))
    Model(config_from_dict(dict(raw, head_dim=256))[0].build_spec(config_from_dict(dict(raw, head_dim=256))[1]))
    # an activation the gated feed-forward's kernels do not have is named with the ones they have
    from xyntetik_runner_amd.config import PartSpec
    from xyntetik_runner_amd.parts import make_part
    with pytest.raises(ValueError, match="silu"):
        make_part("feed_forward", PartSpec("gated_mlp", {"hidden_size": 8, "intermediate_size": 16, "activation": "gelu"}))


def test_a_layer_brings_exactly_the_parts_its_arrangement_names():
    """The arrangement names its norms and says whether it has a mixer and a feed-forward; a layer
    spec that brings other norms, or lacks a part, is refused when the model is built."""
    from xyntetik_runner_amd.config import LayerSpec, PartSpec
    from xyntetik_runner_amd.engine.model import Model
    import dataclasses
    arch, cfg = config_from_dict(TINY_A)
    spec = arch.build_spec(cfg)
    layer = spec.layers[0]
    assert set(layer.norms) == {"mixer_norm", "feed_forward_norm"}
    third = dict(layer.norms, extra_norm=PartSpec("rmsnorm", {"size": 64, "eps": 1e-5}, prefix="x."))
    for bad in (dataclasses.replace(layer, norms=third),
                dataclasses.replace(layer, norms={"mixer_norm": layer.norms["mixer_norm"]}),
                dataclasses.replace(layer, feed_forward=None)):
        with pytest.raises(ValueError):
            Model(dataclasses.replace(spec, layers=[bad] + list(spec.layers[1:])))
    names = Model(spec).expected()
    assert "model.layers.0.input_layernorm.weight" in names and "model.layers.1.post_attention_layernorm.weight" in names
