"""Kosesun without a GPU: the configuration reader, the model's description as parts, the map
from checkpoint tensors to parameters, and loading a written folder."""

import copy

import pytest
import torch

import kosesun_models
from pagedserve_amd.config.base import ConfigError
from pagedserve_amd.config.kosesun import KosesunConfig
from pagedserve_amd.config.registry import resolve_architecture
from pagedserve_amd.model import load_model
from pagedserve_amd.model.decoder import DecoderModel
from pagedserve_amd.weights.loader import WeightError


def test_the_architecture_is_found_by_the_single_name_key():
    entry = resolve_architecture({"architecture": "Kosesun"})
    assert entry.name == "Kosesun" and entry.config_class is KosesunConfig
    assert resolve_architecture({"architectures": ["Kosesun"]}) is entry


@pytest.mark.parametrize("which", sorted(kosesun_models.MODELS))
def test_configuration_round_trip_and_spec(which):
    raw = kosesun_models.MODELS[which][0]
    config = KosesunConfig.from_dict(raw)
    assert KosesunConfig.from_dict(config.to_dict()) == config
    entry = resolve_architecture(raw)
    spec = entry.build_spec(config)
    assert spec.streams == raw.get("streams", 0) and spec.vocab_size == raw["vocab"]
    mixes = []
    for layer, block in zip(raw["layers"], spec.blocks):
        names = [name for name, _ in block.parts]
        assert ("feed_forward" in names) == (layer["mlp"] is not None)
        assert ("connect1" in names) == bool(raw.get("streams"))
        assert block.arrangement.startswith("hyper_connected" if raw.get("streams") else "pre_norm")
        assert block.arrangement.endswith("_mixer") == (layer["mlp"] is None)
        mixer = dict(block.mixer.params)
        if layer["type"] == "attention":
            assert block.mixer.kind == "attention"
            assert (mixer["heads"], mixer["kv_heads"], mixer["head_dim"], mixer["value_dim"]) == (
                layer["mixer"]["heads"], layer["mixer"]["kv_heads"], layer["mixer"]["dim"], layer["mixer"]["vdim"])
            assert mixer["rotary_dims"] == layer["mixer"]["rot"]["dims"]
            assert mixer["rotary_base"] == layer["mixer"]["rot"]["base"]
            assert mixer["scale"] == layer["mixer"]["scale"] and mixer["sink"] and mixer["head_gate"]
            mixes.append(mixer["value_mix"])
        else:
            assert block.mixer.kind == "gated_linear_attention"
            assert (mixer["key_dim"], mixer["value_dim"], mixer["tau"]) == (
                layer["mixer"]["dim"], layer["mixer"]["vdim"], layer["mixer"]["tau"])
    # the first layer that mixes values is the source, later ones mix, others do neither
    wanted, seen = [], False
    for layer in raw["layers"]:
        if layer["type"] != "attention":
            continue
        wanted.append("none" if not layer["mixer"]["v_mix"] else "mix" if seen else "source")
        seen = seen or layer["mixer"]["v_mix"]
    assert mixes == wanted


def test_every_parameter_has_a_source_and_every_tensor_a_parameter(tmp_path):
    for which in sorted(kosesun_models.MODELS):
        folder, raw, tensors, _ = kosesun_models.folder_of(tmp_path, which)
        model, config = load_model(folder, dtype="float32", device="cpu")
        entry = resolve_architecture(raw)
        used = set()
        for source in entry.weight_sources(config, model.spec).values():
            used.update(source.names)
        unused = set(tensors) - used
        assert all(entry.ignorable(config, name) for name in unused), unused
        # the one stored tensor that nothing reads: the mixing weight of the source layer
        assert len(unused) == (1 if any(l["type"] == "attention" and l["mixer"]["v_mix"]
                                        for l in raw["layers"]) else 0)
        groups, states = model.cache_requirements()
        assert len(states) == sum(l["type"] == "gla" for l in raw["layers"])
        assert bool(groups) == any(l["type"] == "attention" for l in raw["layers"])
        # the decay rank came from the tensor's shape
        for index, layer in enumerate(raw["layers"]):
            if layer["type"] == "gla":
                assert config.layers[index].mixer.decay_rank == tensors[f"l{index}.mix.a1"].shape[0]
        # scales that are stored around zero are bound with the one added
        gamma = model.final_norm.gamma
        assert torch.allclose(gamma, 1.0 + tensors["final.norm"])


def test_cache_requirements_follow_the_layers(tmp_path):
    folder, raw, _, _ = kosesun_models.folder_of(tmp_path, "A")
    model, _ = load_model(folder, dtype="bfloat16", device="cpu")
    groups, states = model.cache_requirements()
    # three attention layers of one geometry share a pool; heads are cached as wide as the larger size
    assert len(groups) == 1 and groups[0].entries == (1, 2, 3)
    assert (groups[0].kv_heads, groups[0].head_dim) == (2, 32)
    assert [(s.entry, s.shape, s.dtype) for s in states] == [(0, (2, 16, 24), torch.float32)]


def test_errors_name_what_is_wrong(tmp_path):
    raw = copy.deepcopy(kosesun_models.MODEL_A)
    raw["layers"][1]["type"] = "convolution"
    with pytest.raises(ConfigError, match="layers\\[1\\]"):
        KosesunConfig.from_dict(raw)
    raw = copy.deepcopy(kosesun_models.MODEL_A)
    raw["layers"][2]["mixer"]["vdim"] = 16        # mixing layers must agree
    with pytest.raises(ConfigError, match="agree"):
        KosesunConfig.from_dict(raw)
    raw = copy.deepcopy(kosesun_models.MODEL_A)
    raw["layers"][1]["mixer"]["rot"]["dims"] = 7
    with pytest.raises(ConfigError, match="rot.dims"):
        KosesunConfig.from_dict(raw)
    del raw["norm"]
    with pytest.raises(ConfigError):
        KosesunConfig.from_dict(raw)
    # a tensor of the wrong shape is reported by its stored name
    folder, raw, tensors, _ = kosesun_models.folder_of(tmp_path, "B")
    from safetensors.torch import save_file
    import os

    tensors["l0.mix.sink"] = torch.zeros(5)
    del tensors["l1.mix.a2.b"]
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightError) as caught:
        load_model(folder, dtype="float32", device="cpu")
    assert "l1.mix.a2.b" in caught.value.missing
    assert any(name == "l0.mix.sink" for name, _, _ in caught.value.wrong_shape)


def test_random_weights_mode_builds_a_model():
    from pagedserve_amd.model import random_model

    model, config = random_model(dict(kosesun_models.MODEL_C), seed=3, dtype="float32", device="cpu")
    assert isinstance(model, DecoderModel) and model.parameter_count > 0
    assert config.layers[1].mixer.decay_rank is None     # named by no one: the mode's own default
