"""Zetunex without a GPU: the configuration reader, the model's description as parts, the run
order with its passes, the map from checkpoint tensors to parameters, and the plain
implementation's own consistency (a sequence in pieces equals the sequence in one go)."""

import copy
import os

import pytest
import torch

import plain_zetunex as plain
import zetunex_models
from pagedserve_amd.config.base import ConfigError
from pagedserve_amd.config.registry import resolve_architecture
from pagedserve_amd.config.zetunex import ZetunexConfig
from pagedserve_amd.model import load_model
from pagedserve_amd.model.decoder import DecoderModel
from pagedserve_amd.weights.loader import WeightError

F64 = torch.float64


def test_the_architecture_is_found_by_its_name():
    entry = resolve_architecture({"architecture": "Zetunex"})
    assert entry.name == "Zetunex" and entry.config_class is ZetunexConfig


@pytest.mark.parametrize("which", sorted(zetunex_models.MODELS))
def test_configuration_round_trip_and_spec(which):
    raw = zetunex_models.MODELS[which][0]
    config = ZetunexConfig.from_dict(raw)
    assert ZetunexConfig.from_dict(config.to_dict()) == config
    spec = resolve_architecture(raw).build_spec(config)
    assert spec.vocab_size == raw["vocab"] and spec.tie_head and spec.streams == 0
    for layer, block in zip(raw["layers"], spec.blocks):
        names = [name for name, _ in block.parts]
        assert ("feed_forward" in names) == (layer["mlp"] is not None)
        assert block.arrangement == ("parallel_scaled" if layer["mlp"] is not None else "parallel_scaled_mixer")
        assert dict(block.params) == {"factor": raw.get("residual_mult", 1.0)}
        mixer = dict(block.mixer.params)
        if layer["type"] == "lightning":
            assert block.mixer.kind == "lightning_attention"
            assert mixer["decays"] == tuple(layer["mixer"]["decay"])
            assert (mixer["heads"], mixer["key_dim"], mixer["value_dim"]) == (
                layer["mixer"]["heads"], layer["mixer"]["dim"], layer["mixer"]["vdim"])
        else:
            assert block.mixer.kind == "side_by_side"
            left, right = dict(mixer["left"].params), dict(mixer["right"].params)
            wanted = layer["mixer"]["left"]
            assert (left["heads"], left["kv_heads"], left["head_dim"], left["value_dim"], left["scale"],
                    left["window"]) == (wanted["heads"], wanted["kv_heads"], wanted["dim"], wanted["vdim"],
                                        wanted["scale"], wanted["mask"]["size"])
            assert left["bias"] and not left["out_bias"]
            wanted = layer["mixer"]["right"]
            assert (right["inner"], right["states"], right["dt_rank"], right["taps"]) == (
                wanted["inner"], wanted["state"], wanted["dt_rank"], wanted["conv"])
        if layer["mlp"] is not None and layer["mlp"]["kind"] == "moe":
            router = layer["mlp"]["router"]
            ff = dict(block.feed_forward.params)
            assert block.feed_forward.kind == "moe"
            assert (ff["experts"], ff["top"], ff["groups"], ff["keep"], ff["scale"], ff["inner"]) == (
                router["experts"], router["top"], router["groups"]["count"], router["groups"]["keep"],
                router["scale"], layer["mlp"]["expert"]["ff"])


def test_the_run_order_passes_a_run_of_layers_several_times():
    config = ZetunexConfig.from_dict(zetunex_models.MODEL_A)      # layers 1..2 three times
    assert config.run_order() == [(0, -1), (1, 0), (2, -1), (1, 1), (2, -1), (1, 2), (2, -1), (3, -1)]
    assert config.run_order() == [(i, -1 if t is None else t) for i, t in plain.run_order(zetunex_models.MODEL_A)]
    spec = resolve_architecture(zetunex_models.MODEL_A).build_spec(config)
    # every call has a cache entry of its own, and the calls that open a pass name its vector
    assert [call.cache for call in spec.schedule] == list(range(8))
    assert [call.enter for call in spec.schedule] == [-1, 0, -1, 1, -1, 2, -1, -1]
    assert spec.pass_rows == 3
    config = ZetunexConfig.from_dict(zetunex_models.MODEL_B)      # no loop
    assert config.run_order() == [(0, -1), (1, -1), (2, -1)]
    assert resolve_architecture(zetunex_models.MODEL_B).build_spec(config).pass_rows == 0


def test_every_parameter_has_a_source_and_every_tensor_a_parameter(tmp_path):
    for which in sorted(zetunex_models.MODELS):
        folder, raw, tensors, _ = zetunex_models.folder_of(tmp_path, which)
        model, config = load_model(folder, dtype="float32", device="cpu")
        entry = resolve_architecture(raw)
        used = set()
        for source in entry.weight_sources(config, model.spec).values():
            used.update(source.names)
        assert used == set(tensors)
        # the experts' matrices lie one behind the other
        for index, layer in enumerate(raw["layers"]):
            if layer["mlp"] is not None and layer["mlp"]["kind"] == "moe":
                part = model.blocks[index].feed_forward
                ff = layer["mlp"]["expert"]["ff"]
                last = layer["mlp"]["router"]["experts"] - 1
                assert torch.equal(part.gate_up_weight[1, ff:], tensors[f"l{index}.mlp.e1.up"])
                assert torch.equal(part.down_weight[last], tensors[f"l{index}.mlp.e{last}.down"])
        if raw.get("loop"):
            assert torch.equal(model.pass_table, tensors["loop.step"])


def test_cache_requirements_follow_the_calls(tmp_path):
    folder, raw, _, _ = zetunex_models.folder_of(tmp_path, "A")
    model, _ = load_model(folder, dtype="bfloat16", device="cpu")
    groups, states = model.cache_requirements()
    # six calls of parallel layers: one windowed pool of six entries (heads cached as wide as the
    # larger size) and six scan states; two calls of recurrent layers: two matrix states
    assert len(groups) == 1 and len(groups[0].entries) == 6
    assert (groups[0].kv_heads, groups[0].head_dim, groups[0].window) == (2, 32, 10)
    shapes = sorted(tuple(s.shape) for s in states)
    assert shapes == [(2, 16, 24)] * 2 + [(48, 8 + 4 - 1)] * 6
    entries = [s.entry for s in states] + list(groups[0].entries)
    assert len(set(entries)) == len(entries)


def test_errors_name_what_is_wrong(tmp_path):
    raw = copy.deepcopy(zetunex_models.MODEL_A)
    raw["layers"][1]["type"] = "convolution"
    with pytest.raises(ConfigError, match="layers\\[1\\]"):
        ZetunexConfig.from_dict(raw)
    raw = copy.deepcopy(zetunex_models.MODEL_A)
    raw["layers"][0]["mixer"]["decay"] = [0.9]
    with pytest.raises(ConfigError, match="decay"):
        ZetunexConfig.from_dict(raw)
    raw = copy.deepcopy(zetunex_models.MODEL_A)
    raw["layers"][0]["mlp"]["router"]["top"] = 5         # two open groups of two experts
    with pytest.raises(ConfigError, match="per token"):
        ZetunexConfig.from_dict(raw)
    raw = copy.deepcopy(zetunex_models.MODEL_A)
    raw["loop"]["stop"] = 9
    with pytest.raises(ConfigError, match="loop"):
        ZetunexConfig.from_dict(raw)
    folder, raw, tensors, _ = zetunex_models.folder_of(tmp_path, "B")
    from safetensors.torch import save_file

    tensors["l0.mix.right.A_log"] = torch.zeros(5)
    del tensors["l1.mix.norm"]
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightError) as caught:
        load_model(folder, dtype="float32", device="cpu")
    assert "l1.mix.norm" in caught.value.missing
    assert any(name == "l0.mix.right.A_log" for name, _, _ in caught.value.wrong_shape)


def test_random_weights_mode_builds_a_model():
    from pagedserve_amd.model import random_model

    model, _ = random_model(dict(zetunex_models.MODEL_C), seed=3, dtype="float32", device="cpu")
    assert isinstance(model, DecoderModel) and model.parameter_count > 0


# ---------------------------------------------------------------- the plain implementation itself
def test_plain_recurrences_in_pieces_equal_one_go():
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn((20, 2, 4), generator=g, dtype=F64), torch.randn((20, 2, 4), generator=g, dtype=F64)
    v = torch.randn((20, 2, 6), generator=g, dtype=F64)
    decay = torch.tensor([0.9, 0.5], dtype=F64)
    whole, last = plain.decayed_recurrence(q, k, v, decay)
    first, state = plain.decayed_recurrence(q[:7], k[:7], v[:7], decay)
    second, state = plain.decayed_recurrence(q[7:], k[7:], v[7:], decay, state)
    assert torch.allclose(torch.cat([first, second]), whole) and torch.allclose(state, last)
    # the closed form of the same sum
    t = 13
    direct = sum(decay[1] ** (t - j) * (q[t, 1] @ k[j, 1]) * v[j, 1] for j in range(t + 1))
    assert torch.allclose(whole[t, 1], direct)
    raw = torch.randn((12, 3), generator=g, dtype=F64)
    weight, bias = torch.randn((3, 4), generator=g, dtype=F64), torch.randn(3, generator=g, dtype=F64)
    whole = plain.causal_conv(raw, weight, bias)
    tail = plain.causal_conv(raw[5:], weight, bias, before=raw[2:5])
    assert torch.allclose(tail, whole[5:])
    assert torch.allclose(whole[0], bias + weight[:, -1] * raw[0])      # zeros before the start


def test_plain_window_and_router():
    g = torch.Generator().manual_seed(1)
    q = torch.randn((9, 2, 4), generator=g, dtype=F64)
    k, v = torch.randn((9, 1, 4), generator=g, dtype=F64), torch.randn((9, 1, 3), generator=g, dtype=F64)
    # a window of one sees the token itself only; a window that nothing outgrows is no window
    assert torch.allclose(plain.windowed_attention(q, k, v, 0.5, 1), v.expand(9, 2, 3))
    assert torch.allclose(plain.windowed_attention(q, k, v, 0.5, 50), plain.windowed_attention(q, k, v, 0.5, 0))
    # the best expert of a closed group is not chosen
    logits = torch.tensor([[5.0, -9.0, 4.0, 3.9, 0.0, 0.1]], dtype=F64)
    chosen, weights = plain.route(logits, 3, 1, 2, 2.0)
    assert chosen == [[0, 1]]
    scores = torch.softmax(logits[0], 0)
    assert weights[0] == pytest.approx([2.0 * float(scores[0]), 2.0 * float(scores[1])])
    chosen, _ = plain.route(logits, 3, 2, 2, 1.0)
    assert chosen == [[0, 2]]
