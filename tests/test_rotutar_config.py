"""Rotutar without a GPU: configuration, plan, contract (with extents that only the checkpoint gives), the cache
ledger's window, and pins of the plain implementation the GPU tests compare with."""

import copy
import math

import pytest
import torch

import burn_transformers_amd as bt
import plain_rotutar as plain
from burn_transformers_amd.cache.ledger import BLOCK, RELEASED, CacheLedger
from burn_transformers_amd.config import ConfigError, RotutarConfig, resolve_family
from burn_transformers_amd.weights.contract import WeightError, fits
from burn_transformers_amd.weights.loader import store_from_tensors
from rotutar_helpers import BASIC, CONFIGS, ODD, config_for, prompts_for, weights_for


def test_configuration_round_trip_and_family():
    for name, (config, _) in CONFIGS.items():
        for data in (config, config_for(name, "bfloat16")):
            typed = RotutarConfig.from_dict(data)
            assert RotutarConfig.from_dict(typed.to_dict()) == typed and typed.to_dict() == data
            assert resolve_family(data).name == "rotutar"
    typed = RotutarConfig.from_dict(BASIC)
    assert [layer.type for layer in typed.layers] == ["hgrn2", "parallel", "hgrn2"]
    assert typed.layers[1].mixer.left.window == 24 and typed.layers[1].mixer.right.taps == 3
    assert typed.layers[1].mlp.groups == 3 and typed.layers[2].mlp.groups == 0 and typed.layers[0].mlp.ff == 96
    odd = RotutarConfig.from_dict(ODD)
    assert odd.layers[0].mlp is None and odd.logit_softcap is None and odd.norm_groups == 1
    assert odd.layers[2].mixer.left.window == 0 and odd.layers[2].mixer.left.rot_dims == 0


@pytest.mark.parametrize("path,value,field", [
    (("width",), None, "width"), (("norm", "eps"), 0.0, "norm.eps"), (("norm", "groups"), 3, "norm.groups"),
    (("layers", 0, "type"), "conv", "layers[0].type"), (("layers", 0, "mixer", "dim"), 0, "layers[0].mixer.dim"),
    (("layers", 1, "mixer", "left", "kv_heads"), 3, "layers[1].mixer.left.kv_heads"),
    (("layers", 1, "mixer", "left", "rot", "dims"), 18, "layers[1].mixer.left.rot.dims"),
    (("layers", 1, "mixer", "right", "conv"), 0, "layers[1].mixer.right.conv"),
    (("layers", 1, "mixer", "right", "kv_heads"), 3, "layers[1].mixer.right.kv_heads"),
    (("layers", 1, "mixer", "left_scale"), None, "layers[1].mixer.left_scale"),
    (("layers", 1, "mlp", "router", "top"), 9, "layers[1].mlp.router.top"),
    (("layers", 1, "mlp", "router", "groups", "count"), 4, "layers[1].mlp.router.groups.count"),
    (("layers", 1, "mlp", "router", "groups", "keep"), 1, "layers[1].mlp.router.groups.keep"),
    (("layers", 1, "mlp", "expert", "limit"), -1.0, "layers[1].mlp.expert.limit"),
    (("layers", 0, "mlp", "kind"), "conv", "layers[0].mlp.kind"), (("logit_softcap",), -2.0, "logit_softcap")])
def test_configuration_errors_name_the_field(path, value, field):
    config = copy.deepcopy(BASIC)
    at = config
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ConfigError) as error:
        RotutarConfig.from_dict(config)
    assert error.value.field == field


def test_plan_names_the_parts_and_their_constants():
    family = resolve_family(BASIC)
    plan = family.plan(RotutarConfig.from_dict(BASIC))
    assert [layer.block for layer in plan.layers] == ["output_norm"] * 3
    assert [entry.cache for entry in plan.schedule] == [0, 1, 2]
    first, second, third = (layer.parts for layer in plan.layers)
    assert first["mixer"].kind == "forget_gate_attention" and first["ff"].kind == "gated_dense"
    assert second["mixer"].kind == "parallel_mixers" and second["ff"].kind == "routed_experts"
    assert all(parts[role].kind == "sigmoid_projection" for parts in (first, second, third) for role in ("mixer_gate", "ff_gate"))
    assert all(parts[role].params["groups"] == 2 for parts in (first, second, third) for role in ("mixer_norm", "ff_norm"))
    left, right = second["mixer"].params["left"], second["mixer"].params["right"]
    assert left["kind"] == "rotary_attention" and left["params"]["window"] == 24 and left["params"]["rot_pairing"] == "neighbours"
    assert left["params"]["norm_span"] == "whole" and right["kind"] == "gated_delta_rule" and right["params"]["taps"] == 3
    assert second["mixer"].tensors["left.sink"] == "l1.mix.left.sink" and second["mixer"].tensors["right.a2"] == "l1.mix.right.a2"
    experts = second["ff"].params
    assert (experts["score"], experts["group_rank"], experts["normalize"], experts["limit"]) == ("sigmoid", 2, False, 1.0)
    assert plan.readout.params["soft_cap"] == 20.0 and plan.readout.tensors["weight"] == "head"
    assert plan.embedding.params["keep_operand"] is True
    late = family.plan(RotutarConfig.from_dict(ODD))
    assert "ff" not in late.layers[0].parts and "ff_gate" not in late.layers[0].parts and "soft_cap" not in late.readout.params


def test_contract_and_random_weights_agree_and_ranks_are_free():
    for config, seed in CONFIGS.values():
        family = resolve_family(config)
        typed, tensors = bt.random_tensors(config, seed)
        contract = family.contract(typed)
        assert {spec.name for spec in contract.tensors} == set(tensors)
        free = {}
        for spec in contract.tensors:
            assert fits(tuple(tensors[spec.name].shape), spec.shape, free), spec.name
    typed = RotutarConfig.from_dict(BASIC)
    specs = {spec.name: spec for spec in resolve_family(BASIC).contract(typed).tensors}
    assert specs["l1.mix.right.a1"].shape == ("l1.mix.right.a.rank", 64) and specs["l1.mix.right.a2"].shape == (64, "l1.mix.right.a.rank")
    assert specs["l1.mlp.router"].layout == "vector" and specs["l1.rg2"].shape == (64, 64) and "l1.mix.left.sink" in specs
    # an extent that a name stands for fits any size, but the same everywhere
    free = {}
    assert fits((7, 64), ("r", 64), free) and fits((64, 7), (64, "r"), free) and not fits((64, 8), (64, "r"), free)
    assert not fits((7,), ("r", 64), {}) and not fits((0, 64), ("r", 64), {})
    _, tensors = bt.random_tensors(BASIC, 1)
    tensors["l1.mix.right.g2"] = tensors["l1.mix.right.g2"][:, :4]
    with pytest.raises(WeightError):
        store_from_tensors(tensors, resolve_family(BASIC).contract(typed), torch.float32, "cpu")


def test_ledger_gives_blocks_behind_a_window_back():
    window = 70
    ledger = CacheLedger(2, 64, 4, 32, windows=[0, window])
    slot = ledger.acquire()
    for length in (130, 131, 132, 192, 193, 500):
        ledger.check_growth({slot: length})
        ledger.reserve(slot, length)
        ledger.commit(slot, length)
        ledger.check()
        first = max(0, length - window + 1) // BLOCK          # the block of the first key the NEXT token's window holds
        held = ledger.held_blocks[1][slot]
        assert all(block == RELEASED for block in held[:first]) and RELEASED not in held[first:]
        assert RELEASED not in ledger.held_blocks[0][slot]
    ledger.release(slot)
    ledger.check()
    assert ledger.blocks[1].available() == 64


def test_plain_mechanisms_are_pinned():
    """The plain implementation on inputs whose answers are known by hand."""
    # norm in parts: every part of the row ends with a mean square of one
    x = torch.tensor([[3.0, 4.0, 0.0, 0.5]], dtype=torch.float64)
    normed = plain.group_norm(x, torch.ones(4, dtype=torch.float64), 2, 0.0)
    assert torch.allclose((normed.view(1, 2, 2) ** 2).mean(-1), torch.ones(1, 2, dtype=torch.float64))
    # the short convolution: the last tap meets the current token, zeros stand before the start
    taps = torch.tensor([[10.0, 1.0]], dtype=torch.float64)
    y = plain.short_conv(torch.tensor([[1.0], [2.0], [3.0]], dtype=torch.float64), taps)
    assert torch.allclose(y, plain.silu(torch.tensor([[1.0], [12.0], [23.0]], dtype=torch.float64)))
    # the choice: groups ranked by their two best, the lowest index among equals
    scores = torch.tensor([0.9, 0.05, 0.05, 0.6, 0.55, 0.1, 0.5, 0.5, 0.1], dtype=torch.float64)
    assert plain.choose(scores, {"experts": 9, "top": 2, "groups": {"count": 3, "keep": 2}}) == [3, 4]
    assert plain.choose(scores, {"experts": 9, "top": 3, "groups": None}) == [0, 3, 4]
    assert plain.choose(torch.full((4,), 0.5, dtype=torch.float64), {"experts": 4, "top": 2, "groups": None}) == [0, 1]


def test_plain_sink_takes_weight_from_every_key_and_windows_hide_keys():
    name = "attention"
    config, weights = CONFIGS[name][0], dict(weights_for(name))
    ids = prompts_for(name, [60])[0]
    base = plain.forward(ids, weights, config)
    weights["l0.mix.left.sink"] = weights["l0.mix.left.sink"] + 3.0
    assert float((plain.forward(ids, weights, config) - base).abs().max()) > 1e-3
    mixer = copy.deepcopy(config["layers"][0]["mixer"])
    mixer["left"]["mask"] = {"size": 39}
    shorter = plain.forward(ids, weights_for(name), dict(config, layers=[dict(config["layers"][0], mixer=mixer)]))
    # the first 39 positions see the same keys under both windows; position 39 loses its first key
    assert float((shorter[:39] - base[:39]).abs().max()) < 1e-12 and float((shorter[39] - base[39]).abs().max()) > 1e-6


def test_plain_recurrences_carry_their_state():
    """A change of the first token reaches the last logits through the states alone (one layer, no attention seen)."""
    for name in ("forget", "delta"):
        config, weights = CONFIGS[name][0], weights_for(name)
        ids = prompts_for(name, [80])[0]
        other = [(ids[0] + 1) % config["vocab"]] + ids[1:]
        assert float((plain.forward(ids, weights, config)[-1] - plain.forward(other, weights, config)[-1]).abs().max()) > 1e-6
