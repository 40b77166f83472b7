"""Gavasun without a GPU: configuration, plan (loops, cache numbers), contract, the slowed frequencies, the cache
ledger's chunks and windows side by side, and pins of the plain implementation the GPU tests compare with."""

import copy
import math

import pytest
import torch

import burn_transformers_amd as bt
import plain_gavasun as plain
from burn_transformers_amd.cache.ledger import BLOCK, RELEASED, CacheLedger
from burn_transformers_amd.config import ConfigError, GavasunConfig, resolve_family
from burn_transformers_amd.parts.rotary_attention import rotary_amplitude, rotary_frequencies
from burn_transformers_amd.weights.contract import WeightError
from burn_transformers_amd.weights.loader import store_from_tensors
from gavasun_helpers import BASIC, CONFIGS, ODD, config_for, prompts_for, random_config, weights_for


def test_configuration_round_trip_and_family():
    for name, (config, _) in CONFIGS.items():
        for data in (config, config_for(name, "bfloat16")):
            typed = GavasunConfig.from_dict(data)
            assert GavasunConfig.from_dict(typed.to_dict()) == typed and typed.to_dict() == data
            assert resolve_family(data).name == "gavasun"
    for seed in range(30):
        data = random_config(seed)
        assert GavasunConfig.from_dict(data).to_dict() == data
    typed = GavasunConfig.from_dict(BASIC)
    assert [layer.type for layer in typed.layers] == ["attention", "delta", "latent_attention", "attention"]
    assert typed.layers[0].mixer.chunk == 24 and typed.layers[0].mixer.taps == 3 and typed.layers[0].mixer.rot.scaling.factor == 4.0
    assert typed.layers[2].mixer.window == 20 and typed.layers[2].mixer.rot.dims == 8 and typed.layers[3].mixer.rot.scaling is None
    assert typed.layers[1].mlp.shared_ff == 40 and typed.layers[2].mlp.shared_ff == 0 and typed.layers[3].mlp is None
    assert typed.runs() == [0, 1, 2, 1, 2, 3] and typed.embedding_scale == 2.0
    odd = GavasunConfig.from_dict(ODD)
    assert odd.runs() == [0, 1, 0, 1, 0, 1, 2, 3, 4, 5]
    assert odd.layers[3].mixer.taps == 0 and odd.layers[3].mixer.rot is None and odd.layers[3].mixer.chunk == 0
    assert odd.layers[4].mixer.rot_dim == 0 and odd.layers[4].mixer.window == 0
    assert GavasunConfig.from_dict(dict(BASIC, loop=None)).runs() == [0, 1, 2, 3]


@pytest.mark.parametrize("path,value,field", [
    (("width",), None, "width"), (("norm", "eps"), 0.0, "norm.eps"), (("embedding", "scale"), "x", "embedding.scale"),
    (("layers", 0, "type"), "conv", "layers[0].type"), (("layers", 0, "mixer", "dim"), 0, "layers[0].mixer.dim"),
    (("layers", 0, "mixer", "kv_heads"), 3, "layers[0].mixer.kv_heads"), (("layers", 0, "mixer", "rot", "dims"), 18, "layers[0].mixer.rot.dims"),
    (("layers", 0, "mixer", "rot", "scaling", "factor"), 0.0, "layers[0].mixer.rot.scaling.factor"),
    (("layers", 0, "mixer", "mask", "size"), -1, "layers[0].mixer.mask.size"), (("layers", 0, "mixer", "scale"), None, "layers[0].mixer.scale"),
    (("layers", 1, "mixer", "conv"), 0, "layers[1].mixer.conv"), (("layers", 1, "mixer", "kv_heads"), 3, "layers[1].mixer.kv_heads"),
    (("layers", 2, "mixer", "rot_dim"), 6, "layers[2].mixer.rot.dims"), (("layers", 2, "mixer", "kv_rank"), None, "layers[2].mixer.kv_rank"),
    (("layers", 2, "mixer", "rot"), None, "layers[2].mixer.rot"),
    (("layers", 1, "mlp", "router", "top"), 9, "layers[1].mlp.router.top"), (("layers", 1, "mlp", "expert", "ff"), 0, "layers[1].mlp.expert.ff"),
    (("layers", 0, "mlp", "kind"), "conv", "layers[0].mlp.kind"), (("loop", "stop"), 7, "loop.stop"), (("loop", "times"), 0, "loop.times")])
def test_configuration_errors_name_the_field(path, value, field):
    config = copy.deepcopy(BASIC)
    at = config
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ConfigError) as error:
        GavasunConfig.from_dict(config)
    assert error.value.field == field


def test_plan_names_the_parts_their_constants_and_a_cache_entry_for_every_run():
    family = resolve_family(BASIC)
    plan = family.plan(GavasunConfig.from_dict(BASIC))
    assert [layer.block for layer in plan.layers] == ["pre_norm"] * 4
    assert [(entry.layer, entry.cache) for entry in plan.schedule] == [(0, 0), (1, 1), (2, 2), (1, 3), (2, 4), (3, 5)]
    first, second, third, fourth = (layer.parts for layer in plan.layers)
    assert first["mixer"].kind == "rotary_attention" and first["ff"].kind == "gated_dense"
    assert second["mixer"].kind == "gated_delta_rule" and second["ff"].kind == "routed_experts"
    assert third["mixer"].kind == "latent_attention" and "ff" not in fourth and "ff_norm" not in fourth
    assert all(parts["mixer_norm"].kind == "rms_norm" and parts["mixer_norm"].params["offset"] == 1.0 for parts in (first, second, third, fourth))
    a = first["mixer"].params
    assert (a["chunk"], a["taps"], a["norm_span"], a["rot_pairing"], a["rot_dims"]) == (24, 3, "whole", "halves", 8)
    assert a["rot_scaling"] == {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0} and "window" not in a
    assert first["mixer"].tensors["q_bias"] == "l0.mix.q.b" and first["mixer"].tensors["v_conv"] == "l0.mix.v.conv"
    d = second["mixer"].params
    assert (d["decay_span"], d["low_rank"], d["gate_act"], d["taps"], d["unit_eps"]) == ("head", False, "silu", 4, 1e-6)
    assert second["mixer"].tensors["a_weight"] == "l1.mix.a" and second["mixer"].tensors["beta_weight"] == "l1.mix.b"
    m = third["mixer"].params
    assert (m["window"], m["rot_dim"], m["rot_pairing"], m["q_rank"], m["kv_rank"]) == (20, 8, "neighbours", 40, 32)
    assert "gate" not in third["mixer"].tensors
    e = second["ff"].params
    assert (e["score"], e["normalize"], e["unit"], e["shared_ff"], e["top"]) == ("softmax", True, "gelu_erf", 40, 3)
    assert "shared_mix" not in second["ff"].tensors and "shared_up" not in third["ff"].tensors
    assert plan.embedding.params["scale"] == 2.0 and plan.readout.tensors["weight"] == "head"
    late = family.plan(GavasunConfig.from_dict(ODD))
    assert "ff" not in late.layers[1].parts and late.layers[3].parts["mixer"].params["taps"] == 0
    assert "q_conv" not in late.layers[3].parts["mixer"].tensors and [entry.cache for entry in late.schedule] == list(range(10))


def test_contract_and_random_weights_agree():
    for config, seed in CONFIGS.values():
        family = resolve_family(config)
        typed, tensors = bt.random_tensors(config, seed)
        contract = family.contract(typed)
        assert {spec.name for spec in contract.tensors} == set(tensors)
        assert all(tuple(tensors[spec.name].shape) == tuple(spec.shape) for spec in contract.tensors)
    typed = GavasunConfig.from_dict(BASIC)
    specs = {spec.name: spec for spec in resolve_family(BASIC).contract(typed).tensors}
    assert specs["l0.mix.q.b"].shape == (64,) and specs["l0.mix.k.conv"].shape == (32, 3) and specs["l0.mix.q.norm"].shape == (64,)
    assert specs["l1.mix.a"].shape == (4, 64) and specs["l1.mix.dt_bias"].shape == (4,) and specs["l1.mix.g"].shape == (96, 64)
    assert specs["l2.mix.dkv"].shape == (40, 64) and specs["l2.mix.uq"].shape == (72, 40) and specs["l2.mix.dkv.norm"].shape == (32,)
    assert specs["l1.mlp.router"].layout == "vector" and "l1.mlp.e0.gate" not in specs and "l3.norm2" not in specs
    _, tensors = bt.random_tensors(BASIC, 1)
    tensors["l1.mix.a"] = tensors["l1.mix.a"][:3]
    with pytest.raises(WeightError):
        store_from_tensors(tensors, resolve_family(BASIC).contract(typed), torch.float32, "cpu")


def test_slowed_frequencies():
    """By hand: 8 pairs of base 10,000; a wave turns `original` / wavelength times.  Pairs that turn more than `fast`
    times keep their frequency, pairs that turn less than `slow` times are divided by the factor."""
    dims, base = 16, 10000.0
    scaling = {"factor": 4.0, "original": 100, "fast": 4.0, "slow": 1.0}
    plain_f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    got = rotary_frequencies(dims, base, scaling)
    turns = 100 * plain_f / (2.0 * math.pi)
    for i in range(dims // 2):
        if turns[i] > 4.0 * 3.2:          # well inside the kept end (the ramp's ends are rounded outwards to whole pairs)
            assert got[i] == plain_f[i]
        if turns[i] < 1.0 / 3.2:
            assert got[i] == pytest.approx(float(plain_f[i]) / 4.0, rel=1e-14)
    assert all(got[i] <= plain_f[i] and got[i] >= plain_f[i] / 4.0 for i in range(dims // 2))
    assert rotary_amplitude(scaling) == pytest.approx(0.1 * math.log(4.0) + 1.0) and rotary_amplitude(None) == 1.0
    assert torch.equal(rotary_frequencies(dims, base, None), plain_f)
    for rot in ({"dims": 24, "base": 3e5, "scaling": {"factor": 5.0, "original": 300, "fast": 20.0, "slow": 1.5}},
                {"dims": 6, "base": 50.0, "scaling": {"factor": 2.0, "original": 16, "fast": 2.0, "slow": 0.25}}):
        f, amplitude = plain.frequencies(rot)
        assert torch.allclose(rotary_frequencies(rot["dims"], rot["base"], rot["scaling"]), f, rtol=1e-13, atol=0.0)
        assert rotary_amplitude(rot["scaling"]) == pytest.approx(amplitude)


def test_ledger_gives_blocks_back_behind_a_chunk_and_behind_a_window():
    chunk, window = 150, 70
    ledger = CacheLedger(3, 64, 4, 32, windows=[0, window, 0], chunks=[0, 0, chunk])
    slot = ledger.acquire()
    for length in (130, 149, 150, 151, 299, 300, 500):
        ledger.check_growth({slot: length})
        ledger.reserve(slot, length)
        ledger.commit(slot, length)
        ledger.check()
        behind_window = max(0, length - window + 1) // BLOCK          # the block of the first key the NEXT token's window holds
        behind_chunk = (length // chunk * chunk) // BLOCK              # the block in which the NEXT token's chunk begins
        for group, first in ((1, behind_window), (2, behind_chunk)):
            held = ledger.held_blocks[group][slot]
            assert all(block == RELEASED for block in held[:first]) and RELEASED not in held[first:]
        assert RELEASED not in ledger.held_blocks[0][slot]
    ledger.release(slot)
    ledger.check()


def test_plain_mechanisms_are_pinned():
    """The plain implementation on inputs whose answers are known by hand."""
    # the layers' norm: the stored scale is the distance from one
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    assert torch.allclose(plain.layer_norm(x, torch.tensor([0.0, 1.0], dtype=torch.float64), 0.0),
                          torch.tensor([[3.0, 8.0]], dtype=torch.float64) / math.sqrt(12.5))
    # the short convolution: the last tap meets the current token, zeros stand before the start, nothing follows it
    taps = torch.tensor([[10.0, 1.0]], dtype=torch.float64)
    y = plain.short_conv(torch.tensor([[1.0], [2.0], [3.0]], dtype=torch.float64), taps)
    assert torch.equal(y, torch.tensor([[1.0], [12.0], [23.0]], dtype=torch.float64))
    # pairs: halves turn channel i with i + dims / 2, neighbours 2i with 2i + 1; channels behind dims stay; a quarter turn
    rot = {"dims": 4, "base": 1.0, "scaling": None}
    v = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0]]], dtype=torch.float64)
    quarter = torch.tensor([math.pi / 2.0])
    assert torch.allclose(plain.turn(v, quarter, rot, "halves"), torch.tensor([[[-3.0, -4.0, 1.0, 2.0, 5.0]]], dtype=torch.float64))
    assert torch.allclose(plain.turn(v, quarter, rot, "neighbours"), torch.tensor([[[-2.0, 1.0, -4.0, 3.0, 5.0]]], dtype=torch.float64))
    # the exact GELU
    assert float(plain.gelu_erf(torch.tensor(1.0, dtype=torch.float64))) == pytest.approx(0.8413447460685429)


def test_plain_experts_by_hand():
    """Two of three experts: the scores' softmax, the two largest, their scores over their sum; the shared expert on top."""
    width = 2
    w = {"m.router": torch.tensor([[1.0, 0.0], [0.0, 1.0], [-1.0, -1.0]], dtype=torch.float64)}
    for e in range(3):
        w[f"m.e{e}.up"] = torch.eye(width, dtype=torch.float64) * (e + 1)
        w[f"m.e{e}.down"] = torch.eye(width, dtype=torch.float64)
    w["m.shared.up"], w["m.shared.down"] = torch.eye(width, dtype=torch.float64), 2.0 * torch.eye(width, dtype=torch.float64)
    h = torch.tensor([[2.0, 1.0]], dtype=torch.float64)
    mlp = {"kind": "moe", "expert": {"ff": 2}, "router": {"experts": 3, "top": 2}, "shared": {"ff": 2}}
    s = torch.softmax(torch.tensor([2.0, 1.0, -3.0], dtype=torch.float64), 0)
    want = (s[0] * plain.gelu_erf(h) + s[1] * plain.gelu_erf(2.0 * h)) / (s[0] + s[1]) + 2.0 * plain.gelu_erf(h)
    assert torch.allclose(plain.experts(h, w, "m.", mlp), want, rtol=1e-14)
    assert torch.allclose(plain.experts(h, w, "m.", dict(mlp, shared=None)), want - 2.0 * plain.gelu_erf(h), rtol=1e-13)


def test_plain_chunks_and_windows_hide_exactly_the_keys_before_them():
    for name, index, sizes in (("attention", 0, (40, 39)), ("latent", 0, (33, 32))):
        config, weights = CONFIGS[name][0], weights_for(name)
        ids = prompts_for(name, [90])[0]
        base = plain.forward(ids, weights, config)
        mixer = copy.deepcopy(config["layers"][index]["mixer"])
        mixer["mask"] = {"size": sizes[1]}
        other = plain.forward(ids, weights, dict(config, layers=[dict(config["layers"][index], mixer=mixer)]))
        # up to the shorter edge both see the same keys; the next position loses its first key (window) or all but itself (chunk)
        assert float((other[:sizes[1]] - base[:sizes[1]]).abs().max()) < 1e-12
        assert float((other[sizes[1]] - base[sizes[1]]).abs().max()) > 1e-6


def test_plain_recurrence_carries_its_state_and_loops_run_their_layers_again():
    config, weights = CONFIGS["delta"][0], weights_for("delta")
    ids = prompts_for("delta", [80])[0]
    other = [(ids[0] + 1) % config["vocab"]] + ids[1:]
    assert float((plain.forward(ids, weights, config)[-1] - plain.forward(other, weights, config)[-1]).abs().max()) > 1e-6
    streams = []
    plain.forward(ids[:9], weights_for("basic"), BASIC, streams=streams)
    assert len(streams) == 6 and plain.runs(BASIC) == [0, 1, 2, 1, 2, 3]
