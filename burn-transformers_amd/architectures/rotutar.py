"""Rotutar as a family: its plan, its checkpoint contract and its random initialisation.

This is the only file that knows Rotutar's wiring and tensor names.
  plan      token table; layers of the kinds config.json lists, each an ``output_norm`` block with gates:
            x += norm1(mixer(x) * sigmoid(rg1 x + b)), then, where the layer has a feed-forward,
            x += norm2(ff(x) * sigmoid(rg2 x + b)); the norms are RMS norms in ``norm.groups`` parts.
            Mixers: ``forget_gate_attention`` (config type hgrn2), and ``parallel_mixers`` (type parallel) of a
            ``rotary_attention`` (root mean square over the whole query / key projection, neighbouring channels
            turned together, a window of the latest positions, a sink logit per head) beside a
            ``gated_delta_rule``.  Feed-forwards: ``gated_dense``, or ``routed_experts`` with sigmoid scores,
            groups ranked by their two best, weights that are the scores as they are, and clamped units.
            Final norm in parts, readout with a table of its own and capped logits.
  contract  tensor names ('l<i>.mix.*', 'l<i>.mlp.*', 'l<i>.norm1', 'l<i>.rg1' ...), shapes; the ranks of the delta
            rule's low-rank projections are whatever the checkpoint holds
  init      random weights for tests and benchmarks
"""

import math

import torch

from ..config.registry import Family, register_family
from ..config.rotutar import DenseSizes, ExpertSizes, RotutarConfig
from ..engine.plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from ..weights.contract import Contract, TensorSpec

GROUP_RANK = 2            # a group of experts is ranked by the sum of its two best scores
UNIT_ALPHA = 1.702        # the experts' unit is g * sigmoid(1.702 g) * (u + 1)
UNIT_EPS = 1e-6           # queries and keys of the delta rule: x / sqrt(sum x^2 + 1e-6)


def _forget_tensors(sizes, width):
    """[(name below '<layer>.mix.', shape, layout, role in the part)]"""
    qk, inner = sizes.heads * sizes.dim, sizes.heads * sizes.vdim
    return [("q", (qk, width), "out_in", "q_weight"), ("f", (qk, width), "out_in", "f_weight"),
            ("f.b", (qk,), "vector", "f_bias"), ("lower", (qk,), "vector", "lower"),
            ("v", (inner, width), "out_in", "v_weight"), ("norm", (sizes.vdim,), "vector", "norm_weight"),
            ("o", (width, inner), "out_in", "out_weight")]


def _left_tensors(sizes, width):
    q, k, v = sizes.heads * sizes.dim, sizes.kv_heads * sizes.dim, sizes.kv_heads * sizes.vdim
    return [("q", (q, width), "out_in", "q_weight"), ("k", (k, width), "out_in", "k_weight"),
            ("v", (v, width), "out_in", "v_weight"), ("q.norm", (q,), "vector", "q_norm"),
            ("k.norm", (k,), "vector", "k_norm"), ("sink", (sizes.heads,), "vector", "sink"),
            ("o", (width, sizes.heads * sizes.vdim), "out_in", "out_weight")]


def _right_tensors(sizes, width, where):
    qk, inner, decays = sizes.kv_heads * sizes.dim, sizes.heads * sizes.vdim, sizes.heads * sizes.dim
    rank_a, rank_g = where + "a.rank", where + "g.rank"          # sizes that only the checkpoint gives
    return [("q", (qk, width), "out_in", "q_weight"), ("q.conv", (qk, sizes.taps), "vector", "q_conv"),
            ("k", (qk, width), "out_in", "k_weight"), ("k.conv", (qk, sizes.taps), "vector", "k_conv"),
            ("v", (inner, width), "out_in", "v_weight"), ("v.conv", (inner, sizes.taps), "vector", "v_conv"),
            ("b", (sizes.heads, width), "out_in", "beta_weight"), ("A_log", (sizes.heads,), "vector", "A_log"),
            ("norm", (sizes.vdim,), "vector", "norm_weight"), ("a1", (rank_a, width), "out_in", "a1"),
            ("a2", (decays, rank_a), "out_in", "a2"), ("dt_bias", (decays,), "vector", "dt_bias"),
            ("g1", (rank_g, width), "out_in", "g1"), ("g2", (inner, rank_g), "out_in", "g2"),
            ("o", (width, inner), "out_in", "out_weight")]


def _mixer_tensors(layer, index, width):
    """[(checkpoint name, shape, layout, role in the layer's mixer part)]"""
    p = f"l{index}.mix."
    if layer.type == "hgrn2":
        return [(p + name, shape, layout, role) for name, shape, layout, role in _forget_tensors(layer.mixer, width)]
    return [(p + "left." + name, shape, layout, "left." + role)
            for name, shape, layout, role in _left_tensors(layer.mixer.left, width)] + \
           [(p + "right." + name, shape, layout, "right." + role)
            for name, shape, layout, role in _right_tensors(layer.mixer.right, width, p + "right.")]


def _mlp_tensors(mlp, index, width):
    p = f"l{index}.mlp."
    if isinstance(mlp, DenseSizes):
        return [(p + "gate", (mlp.ff, width), "out_in", "gate_weight"), (p + "up", (mlp.ff, width), "out_in", "up_weight"),
                (p + "down", (width, mlp.ff), "out_in", "down_weight")]
    names = []
    for e in range(mlp.experts):
        names += [(f"{p}e{e}.gate", (mlp.ff, width), "out_in", f"gate_{e}"), (f"{p}e{e}.up", (mlp.ff, width), "out_in", f"up_{e}"),
                  (f"{p}e{e}.down", (width, mlp.ff), "out_in", f"down_{e}")]
    return names + [(p + "router", (mlp.experts, width), "vector", "router")]      # routers are 32-bit: held widened


def _mixer_spec(layer, index, config):
    width, eps = config.width, config.norm_eps
    tensors = {role: name for name, _, _, role in _mixer_tensors(layer, index, width)}
    m = layer.mixer
    if layer.type == "hgrn2":
        return PartSpec("forget_gate_attention", {"width": width, "heads": m.heads, "dim": m.dim, "vdim": m.vdim, "eps": eps},
                        tensors)
    left = {"kind": "rotary_attention",
            "params": {"width": width, "heads": m.left.heads, "kv_heads": m.left.kv_heads, "dim": m.left.dim,
                       "vdim": m.left.vdim, "scale": m.left.scale, "eps": eps, "head_norm": True, "norm_span": "whole",
                       "rot_dims": m.left.rot_dims, "rot_base": m.left.rot_base, "rot_pairing": "neighbours",
                       "window": m.left.window}}
    right = {"kind": "gated_delta_rule",
             "params": {"width": width, "heads": m.right.heads, "kv_heads": m.right.kv_heads, "dim": m.right.dim,
                        "vdim": m.right.vdim, "taps": m.right.taps, "eps": eps, "unit_eps": UNIT_EPS}}
    return PartSpec("parallel_mixers", {"left": left, "right": right, "left_scale": m.left_scale,
                                        "right_scale": m.right_scale}, tensors)


def _mlp_spec(mlp, index, config):
    tensors = {role: name for name, _, _, role in _mlp_tensors(mlp, index, config.width)}
    if isinstance(mlp, DenseSizes):
        return PartSpec("gated_dense", {"width": config.width, "inner": mlp.ff}, tensors)
    return PartSpec("routed_experts",
                    {"width": config.width, "experts": mlp.experts, "ff": mlp.ff, "top": mlp.top, "groups": mlp.groups,
                     "keep": mlp.keep, "score": "sigmoid", "group_rank": GROUP_RANK, "normalize": False,
                     "limit": mlp.limit, "alpha": UNIT_ALPHA}, tensors)


def plan(config: RotutarConfig) -> ModelPlan:
    width = config.width

    def norm(name):
        return PartSpec("rms_norm", {"width": width, "eps": config.norm_eps, "groups": config.norm_groups}, {"weight": name})

    def gate(name):
        return PartSpec("sigmoid_projection", {"width": width}, {"weight": name, "bias": name + ".b"})

    layers = []
    for index, layer in enumerate(config.layers):
        p = f"l{index}."
        parts = {"mixer": _mixer_spec(layer, index, config), "mixer_norm": norm(p + "norm1"), "mixer_gate": gate(p + "rg1")}
        if layer.mlp is not None:
            parts.update(ff=_mlp_spec(layer.mlp, index, config), ff_norm=norm(p + "norm2"), ff_gate=gate(p + "rg2"))
        layers.append(LayerPlan("output_norm", parts, {"mult": 1.0}))
    readout = {"width": width, "vocab_size": config.vocab}
    if config.logit_softcap is not None:
        readout["soft_cap"] = config.logit_softcap
    return ModelPlan(
        width=width, vocab_size=config.vocab, max_positions=2 ** 31 - 1,      # positions are angles: no table bounds them
        embedding=PartSpec("token_only", {"width": width, "vocab_size": config.vocab, "keep_operand": True}, {"tokens": "embed"}),
        layers=layers, schedule=[ScheduleEntry(layer=i, cache=i) for i in range(len(layers))],
        final_norm=norm("final.norm"), readout=PartSpec("linear_readout", readout, {"weight": "head"}))


def contract(config: RotutarConfig) -> Contract:
    width = config.width
    tensors = [TensorSpec("embed", (config.vocab, width), "table")]
    for index, layer in enumerate(config.layers):
        p = f"l{index}."
        sublayers = ("1", "2") if layer.mlp is not None else ("1",)
        tensors += [TensorSpec(p + "norm" + n, (width,), "vector") for n in sublayers]
        tensors += [TensorSpec(name, shape, layout) for name, shape, layout, _ in _mixer_tensors(layer, index, width)]
        if layer.mlp is not None:
            tensors += [TensorSpec(name, shape, layout) for name, shape, layout, _ in _mlp_tensors(layer.mlp, index, width)]
        for n in sublayers:
            tensors += [TensorSpec(p + "rg" + n, (width, width), "out_in"), TensorSpec(p + "rg" + n + ".b", (width,), "vector")]
    tensors += [TensorSpec("final.norm", (width,), "vector"), TensorSpec("head", (config.vocab, width), "table")]
    return Contract(tensors=tensors, prefixes=("",), anchor="embed")


def init(config: RotutarConfig, generator):
    """Matrices N(0, 1/in); norm scales around one; the recurrences' constants in ranges that keep decays between
    a half and nearly one; sinks around zero."""

    def normal(shape, std, mean=0.0):
        return torch.randn(shape, generator=generator, dtype=torch.float32) * std + mean

    def uniform(shape, low, high):
        return torch.rand(shape, generator=generator, dtype=torch.float32) * (high - low) + low

    ranks = {}
    for index, layer in enumerate(config.layers):
        if layer.type == "parallel":
            rank = layer.mixer.right.rank or max(8, config.width // 8)
            ranks[f"l{index}.mix.right.a.rank"] = ranks[f"l{index}.mix.right.g.rank"] = rank
    tensors = {}
    for spec in contract(config).tensors:
        name = spec.name
        shape = tuple(ranks[extent] if isinstance(extent, str) else extent for extent in spec.shape)
        leaf = name.rsplit(".", 1)[-1]
        if name in ("embed", "head"):
            tensors[name] = normal(shape, 1.0 if name == "embed" else 1.0 / math.sqrt(shape[-1]))
        elif name.endswith(".conv"):
            tensors[name] = normal(shape, 1.0 / math.sqrt(shape[1]))
        elif leaf == "lower":
            tensors[name] = uniform(shape, 0.0, 0.9)
        elif leaf == "A_log":
            tensors[name] = torch.log(uniform(shape, 0.5, 4.0))
        elif leaf == "dt_bias":                                        # softplus^-1 of a step size in 0.01 .. 0.2
            step = torch.exp(uniform(shape, math.log(0.01), math.log(0.2)))
            tensors[name] = step + torch.log(-torch.expm1(-step))
        elif leaf == "sink":
            tensors[name] = normal(shape, 1.0)
        elif leaf == "b" and spec.layout == "vector":                  # biases of the gates
            tensors[name] = normal(shape, 0.5)
        elif spec.layout == "vector" and len(shape) == 1:              # scales of norms
            tensors[name] = normal(shape, 0.1, 1.0)
        else:
            tensors[name] = normal(shape, 1.0 / math.sqrt(shape[-1]))
    return tensors


FAMILY = register_family(Family(
    name="rotutar", architectures=("Rotutar",), model_types=("rotutar",),
    config_class=RotutarConfig, plan=plan, contract=contract, init=init))
