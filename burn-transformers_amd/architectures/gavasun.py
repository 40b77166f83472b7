"""Gavasun as a family: its plan, its checkpoint contract and its random initialisation.

This is the only file that knows Gavasun's wiring and tensor names.
  plan      token table times a scale; layers of the kinds config.json lists, each a ``pre_norm`` block:
            x += mixer(norm1(x)), then, where the layer has a feed-forward, x += ff(norm2(x)); the norms are
            RMS norms whose scales are stored as their distance from one.  Mixers: ``rotary_attention`` (config
            type attention: biased projections, a short convolution behind each, norms over the whole query and
            key projections, halves turned together, keys seen in chunks), ``latent_attention`` (queries and
            keys/values through normalised latents, one turned key part for all heads, neighbouring channels
            turned together, a window of the latest positions) and ``gated_delta_rule`` (type delta: one decay
            per head, full-rank step sizes and output gate, the gate's SiLU).  The rotations' frequencies are
            slowed for long waves with a ramp over the pair index.  Feed-forwards: ``gated_dense``, or
            ``routed_experts`` with softmax scores, ungated units with the exact GELU and an expert every token
            uses.  With ``loop``, layers start .. stop - 1 run ``times`` times with the same tensors and a cache
            entry per run.  Final norm, readout with a table of its own.
  contract  tensor names ('l<i>.mix.*', 'l<i>.mlp.*', 'l<i>.norm1' ...), shapes
  init      random weights for tests and benchmarks
"""

import math

import torch

from ..config.gavasun import DenseSizes, GavasunConfig
from ..config.registry import Family, register_family
from ..engine.plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from ..weights.contract import Contract, TensorSpec

UNIT_EPS = 1e-6           # queries and keys of the delta rule: x / sqrt(sum x^2 + 1e-6)


def _attention_tensors(m, width):
    """[(name below '<layer>.mix.', shape, layout, role in the part)]"""
    q, k, v = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
    names = []
    for name, rows in (("q", q), ("k", k), ("v", v)):
        names += [(name, (rows, width), "out_in", name + "_weight"), (name + ".b", (rows,), "vector", name + "_bias")]
        if m.taps:
            names.append((name + ".conv", (rows, m.taps), "vector", name + "_conv"))
    return names + [("q.norm", (q,), "vector", "q_norm"), ("k.norm", (k,), "vector", "k_norm"),
                    ("o", (width, m.heads * m.vdim), "out_in", "out_weight")]


def _latent_tensors(m, width):
    return [("dq", (m.q_rank, width), "out_in", "down_q"), ("dq.norm", (m.q_rank,), "vector", "q_norm"),
            ("uq", (m.heads * (m.dim + m.rot_dim), m.q_rank), "out_in", "up_q"),
            ("dkv", (m.kv_rank + m.rot_dim, width), "out_in", "down_kv"), ("dkv.norm", (m.kv_rank,), "vector", "kv_norm"),
            ("uk", (m.heads * m.dim, m.kv_rank), "out_in", "up_k"), ("uv", (m.heads * m.vdim, m.kv_rank), "out_in", "up_v"),
            ("o", (width, m.heads * m.vdim), "out_in", "out_weight")]


def _delta_tensors(m, width):
    qk, inner = m.kv_heads * m.dim, m.heads * m.vdim
    return [("q", (qk, width), "out_in", "q_weight"), ("q.conv", (qk, m.taps), "vector", "q_conv"),
            ("k", (qk, width), "out_in", "k_weight"), ("k.conv", (qk, m.taps), "vector", "k_conv"),
            ("v", (inner, width), "out_in", "v_weight"), ("v.conv", (inner, m.taps), "vector", "v_conv"),
            ("b", (m.heads, width), "out_in", "beta_weight"), ("A_log", (m.heads,), "vector", "A_log"),
            ("norm", (m.vdim,), "vector", "norm_weight"), ("a", (m.heads, width), "out_in", "a_weight"),
            ("dt_bias", (m.heads,), "vector", "dt_bias"), ("g", (inner, width), "out_in", "g_weight"),
            ("o", (width, inner), "out_in", "out_weight")]


_MIXER_TENSORS = {"attention": _attention_tensors, "latent_attention": _latent_tensors, "delta": _delta_tensors}


def _mixer_tensors(layer, index, width):
    """[(checkpoint name, shape, layout, role in the layer's mixer part)]"""
    return [(f"l{index}.mix.{name}", shape, layout, role)
            for name, shape, layout, role in _MIXER_TENSORS[layer.type](layer.mixer, width)]


def _mlp_tensors(mlp, index, width):
    p = f"l{index}.mlp."
    if isinstance(mlp, DenseSizes):
        return [(p + "gate", (mlp.ff, width), "out_in", "gate_weight"), (p + "up", (mlp.ff, width), "out_in", "up_weight"),
                (p + "down", (width, mlp.ff), "out_in", "down_weight")]
    names = []
    for e in range(mlp.experts):
        names += [(f"{p}e{e}.up", (mlp.ff, width), "out_in", f"up_{e}"), (f"{p}e{e}.down", (width, mlp.ff), "out_in", f"down_{e}")]
    names.append((p + "router", (mlp.experts, width), "vector", "router"))          # routers are 32-bit: held widened
    if mlp.shared_ff:
        names += [(p + "shared.up", (mlp.shared_ff, width), "out_in", "shared_up"),
                  (p + "shared.down", (width, mlp.shared_ff), "out_in", "shared_down")]
    return names


def _rotation(rot):
    if rot is None:
        return {}
    return {"rot_base": rot.base, "rot_scaling": rot.scaling.to_dict() if rot.scaling else None}


def _mixer_spec(layer, index, config):
    width, eps, m = config.width, config.norm_eps, layer.mixer
    tensors = {role: name for name, _, _, role in _mixer_tensors(layer, index, width)}
    if layer.type == "attention":
        params = {"width": width, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                  "eps": eps, "head_norm": True, "norm_span": "whole", "rot_dims": m.rot.dims if m.rot else 0,
                  "rot_pairing": "halves", "chunk": m.chunk, "taps": m.taps}
        return PartSpec("rotary_attention", {**params, **_rotation(m.rot)}, tensors)
    if layer.type == "latent_attention":
        params = {"width": width, "heads": m.heads, "dim": m.dim, "vdim": m.vdim, "q_rank": m.q_rank, "kv_rank": m.kv_rank,
                  "scale": m.scale, "eps": eps, "window": m.window, "rot_dim": m.rot_dim, "rot_pairing": "neighbours"}
        return PartSpec("latent_attention", {**params, **_rotation(m.rot)}, tensors)
    return PartSpec("gated_delta_rule",
                    {"width": width, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "taps": m.taps,
                     "eps": eps, "unit_eps": UNIT_EPS, "low_rank": False, "decay_span": "head", "gate_act": "silu"}, tensors)


def _mlp_spec(mlp, index, config):
    tensors = {role: name for name, _, _, role in _mlp_tensors(mlp, index, config.width)}
    if isinstance(mlp, DenseSizes):
        return PartSpec("gated_dense", {"width": config.width, "inner": mlp.ff}, tensors)
    return PartSpec("routed_experts",
                    {"width": config.width, "experts": mlp.experts, "ff": mlp.ff, "top": mlp.top, "shared_ff": mlp.shared_ff,
                     "score": "softmax", "normalize": True, "unit": "gelu_erf"}, tensors)


def plan(config: GavasunConfig) -> ModelPlan:
    width = config.width

    def norm(name):
        return PartSpec("rms_norm", {"width": width, "eps": config.norm_eps, "offset": 1.0}, {"weight": name})

    layers = []
    for index, layer in enumerate(config.layers):
        p = f"l{index}."
        parts = {"mixer_norm": norm(p + "norm1"), "mixer": _mixer_spec(layer, index, config)}
        if layer.mlp is not None:
            parts.update(ff_norm=norm(p + "norm2"), ff=_mlp_spec(layer.mlp, index, config))
        layers.append(LayerPlan("pre_norm", parts))
    # every run of a layer keeps a cache entry of its own, numbered in the order the runs come
    schedule = [ScheduleEntry(layer=index, cache=run) for run, index in enumerate(config.runs())]
    return ModelPlan(
        width=width, vocab_size=config.vocab, max_positions=2 ** 31 - 1,      # positions are angles: no table bounds them
        embedding=PartSpec("token_only", {"width": width, "vocab_size": config.vocab, "scale": config.embedding_scale},
                           {"tokens": "embed"}),
        layers=layers, schedule=schedule, final_norm=norm("final.norm"),
        readout=PartSpec("linear_readout", {"width": width, "vocab_size": config.vocab}, {"weight": "head"}))


def contract(config: GavasunConfig) -> Contract:
    width = config.width
    tensors = [TensorSpec("embed", (config.vocab, width), "table")]
    for index, layer in enumerate(config.layers):
        p = f"l{index}."
        tensors += [TensorSpec(p + "norm" + n, (width,), "vector") for n in (("1", "2") if layer.mlp is not None else ("1",))]
        tensors += [TensorSpec(name, shape, layout) for name, shape, layout, _ in _mixer_tensors(layer, index, width)]
        if layer.mlp is not None:
            tensors += [TensorSpec(name, shape, layout) for name, shape, layout, _ in _mlp_tensors(layer.mlp, index, width)]
    tensors += [TensorSpec("final.norm", (width,), "vector"), TensorSpec("head", (config.vocab, width), "table")]
    return Contract(tensors=tensors, prefixes=("",), anchor="embed")


def init(config: GavasunConfig, generator):
    """Matrices N(0, 1/in); the layers' norm scales around zero (they are stored as the distance from one), the
    others around one; the recurrence's constants in ranges that keep decays between a half and nearly one."""

    def normal(shape, std, mean=0.0):
        return torch.randn(shape, generator=generator, dtype=torch.float32) * std + mean

    def uniform(shape, low, high):
        return torch.rand(shape, generator=generator, dtype=torch.float32) * (high - low) + low

    tensors = {}
    for spec in contract(config).tensors:
        name, shape = spec.name, spec.shape
        leaf = name.rsplit(".", 1)[-1]
        if name in ("embed", "head"):
            tensors[name] = normal(shape, 1.0 if name == "embed" else 1.0 / math.sqrt(shape[-1]))
        elif leaf == "conv":
            tensors[name] = normal(shape, 1.0 / math.sqrt(shape[1]))
        elif leaf == "A_log":
            tensors[name] = torch.log(uniform(shape, 0.5, 4.0))
        elif leaf == "dt_bias":                                        # softplus^-1 of a step size in 0.01 .. 0.2
            step = torch.exp(uniform(shape, math.log(0.01), math.log(0.2)))
            tensors[name] = step + torch.log(-torch.expm1(-step))
        elif leaf == "b" and spec.layout == "vector":                  # biases of the projections
            tensors[name] = normal(shape, 0.1)
        elif leaf in ("norm1", "norm2") or name == "final.norm":
            tensors[name] = normal(shape, 0.1)
        elif spec.layout == "vector" and len(shape) == 1:              # plain scales of the other norms
            tensors[name] = normal(shape, 0.1, 1.0)
        else:
            tensors[name] = normal(shape, 1.0 / math.sqrt(shape[-1]))
    return tensors


FAMILY = register_family(Family(
    name="gavasun", architectures=("Gavasun",), model_types=("gavasun",),
    config_class=GavasunConfig, plan=plan, contract=contract, init=init))
