"""Rotutar's typed configuration, read from the keys of its own config.json.

    architecture     "Rotutar"
    vocab, width     sizes of the token table and of the residual stream
    logit_softcap    null / absent, or c: logits <- c * tanh(logits / c)
    norm.eps         the epsilon of every norm of the model (layers, heads, the final norm)
    norm.groups      equal consecutive parts of a row that the layer and final norms divide by a root mean
                     square each
    layers           a list; each entry has ``type``, ``mixer`` and ``mlp``:
        type "hgrn2"     mixer {heads, dim, vdim}
        type "parallel"  mixer {left, right, left_scale, right_scale} with
                         left  {heads, kv_heads, dim, vdim, scale, rot: null or {dims, base}, mask: null or {size}}
                         right {heads, kv_heads, dim, vdim, conv}
        mlp              null, {kind: "dense", ff}, or {kind: "moe", expert {ff, limit}, router {experts, top,
                         groups: null or {count, keep}}}

Every size and constant of a model is one of these keys or a tensor's shape (the ranks of the delta rule's
low-rank projections are their tensors' shapes; the optional key ``rank`` of ``right`` only sizes random
weights).
"""

from dataclasses import dataclass
from typing import Optional, Tuple, Union

from .base import ConfigError, MAX_LAYERS, positive_extent, positive_finite, take

FAMILY = "rotutar"
MIXERS = ("hgrn2", "parallel")


def _need(data, field, kind, where):
    full = f"{where}.{field}" if where else field
    if not isinstance(data, dict) or field not in data or data[field] is None:
        raise ConfigError(FAMILY, full, "is required")
    return take({full: data[field]}, FAMILY, full, kind, None)


def _optional(data, field, where):
    """A nested object that may be absent or null."""
    value = data.get(field) if isinstance(data, dict) else None
    if value is not None and not isinstance(value, dict):
        raise ConfigError(FAMILY, f"{where}.{field}", "must be an object or null")
    return value


def _object(data, field, where):
    value = data.get(field) if isinstance(data, dict) else None
    if not isinstance(value, dict):
        raise ConfigError(FAMILY, f"{where}.{field}" if where else field, "must be an object")
    return value


@dataclass(frozen=True)
class ForgetGateSizes:
    heads: int
    dim: int
    vdim: int

    def to_dict(self):
        return {"dim": self.dim, "heads": self.heads, "vdim": self.vdim}


@dataclass(frozen=True)
class WindowAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int                                # 0: no rotation
    rot_base: float
    window: int                                  # mask.size; 0: every earlier position is seen

    def to_dict(self):
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim, "scale": self.scale,
                "rot": {"base": self.rot_base, "dims": self.rot_dims} if self.rot_dims else None,
                "mask": {"size": self.window} if self.window else None}


@dataclass(frozen=True)
class DeltaRuleSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    taps: int
    rank: Optional[int] = None                   # of the low-rank projections of random weights only

    def to_dict(self):
        data = {"conv": self.taps, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}
        if self.rank is not None:
            data["rank"] = self.rank
        return data


@dataclass(frozen=True)
class ParallelSizes:
    left: WindowAttentionSizes
    right: DeltaRuleSizes
    left_scale: float
    right_scale: float

    def to_dict(self):
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class DenseSizes:
    ff: int

    def to_dict(self):
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class ExpertSizes:
    experts: int
    ff: int
    limit: float
    top: int
    groups: int                                  # 0: no groups
    keep: int

    def to_dict(self):
        return {"expert": {"ff": self.ff, "limit": self.limit}, "kind": "moe",
                "router": {"experts": self.experts, "groups": {"count": self.groups, "keep": self.keep} if self.groups else None,
                           "top": self.top}}


@dataclass(frozen=True)
class RotutarLayer:
    type: str
    mixer: Union[ForgetGateSizes, ParallelSizes]
    mlp: Union[None, DenseSizes, ExpertSizes]

    def to_dict(self):
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None, "type": self.type}


def _mixer(kind, m, at):
    if kind == "hgrn2":
        return ForgetGateSizes(*(_need(m, key, int, at) for key in ("heads", "dim", "vdim")))
    left, right = _object(m, "left", at), _object(m, "right", at)
    la, ra = f"{at}.left", f"{at}.right"
    rot, mask = _optional(left, "rot", la), _optional(left, "mask", la)
    rot_dims = _need(rot, "dims", int, f"{la}.rot") if rot else 0
    return ParallelSizes(
        left=WindowAttentionSizes(
            heads=_need(left, "heads", int, la), kv_heads=_need(left, "kv_heads", int, la), dim=_need(left, "dim", int, la),
            vdim=_need(left, "vdim", int, la), scale=_need(left, "scale", float, la), rot_dims=rot_dims,
            rot_base=_need(rot, "base", float, f"{la}.rot") if rot_dims else 1.0,
            window=_need(mask, "size", int, f"{la}.mask") if mask else 0),
        right=DeltaRuleSizes(
            heads=_need(right, "heads", int, ra), kv_heads=_need(right, "kv_heads", int, ra), dim=_need(right, "dim", int, ra),
            vdim=_need(right, "vdim", int, ra), taps=_need(right, "conv", int, ra),
            rank=take(right, FAMILY, f"{ra}.rank", int, None, ("rank",))),
        left_scale=_need(m, "left_scale", float, at), right_scale=_need(m, "right_scale", float, at))


def _mlp(mlp, at):
    if mlp is None:
        return None
    kind = _need(mlp, "kind", str, at)
    if kind == "dense":
        return DenseSizes(_need(mlp, "ff", int, at))
    if kind != "moe":
        raise ConfigError(FAMILY, f"{at}.kind", f"unknown feed-forward `{kind}`, expected `dense` or `moe`")
    expert, router = _object(mlp, "expert", at), _object(mlp, "router", at)
    groups = _optional(router, "groups", f"{at}.router")
    return ExpertSizes(
        experts=_need(router, "experts", int, f"{at}.router"), ff=_need(expert, "ff", int, f"{at}.expert"),
        limit=_need(expert, "limit", float, f"{at}.expert"), top=_need(router, "top", int, f"{at}.router"),
        groups=_need(groups, "count", int, f"{at}.router.groups") if groups else 0,
        keep=_need(groups, "keep", int, f"{at}.router.groups") if groups else 0)


@dataclass(frozen=True)
class RotutarConfig:
    vocab: int
    width: int
    norm_eps: float
    norm_groups: int
    logit_softcap: Optional[float]
    layers: Tuple[RotutarLayer, ...]

    @classmethod
    def from_dict(cls, data):
        if not isinstance(data.get("layers"), (list, tuple)) or not data["layers"]:
            raise ConfigError(FAMILY, "layers", "must be a list with at least one layer")
        if len(data["layers"]) > MAX_LAYERS:
            raise ConfigError(FAMILY, "layers", f"must not exceed {MAX_LAYERS} entries")
        layers = []
        for index, entry in enumerate(data["layers"]):
            where = f"layers[{index}]"
            if not isinstance(entry, dict):
                raise ConfigError(FAMILY, where, "must be an object")
            kind = _need(entry, "type", str, where)
            if kind not in MIXERS:
                raise ConfigError(FAMILY, f"{where}.type", f"unknown mixer `{kind}`, expected one of " + ", ".join(f"`{m}`" for m in MIXERS))
            mixer = _mixer(kind, _object(entry, "mixer", where), f"{where}.mixer")
            layers.append(RotutarLayer(kind, mixer, _mlp(_optional(entry, "mlp", where), f"{where}.mlp")))
        norm = _object(data, "norm", "")
        config = cls(vocab=_need(data, "vocab", int, ""), width=_need(data, "width", int, ""),
                     norm_eps=_need(norm, "eps", float, "norm"), norm_groups=take(norm, FAMILY, "norm.groups", int, 1, ("groups",)),
                     logit_softcap=take(data, FAMILY, "logit_softcap", float, None), layers=tuple(layers))
        config.validate()
        return config

    def validate(self):
        positive_extent(FAMILY, "vocab", self.vocab)
        positive_extent(FAMILY, "width", self.width)
        positive_finite(FAMILY, "norm.eps", self.norm_eps)
        if self.norm_groups < 1 or self.width % self.norm_groups != 0:
            raise ConfigError(FAMILY, "norm.groups", "must be positive and divide the width")
        if self.logit_softcap is not None:
            positive_finite(FAMILY, "logit_softcap", self.logit_softcap)
        for index, layer in enumerate(self.layers):
            where = f"layers[{index}].mixer"
            if layer.type == "hgrn2":
                for key in ("heads", "dim", "vdim"):
                    positive_extent(FAMILY, f"{where}.{key}", getattr(layer.mixer, key))
            else:
                for side, sizes in (("left", layer.mixer.left), ("right", layer.mixer.right)):
                    for key in ("heads", "kv_heads", "dim", "vdim"):
                        positive_extent(FAMILY, f"{where}.{side}.{key}", getattr(sizes, key))
                    if sizes.heads % sizes.kv_heads != 0:
                        raise ConfigError(FAMILY, f"{where}.{side}.kv_heads", "must divide heads")
                left, right = layer.mixer.left, layer.mixer.right
                positive_finite(FAMILY, f"{where}.left.scale", left.scale)
                if left.rot_dims < 0 or left.rot_dims % 2 != 0 or left.rot_dims > left.dim:
                    raise ConfigError(FAMILY, f"{where}.left.rot.dims", "must be even and at most dim")
                if left.rot_dims:
                    positive_finite(FAMILY, f"{where}.left.rot.base", left.rot_base)
                if left.window < 0:
                    raise ConfigError(FAMILY, f"{where}.left.mask.size", "must be positive")
                positive_extent(FAMILY, f"{where}.right.conv", right.taps)
                if right.rank is not None:
                    positive_extent(FAMILY, f"{where}.right.rank", right.rank)
                for name in ("left_scale", "right_scale"):
                    value = getattr(layer.mixer, name)
                    if value != value or abs(value) == float("inf"):
                        raise ConfigError(FAMILY, f"{where}.{name}", "must be finite")
            e, where = layer.mlp, f"layers[{index}].mlp"
            if isinstance(e, DenseSizes):
                positive_extent(FAMILY, f"{where}.ff", e.ff)
            elif isinstance(e, ExpertSizes):
                for key, name in (("experts", "router.experts"), ("ff", "expert.ff"), ("top", "router.top")):
                    positive_extent(FAMILY, f"{where}.{name}", getattr(e, key))
                positive_finite(FAMILY, f"{where}.expert.limit", e.limit)
                if e.top > e.experts:
                    raise ConfigError(FAMILY, f"{where}.router.top", "must not exceed the experts")
                if e.groups:
                    if e.groups < 0 or e.experts % e.groups != 0:
                        raise ConfigError(FAMILY, f"{where}.router.groups.count", "must divide the experts")
                    if not (0 < e.keep <= e.groups) or e.keep * (e.experts // e.groups) < e.top:
                        raise ConfigError(FAMILY, f"{where}.router.groups.keep", "the groups that stay open must hold `top` experts")

    def to_dict(self):
        return {"architecture": "Rotutar", "layers": [layer.to_dict() for layer in self.layers],
                "logit_softcap": self.logit_softcap, "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
                "vocab": self.vocab, "width": self.width}
