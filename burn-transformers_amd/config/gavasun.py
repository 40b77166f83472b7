"""Gavasun's typed configuration, read from the keys of its own config.json.

    architecture     "Gavasun"
    vocab, width     sizes of the token table and of the residual stream
    embedding.scale  factor on the token table's rows
    norm.eps         the epsilon of every RMS norm of the model (layers, latents, whole projections, heads, final)
    loop             null / absent, or {start, stop, times}: layers start .. stop - 1 run ``times`` times in a row
                     with the same tensors, every run with a cache entry of its own
    layers           a list; each entry has ``type``, ``mixer`` and ``mlp``:
        type "attention"         mixer {heads, kv_heads, dim, vdim, scale, conv, rot, mask}; mask.size is a chunk
        type "latent_attention"  mixer {heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot, mask}; mask.size is
                                 a window of the latest positions
        type "delta"             mixer {heads, kv_heads, dim, vdim, conv}
        rot                      null, or {dims, base, scaling: null or {factor, original, fast, slow}}
        mlp                      null, {kind: "dense", ff}, or {kind: "moe", expert {ff}, router {experts, top},
                                 shared: null or {ff}}
"""

from dataclasses import dataclass
from typing import Optional, Tuple, Union

from .base import ConfigError, MAX_LAYERS, positive_extent, positive_finite, take

FAMILY = "gavasun"
MIXERS = ("attention", "latent_attention", "delta")


def _need(data, field, kind, where):
    full = f"{where}.{field}" if where else field
    if not isinstance(data, dict) or field not in data or data[field] is None:
        raise ConfigError(FAMILY, full, "is required")
    return take({full: data[field]}, FAMILY, full, kind, None)


def _optional(data, field, where):
    """A nested object that may be absent or null."""
    value = data.get(field) if isinstance(data, dict) else None
    if value is not None and not isinstance(value, dict):
        raise ConfigError(FAMILY, f"{where}.{field}" if where else field, "must be an object or null")
    return value


def _object(data, field, where):
    value = data.get(field) if isinstance(data, dict) else None
    if not isinstance(value, dict):
        raise ConfigError(FAMILY, f"{where}.{field}" if where else field, "must be an object")
    return value


@dataclass(frozen=True)
class WaveScaling:
    """Frequencies slowed by ``factor`` for long waves: a wave that turns fewer than ``slow`` times in ``original``
    positions is slowed in full, one that turns more than ``fast`` times is kept."""
    factor: float
    original: float
    fast: float
    slow: float

    def to_dict(self):
        return {"factor": self.factor, "fast": self.fast, "original": self.original, "slow": self.slow}


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    scaling: Optional[WaveScaling]

    def to_dict(self):
        return {"base": self.base, "dims": self.dims, "scaling": self.scaling.to_dict() if self.scaling else None}


@dataclass(frozen=True)
class ChunkAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    taps: int                                    # conv; 0: no convolution behind the projections
    rot: Optional[Rotation]
    chunk: int                                   # mask.size; 0: every earlier position is seen

    def to_dict(self):
        data = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim, "scale": self.scale,
                "rot": self.rot.to_dict() if self.rot else None, "mask": {"size": self.chunk} if self.chunk else None}
        if self.taps:
            data["conv"] = self.taps
        return data


@dataclass(frozen=True)
class LatentAttentionSizes:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: Optional[Rotation]
    window: int                                  # mask.size; 0: every earlier position is seen

    def to_dict(self):
        return {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "q_rank": self.q_rank, "rot_dim": self.rot_dim,
                "vdim": self.vdim, "scale": self.scale, "rot": self.rot.to_dict() if self.rot else None,
                "mask": {"size": self.window} if self.window else None}


@dataclass(frozen=True)
class DeltaSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    taps: int

    def to_dict(self):
        return {"conv": self.taps, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}


@dataclass(frozen=True)
class DenseSizes:
    ff: int

    def to_dict(self):
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class ExpertSizes:
    experts: int
    ff: int
    top: int
    shared_ff: int                               # 0: no expert that every token uses

    def to_dict(self):
        return {"expert": {"ff": self.ff}, "kind": "moe", "router": {"experts": self.experts, "top": self.top},
                "shared": {"ff": self.shared_ff} if self.shared_ff else None}


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int

    def to_dict(self):
        return {"start": self.start, "stop": self.stop, "times": self.times}


@dataclass(frozen=True)
class GavasunLayer:
    type: str
    mixer: Union[ChunkAttentionSizes, LatentAttentionSizes, DeltaSizes]
    mlp: Union[None, DenseSizes, ExpertSizes]

    def to_dict(self):
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None, "type": self.type}


def _rotation(m, at):
    rot = _optional(m, "rot", at)
    if not rot or not rot.get("dims"):
        return None
    where = f"{at}.rot"
    scaling = _optional(rot, "scaling", where)
    if scaling:
        scaling = WaveScaling(*(_need(scaling, key, float, f"{where}.scaling") for key in ("factor", "original", "fast", "slow")))
    return Rotation(_need(rot, "dims", int, where), _need(rot, "base", float, where), scaling or None)


def _mask(m, at):
    mask = _optional(m, "mask", at)
    return _need(mask, "size", int, f"{at}.mask") if mask else 0


def _mixer(kind, m, at):
    if kind == "delta":
        return DeltaSizes(*(_need(m, key, int, at) for key in ("heads", "kv_heads", "dim", "vdim", "conv")))
    if kind == "attention":
        return ChunkAttentionSizes(
            heads=_need(m, "heads", int, at), kv_heads=_need(m, "kv_heads", int, at), dim=_need(m, "dim", int, at),
            vdim=_need(m, "vdim", int, at), scale=_need(m, "scale", float, at),
            taps=take(m, FAMILY, f"{at}.conv", int, 0, ("conv",)), rot=_rotation(m, at), chunk=_mask(m, at))
    return LatentAttentionSizes(
        heads=_need(m, "heads", int, at), dim=_need(m, "dim", int, at), rot_dim=take(m, FAMILY, f"{at}.rot_dim", int, 0, ("rot_dim",)),
        vdim=_need(m, "vdim", int, at), q_rank=_need(m, "q_rank", int, at), kv_rank=_need(m, "kv_rank", int, at),
        scale=_need(m, "scale", float, at), rot=_rotation(m, at), window=_mask(m, at))


def _mlp(mlp, at):
    if mlp is None:
        return None
    kind = _need(mlp, "kind", str, at)
    if kind == "dense":
        return DenseSizes(_need(mlp, "ff", int, at))
    if kind != "moe":
        raise ConfigError(FAMILY, f"{at}.kind", f"unknown feed-forward `{kind}`, expected `dense` or `moe`")
    expert, router, shared = _object(mlp, "expert", at), _object(mlp, "router", at), _optional(mlp, "shared", at)
    return ExpertSizes(experts=_need(router, "experts", int, f"{at}.router"), ff=_need(expert, "ff", int, f"{at}.expert"),
                       top=_need(router, "top", int, f"{at}.router"),
                       shared_ff=_need(shared, "ff", int, f"{at}.shared") if shared else 0)


def _check_rotation(rot, most, where):
    if rot is None:
        return
    if rot.dims <= 0 or rot.dims % 2 != 0 or rot.dims > most:
        raise ConfigError(FAMILY, f"{where}.rot.dims", f"must be even and at most {most}")
    positive_finite(FAMILY, f"{where}.rot.base", rot.base)
    if rot.scaling is not None:
        for key in ("factor", "original", "fast", "slow"):
            positive_finite(FAMILY, f"{where}.rot.scaling.{key}", getattr(rot.scaling, key))
        if rot.base == 1.0:
            raise ConfigError(FAMILY, f"{where}.rot.base", "must not be one where the frequencies are rescaled")


@dataclass(frozen=True)
class GavasunConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    loop: Optional[Loop]
    layers: Tuple[GavasunLayer, ...]

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
            layers.append(GavasunLayer(kind, mixer, _mlp(_optional(entry, "mlp", where), f"{where}.mlp")))
        loop = _optional(data, "loop", "")
        if loop:
            loop = Loop(*(_need(loop, key, int, "loop") for key in ("start", "stop", "times")))
        embedding = _optional(data, "embedding", "") or {}
        config = cls(vocab=_need(data, "vocab", int, ""), width=_need(data, "width", int, ""),
                     embedding_scale=take(embedding, FAMILY, "embedding.scale", float, 1.0, ("scale",)),
                     norm_eps=_need(_object(data, "norm", ""), "eps", float, "norm"), loop=loop or None, layers=tuple(layers))
        config.validate()
        return config

    def validate(self):
        positive_extent(FAMILY, "vocab", self.vocab)
        positive_extent(FAMILY, "width", self.width)
        positive_finite(FAMILY, "norm.eps", self.norm_eps)
        if self.embedding_scale != self.embedding_scale or abs(self.embedding_scale) == float("inf"):
            raise ConfigError(FAMILY, "embedding.scale", "must be finite")
        if self.loop is not None:
            if not 0 <= self.loop.start < self.loop.stop <= len(self.layers):
                raise ConfigError(FAMILY, "loop.stop", "start < stop must name layers of the model")
            positive_extent(FAMILY, "loop.times", self.loop.times)
        for index, layer in enumerate(self.layers):
            where, m = f"layers[{index}].mixer", layer.mixer
            keys = {"attention": ("heads", "kv_heads", "dim", "vdim"), "delta": ("heads", "kv_heads", "dim", "vdim", "taps"),
                    "latent_attention": ("heads", "dim", "vdim", "q_rank", "kv_rank")}[layer.type]
            for key in keys:
                positive_extent(FAMILY, f"{where}.{'conv' if key == 'taps' else key}", getattr(m, key))
            if layer.type != "latent_attention" and m.heads % m.kv_heads != 0:
                raise ConfigError(FAMILY, f"{where}.kv_heads", "must divide heads")
            if layer.type != "delta":
                positive_finite(FAMILY, f"{where}.scale", m.scale)
                if (m.chunk if layer.type == "attention" else m.window) < 0:
                    raise ConfigError(FAMILY, f"{where}.mask.size", "must be positive")
            if layer.type == "attention":
                if m.taps < 0:
                    raise ConfigError(FAMILY, f"{where}.conv", "must be positive")
                _check_rotation(m.rot, m.dim, where)
            if layer.type == "latent_attention":
                if m.rot_dim < 0 or m.rot_dim % 2 != 0:
                    raise ConfigError(FAMILY, f"{where}.rot_dim", "must be even")
                if m.rot_dim and m.rot is None:
                    raise ConfigError(FAMILY, f"{where}.rot", "is required where rot_dim is not zero")
                if m.rot is not None and m.rot.dims != m.rot_dim:
                    raise ConfigError(FAMILY, f"{where}.rot.dims", "must equal rot_dim")
                _check_rotation(m.rot, max(m.rot_dim, 2), where)
            e, where = layer.mlp, f"layers[{index}].mlp"
            if isinstance(e, DenseSizes):
                positive_extent(FAMILY, f"{where}.ff", e.ff)
            elif isinstance(e, ExpertSizes):
                for key, name in (("experts", "router.experts"), ("ff", "expert.ff"), ("top", "router.top")):
                    positive_extent(FAMILY, f"{where}.{name}", getattr(e, key))
                if e.top > e.experts:
                    raise ConfigError(FAMILY, f"{where}.router.top", "must not exceed the experts")
                if e.shared_ff < 0:
                    raise ConfigError(FAMILY, f"{where}.shared.ff", "must be positive")

    def runs(self):
        """The layers in the order they run: the looped stretch ``times`` times in a row."""
        count = len(self.layers)
        if self.loop is None:
            return list(range(count))
        stretch = list(range(self.loop.start, self.loop.stop))
        return list(range(self.loop.start)) + stretch * self.loop.times + list(range(self.loop.stop, count))

    def to_dict(self):
        return {"architecture": "Gavasun", "embedding": {"scale": self.embedding_scale},
                "layers": [layer.to_dict() for layer in self.layers], "loop": self.loop.to_dict() if self.loop else None,
                "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
