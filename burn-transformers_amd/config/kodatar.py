"""Kodatar's typed configuration, read from the keys of its own config.json.

    architecture     "Kodatar"
    vocab, width     sizes of the token table
    embedding.scale  factor on the token's row of the table
    logit_scale      factor on the logits
    norm.eps         the epsilon of every norm of the model (layer norms and head norms)
    loop             null / absent, or {start, stop, times}: layers start .. stop - 1 run ``times`` times
                     in a row with the same tensors, every pass with a cache of its own
    layers           a list; each entry has ``type`` ("attention"), ``mixer`` (dim, vdim, heads, kv_heads,
                     scale, rot {dims, base, scaling: null or {factor, low, high, original}}, mask: null
                     or {size}) and ``mlp``: null, or {kind: "moe", expert {ff}, router {experts, top,
                     identity, groups: null or {count, keep}}, shared: null or {ff}}

Every size and constant of a model is one of these keys or a tensor's shape.
"""

from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError, MAX_LAYERS, positive_extent, positive_finite, take

FAMILY = "kodatar"


def _need(data, field, kind, where):
    full = f"{where}.{field}" if where else field
    if not isinstance(data, dict) or field not in data or data[field] is None:
        raise ConfigError(FAMILY, full, "is required")
    return take({full: data[field]}, FAMILY, full, kind, None)


def _optional(data, field, where):
    """A nested object that may be absent or null."""
    value = data.get(field)
    if value is not None and not isinstance(value, dict):
        raise ConfigError(FAMILY, f"{where}.{field}", "must be an object or null")
    return value


@dataclass(frozen=True)
class RotaryScaling:
    factor: float
    low: float
    high: float
    original: int

    def to_dict(self):
        return {"factor": self.factor, "low": self.low, "high": self.high, "original": self.original}


@dataclass(frozen=True)
class KodatarMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float
    rot_scaling: Optional[RotaryScaling]
    chunk: int                                   # mask.size; 0: every earlier position is seen

    def to_dict(self):
        return {"dim": self.dim, "vdim": self.vdim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale,
                "rot": {"dims": self.rot_dims, "base": self.rot_base,
                        "scaling": self.rot_scaling.to_dict() if self.rot_scaling else None},
                "mask": {"size": self.chunk} if self.chunk else None}


@dataclass(frozen=True)
class KodatarExperts:
    experts: int
    ff: int
    top: int
    identity: int
    groups: int                                  # 0: no groups
    keep: int
    shared_ff: int                               # 0: no shared expert

    def to_dict(self):
        return {"kind": "moe", "expert": {"ff": self.ff},
                "router": {"experts": self.experts, "top": self.top, "identity": self.identity,
                           "groups": {"count": self.groups, "keep": self.keep} if self.groups else None},
                "shared": {"ff": self.shared_ff} if self.shared_ff else None}


@dataclass(frozen=True)
class KodatarLayer:
    mixer: KodatarMixer
    mlp: Optional[KodatarExperts]

    def to_dict(self):
        return {"type": "attention", "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


@dataclass(frozen=True)
class KodatarLoop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class KodatarConfig:
    vocab: int
    width: int
    embedding_scale: float
    logit_scale: float
    norm_eps: float
    loop: Optional[KodatarLoop]
    layers: Tuple[KodatarLayer, ...]

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
            if kind != "attention":
                raise ConfigError(FAMILY, f"{where}.type", f"unknown mixer `{kind}`, expected `attention`")
            m, at = entry.get("mixer"), f"{where}.mixer"
            if not isinstance(m, dict):
                raise ConfigError(FAMILY, at, "must be an object with the mixer's sizes")
            rot = _optional(m, "rot", at)
            scaling = _optional(rot, "scaling", f"{at}.rot") if rot else None
            mask = _optional(m, "mask", at)
            mixer = KodatarMixer(
                heads=_need(m, "heads", int, at), kv_heads=_need(m, "kv_heads", int, at), dim=_need(m, "dim", int, at),
                vdim=_need(m, "vdim", int, at), scale=_need(m, "scale", float, at),
                rot_dims=_need(rot, "dims", int, f"{at}.rot") if rot else 0,
                rot_base=_need(rot, "base", float, f"{at}.rot") if rot else 1.0,
                rot_scaling=RotaryScaling(*(_need(scaling, key, of, f"{at}.rot.scaling") for key, of in
                                            (("factor", float), ("low", float), ("high", float), ("original", int))))
                if scaling else None,
                chunk=_need(mask, "size", int, f"{at}.mask") if mask else 0)
            mlp, at = _optional(entry, "mlp", where), f"{where}.mlp"
            experts = None
            if mlp is not None:
                if _need(mlp, "kind", str, at) != "moe":
                    raise ConfigError(FAMILY, f"{at}.kind", f"unknown feed-forward `{mlp['kind']}`, expected `moe`")
                router, shared = mlp.get("router"), _optional(mlp, "shared", at)
                groups = _optional(router, "groups", f"{at}.router") if isinstance(router, dict) else None
                experts = KodatarExperts(
                    experts=_need(router, "experts", int, f"{at}.router"), ff=_need(mlp.get("expert"), "ff", int, f"{at}.expert"),
                    top=_need(router, "top", int, f"{at}.router"),
                    identity=take(router, FAMILY, f"{at}.router.identity", int, 0, ("identity",)),
                    groups=_need(groups, "count", int, f"{at}.router.groups") if groups else 0,
                    keep=_need(groups, "keep", int, f"{at}.router.groups") if groups else 0,
                    shared_ff=_need(shared, "ff", int, f"{at}.shared") if shared else 0)
            layers.append(KodatarLayer(mixer, experts))
        loop = _optional(data, "loop", "")
        config = cls(vocab=_need(data, "vocab", int, ""), width=_need(data, "width", int, ""),
                     embedding_scale=_need(data.get("embedding"), "scale", float, "embedding"),
                     logit_scale=_need(data, "logit_scale", float, ""), norm_eps=_need(data.get("norm"), "eps", float, "norm"),
                     loop=KodatarLoop(*(_need(loop, key, int, "loop") for key in ("start", "stop", "times"))) if loop else None,
                     layers=tuple(layers))
        config.validate()
        return config

    def validate(self):
        positive_extent(FAMILY, "vocab", self.vocab)
        positive_extent(FAMILY, "width", self.width)
        positive_finite(FAMILY, "norm.eps", self.norm_eps)
        for name, value in (("embedding.scale", self.embedding_scale), ("logit_scale", self.logit_scale)):
            if value != value or abs(value) == float("inf"):
                raise ConfigError(FAMILY, name, "must be finite")
        if self.loop is not None:
            if not (0 <= self.loop.start < self.loop.stop <= len(self.layers)):
                raise ConfigError(FAMILY, "loop", f"layers {self.loop.start} .. {self.loop.stop} - 1 are not layers of the model")
            positive_extent(FAMILY, "loop.times", self.loop.times)
        for index, layer in enumerate(self.layers):
            m, where = layer.mixer, f"layers[{index}].mixer"
            for key in ("heads", "kv_heads", "dim", "vdim"):
                positive_extent(FAMILY, f"{where}.{key}", getattr(m, key))
            positive_finite(FAMILY, f"{where}.scale", m.scale)
            if m.heads % m.kv_heads != 0:
                raise ConfigError(FAMILY, f"{where}.kv_heads", "must divide heads")
            if m.rot_dims < 0 or m.rot_dims % 2 != 0 or m.rot_dims > m.dim:
                raise ConfigError(FAMILY, f"{where}.rot.dims", "must be even and at most dim")
            if m.rot_dims:
                positive_finite(FAMILY, f"{where}.rot.base", m.rot_base)
            if m.rot_scaling is not None:
                s = m.rot_scaling
                positive_finite(FAMILY, f"{where}.rot.scaling.factor", s.factor)
                positive_extent(FAMILY, f"{where}.rot.scaling.original", s.original)
                if not (s.high > s.low > 0):
                    raise ConfigError(FAMILY, f"{where}.rot.scaling", "needs high > low > 0")
            if m.chunk < 0:
                raise ConfigError(FAMILY, f"{where}.mask.size", "must be positive")
            e, where = layer.mlp, f"layers[{index}].mlp"
            if e is None:
                continue
            for key, name in (("experts", "router.experts"), ("ff", "expert.ff"), ("top", "router.top")):
                positive_extent(FAMILY, f"{where}.{name}", getattr(e, key))
            if e.identity < 0 or e.shared_ff < 0:
                raise ConfigError(FAMILY, f"{where}.router.identity", "must not be negative")
            outputs = e.experts + e.identity
            if e.top > outputs:
                raise ConfigError(FAMILY, f"{where}.router.top", "must not exceed the experts and identity experts together")
            if e.groups:
                if outputs % e.groups != 0:
                    raise ConfigError(FAMILY, f"{where}.router.groups.count", "must divide the experts and identity experts together")
                if not (0 < e.keep <= e.groups) or e.keep * (outputs // e.groups) < e.top:
                    raise ConfigError(FAMILY, f"{where}.router.groups.keep", "the groups that stay open must hold `top` experts")

    def runs(self):
        """[(layer, pass or None)] in the order the layers run; ``pass`` is the number of the pass that
        the run opens (the first layer of the loop, once per pass), else None."""
        order = []
        loop = self.loop
        if loop is None:
            return [(index, None) for index in range(len(self.layers))]
        order += [(index, None) for index in range(loop.start)]
        for number in range(loop.times):
            order += [(index, number if index == loop.start else None) for index in range(loop.start, loop.stop)]
        order += [(index, None) for index in range(loop.stop, len(self.layers))]
        return order

    def to_dict(self):
        data = {"architecture": "Kodatar", "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale,
                "norm": {"eps": self.norm_eps}, "layers": [layer.to_dict() for layer in self.layers]}
        if self.loop is not None:
            data["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return data
