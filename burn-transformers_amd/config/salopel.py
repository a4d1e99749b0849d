"""Salopel's typed configuration, read from the keys of its own config.json.

    architecture   "Salopel"
    vocab, width   sizes of the token table
    residual_mult  factor on every normalised sublayer output before it joins the stream
    norm.eps       the epsilon of every norm of the model
    layers         a list; each entry has ``type`` (latent_attention | mamba1 | mamba2), ``mixer`` (the
                   mixer's sizes), ``mlp`` ({"kind": "dense", "ff": n} or null) and optionally
                   ``weights_of``: the index of another layer whose tensors it runs (with a cache
                   or state of its own)

Every size and constant of a model is one of these keys or a tensor's shape; nothing has a default.
"""

from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError, MAX_LAYERS, positive_extent, positive_finite, take

FAMILY = "salopel"

MIXER_KEYS = {
    "latent_attention": {"heads": int, "dim": int, "vdim": int, "q_rank": int, "kv_rank": int, "scale": float},
    "mamba1": {"inner": int, "state": int, "dt_rank": int, "conv": int},
    "mamba2": {"heads": int, "vdim": int, "state": int, "groups": int, "norm_groups": int, "conv": int},
}


@dataclass(frozen=True)
class SalopelLayer:
    type: str
    mixer: Tuple[Tuple[str, object], ...]        # the mixer's sizes as sorted (key, value) pairs
    ff: Optional[int]                            # inner width of the dense feed-forward; None: no feed-forward
    weights_of: Optional[int]

    @property
    def sizes(self):
        return dict(self.mixer)

    def to_dict(self):
        data = {"type": self.type, "mixer": dict(self.mixer),
                "mlp": {"kind": "dense", "ff": self.ff} if self.ff is not None else None}
        if self.weights_of is not None:
            data["weights_of"] = self.weights_of
        return data


def _need(data, field, kind, where):
    if field not in data or data[field] is None:
        raise ConfigError(FAMILY, f"{where}.{field}" if where else field, "is required")
    # ``take`` names the field it checks: hand it the value under the full name
    full = f"{where}.{field}" if where else field
    return take({full: data[field]}, FAMILY, full, kind, None)


@dataclass(frozen=True)
class SalopelConfig:
    vocab: int
    width: int
    residual_mult: float
    norm_eps: float
    layers: Tuple[SalopelLayer, ...]

    @classmethod
    def from_dict(cls, data):
        if not isinstance(data.get("layers"), (list, tuple)) or not data["layers"]:
            raise ConfigError(FAMILY, "layers", "must be a list with at least one layer")
        if len(data["layers"]) > MAX_LAYERS:
            raise ConfigError(FAMILY, "layers", f"must not exceed {MAX_LAYERS} entries")
        norm = data.get("norm")
        if not isinstance(norm, dict):
            raise ConfigError(FAMILY, "norm", "must be an object with `eps`")
        layers = []
        for index, entry in enumerate(data["layers"]):
            where = f"layers[{index}]"
            if not isinstance(entry, dict):
                raise ConfigError(FAMILY, where, "must be an object")
            kind = _need(entry, "type", str, where)
            if kind not in MIXER_KEYS:
                raise ConfigError(FAMILY, f"{where}.type", f"unknown mixer `{kind}`, expected one of "
                                  + ", ".join(f"`{k}`" for k in sorted(MIXER_KEYS)))
            if not isinstance(entry.get("mixer"), dict):
                raise ConfigError(FAMILY, f"{where}.mixer", "must be an object with the mixer's sizes")
            sizes = {key: _need(entry["mixer"], key, of, f"{where}.mixer") for key, of in MIXER_KEYS[kind].items()}
            mlp, ff = entry.get("mlp"), None
            if mlp is not None:
                if not isinstance(mlp, dict):
                    raise ConfigError(FAMILY, f"{where}.mlp", "must be an object or null")
                if _need(mlp, "kind", str, f"{where}.mlp") != "dense":
                    raise ConfigError(FAMILY, f"{where}.mlp.kind", f"unknown feed-forward `{mlp['kind']}`, expected `dense`")
                ff = _need(mlp, "ff", int, f"{where}.mlp")
            owner = take(entry, FAMILY, f"{where}.weights_of", int, None, ("weights_of",))
            layers.append(SalopelLayer(kind, tuple(sorted(sizes.items())), ff, owner))
        config = cls(vocab=_need(data, "vocab", int, ""), width=_need(data, "width", int, ""),
                     residual_mult=_need(data, "residual_mult", float, ""), norm_eps=_need(norm, "eps", float, "norm"),
                     layers=tuple(layers))
        config.validate()
        return config

    def validate(self):
        positive_extent(FAMILY, "vocab", self.vocab)
        positive_extent(FAMILY, "width", self.width)
        positive_finite(FAMILY, "norm.eps", self.norm_eps)
        if self.residual_mult != self.residual_mult or abs(self.residual_mult) == float("inf"):
            raise ConfigError(FAMILY, "residual_mult", "must be finite")
        for index, layer in enumerate(self.layers):
            where = f"layers[{index}]"
            sizes = layer.sizes
            for key, value in sizes.items():
                if key == "scale":
                    positive_finite(FAMILY, f"{where}.mixer.scale", value)
                else:
                    positive_extent(FAMILY, f"{where}.mixer.{key}", value)
            if layer.ff is not None:
                positive_extent(FAMILY, f"{where}.mlp.ff", layer.ff)
            if layer.type == "mamba2":
                if sizes["heads"] % sizes["groups"] != 0:
                    raise ConfigError(FAMILY, f"{where}.mixer.groups", "must divide heads")
                if (sizes["heads"] * sizes["vdim"]) % sizes["norm_groups"] != 0:
                    raise ConfigError(FAMILY, f"{where}.mixer.norm_groups", "must divide heads * vdim")
            if layer.weights_of is not None:
                if not (0 <= layer.weights_of < len(self.layers)) or layer.weights_of == index:
                    raise ConfigError(FAMILY, f"{where}.weights_of", "must name another layer of the model")
                owner = self.owner(index)
                if owner is None:
                    raise ConfigError(FAMILY, f"{where}.weights_of", "leads round in a circle: no layer of it has tensors")
                held = self.layers[owner]
                if (held.type, held.mixer, held.ff) != (layer.type, layer.mixer, layer.ff):
                    raise ConfigError(FAMILY, f"{where}.weights_of", f"differs from layer {owner}, whose tensors it runs")

    def owner(self, index):
        """The layer whose tensors layer ``index`` runs: itself unless it borrows; a borrower may come
        before or after its owner, and may name another borrower (None if that leads round in a circle)."""
        seen = set()
        while self.layers[index].weights_of is not None:
            if index in seen:
                return None
            seen.add(index)
            index = self.layers[index].weights_of
        return index

    def to_dict(self):
        return {"architecture": "Salopel", "vocab": self.vocab, "width": self.width,
                "residual_mult": self.residual_mult, "norm": {"eps": self.norm_eps},
                "layers": [layer.to_dict() for layer in self.layers]}
