"""Typed configuration of the Gufasun decoder: a list of layers, each with a mixer (windowed soft-capped
attention, or an mLSTM matrix memory) and an optional dense feed-forward, read from nested config.json keys.

config.json names the design under `architecture` (one string).  Every size and every constant that can differ
between two models of the design is read here and nowhere else: `vocab`, `width`, `norm.eps`, `embedding.scale`,
`canon.taps`, and per layer `type`, `mixer.*` and `mlp` (null, or `kind` and `ff`).
"""
from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, Key, read_keys

ARCHITECTURE = "Gufasun"

_TOP = (Key("vocab", int), Key("width", int), Key("norm", dict), Key("embedding", dict), Key("canon", dict),
        Key("layers", list))
_ATTENTION = (Key("heads", int), Key("kv_heads", int), Key("dim", int), Key("vdim", int), Key("scale", float),
              Key("softcap", float, default=0.0), Key("conv", int, default=0), Key("mask", dict, default=None),
              Key("q_temp", dict, default=None), Key("kv_from", int, default=None))
_MLSTM = (Key("heads", int), Key("dim", int), Key("vdim", int), Key("gate_cap", float))
_MLP = (Key("kind", str), Key("ff", int))


@dataclass(frozen=True)
class AttentionMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float
    conv: int                      # taps of the convolutions on q, k and v; 0: none
    window: int | None             # mask.size
    temp_coef: float               # q_temp.coef; 0: no temperature
    temp_every: int                # q_temp.every
    kv_from: int | None            # the layer whose keys and values this one reads

    def to_dict(self) -> dict:
        body = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "softcap": self.softcap, "conv": self.conv}
        if self.window is not None:
            body["mask"] = {"size": self.window}
        body["q_temp"] = {"coef": self.temp_coef, "every": self.temp_every}
        if self.kv_from is not None:
            body["kv_from"] = self.kv_from
        return body


@dataclass(frozen=True)
class MLSTMMixerConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class GufasunLayer:
    type: str                      # "attention" | "mlstm"
    mixer: object
    ff: int | None                 # hidden size of the dense feed-forward; None: the layer has none

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


def _positive(where: str, **values) -> None:
    for name, v in values.items():
        if v <= 0:
            raise ConfigError(f"{where}: `{name}` must be positive")
        if v > 2 ** 31 - 1:
            raise ConfigError(f"{where}: `{name}` = {v} is beyond what a 32-bit index reaches")


def _sub(raw: dict, keys, where: str) -> dict:
    try:
        return read_keys(raw, keys)
    except ConfigError as exc:
        raise ConfigError(f"{where}: {exc}") from None


def _read_layer(i: int, raw) -> GufasunLayer:
    where = f"layers[{i}]"
    if not isinstance(raw, dict) or not isinstance(raw.get("mixer"), dict) or not isinstance(raw.get("type"), str):
        raise ConfigError(f"{where}: a layer is an object with `type`, `mixer` and `mlp`")
    kind, m = raw["type"], raw["mixer"]
    if kind == "attention":
        a = _sub(m, _ATTENTION, where + ".mixer")
        mask = _sub(a["mask"], (Key("size", int),), where + ".mixer.mask") if a["mask"] is not None else None
        temp = (_sub(a["q_temp"], (Key("coef", float), Key("every", int)), where + ".mixer.q_temp")
                if a["q_temp"] is not None else {"coef": 0.0, "every": 1})
        mixer = AttentionMixer(a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["scale"], a["softcap"], a["conv"],
                               mask["size"] if mask else None, temp["coef"], temp["every"], a["kv_from"])
        _positive(where, heads=mixer.heads, kv_heads=mixer.kv_heads, dim=mixer.dim, vdim=mixer.vdim,
                  every=mixer.temp_every)
        if mixer.heads % mixer.kv_heads:
            raise ConfigError(f"{where}: heads must be divisible by kv_heads")
        if mixer.window is not None:
            _positive(where, **{"mask.size": mixer.window})
        if mixer.conv < 0 or mixer.softcap < 0:
            raise ConfigError(f"{where}: `conv` and `softcap` must not be negative")
    elif kind == "mlstm":
        mixer = MLSTMMixerConfig(**_sub(m, _MLSTM, where + ".mixer"))
        _positive(where, heads=mixer.heads, dim=mixer.dim, vdim=mixer.vdim)
        if not mixer.gate_cap > 0:
            raise ConfigError(f"{where}: `gate_cap` must be positive")
    else:
        raise ConfigError(f"{where}: unknown layer type {kind!r} (known: attention, mlstm)")
    ff = None
    if raw.get("mlp") is not None:
        if not isinstance(raw["mlp"], dict):
            raise ConfigError(f"{where}.mlp: null or an object with `kind` and `ff`")
        mlp = _sub(raw["mlp"], _MLP, where + ".mlp")
        if mlp["kind"] != "dense":
            raise ConfigError(f"{where}.mlp: unknown kind {mlp['kind']!r} (known: dense)")
        ff = mlp["ff"]
        _positive(where + ".mlp", ff=ff)
    return GufasunLayer(kind, mixer, ff)


@dataclass(frozen=True)
class GufasunConfig:
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    canon_taps: int
    layers: tuple

    architecture = ARCHITECTURE
    eos_token_id = None

    @classmethod
    def from_dict(cls, raw: dict) -> "GufasunConfig":
        top = read_keys(raw, _TOP)
        eps = _sub(top["norm"], (Key("eps", float),), "norm")["eps"]
        scale = _sub(top["embedding"], (Key("scale", float, default=1.0),), "embedding")["scale"]
        taps = _sub(top["canon"], (Key("taps", int),), "canon")["taps"]
        if len(top["layers"]) > 65535:
            raise ConfigError(f"{len(top['layers'])} layers: more than 65,535 are not taken")
        config = cls(top["vocab"], top["width"], eps, scale, taps,
                     tuple(_read_layer(i, layer) for i, layer in enumerate(top["layers"])))
        config.validate()
        return config

    def validate(self) -> None:
        _positive("config.json", vocab=self.vocab, width=self.width, **{"canon.taps": self.canon_taps})
        if not self.eps >= 0.0:
            raise ConfigError("norm.eps must not be negative")
        if not self.layers:
            raise ConfigError("`layers` must name at least one layer")
        for i, layer in enumerate(self.layers):
            j = getattr(layer.mixer, "kv_from", None)
            if j is None:
                continue
            owner = self.layers[j].mixer if 0 <= j < i else None
            if not isinstance(owner, AttentionMixer) or owner.kv_from is not None:
                raise ConfigError(f"layers[{i}]: kv_from = {j} must name an earlier attention layer with keys and "
                                  "values of its own")
            if (owner.kv_heads, owner.dim, owner.vdim) != (layer.mixer.kv_heads, layer.mixer.dim, layer.mixer.vdim):
                raise ConfigError(f"layers[{i}]: its key/value heads and sizes differ from those of layer {j}, "
                                  "whose keys and values it reads")

    def to_dict(self) -> dict:
        """A config.json body that `from_dict` reads back to an equal object."""
        return {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "embedding": {"scale": self.embedding_scale}, "canon": {"taps": self.canon_taps},
                "layers": [layer.to_dict() for layer in self.layers]}

    def cache_window(self, i: int):
        """Keys that layer i's pages keep: its own window or the widest of the layers that read its pages (None:
        all of them)."""
        windows = [self.layers[i].mixer.window] + [l.mixer.window for l in self.layers
                                                   if getattr(l.mixer, "kv_from", None) == i]
        return None if any(w is None for w in windows) else max(windows)
