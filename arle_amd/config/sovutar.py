"""Typed configuration of the Sovutar decoder: a list of layers, each with a mixer (a chunked attention without
positions, or a latent attention over a sliding window) and an optional mixture-of-experts feed-forward, read from
nested config.json keys.

config.json names the design under `architecture` (one string).  Every size and every constant that can differ
between two models of the design is read here and nowhere else: `vocab`, `width`, `norm.eps`, `logit_softcap`, and
per layer `type`, `mixer.*` and `mlp` (null, or `kind`, `expert.ff`, `router.*`, `shared.ff`).
"""
from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, Key, read_keys

ARCHITECTURE = "Sovutar"

_TOP = (Key("vocab", int), Key("width", int), Key("norm", dict), Key("layers", list),
        Key("logit_softcap", float, default=0.0))
_ATTENTION = (Key("heads", int), Key("kv_heads", int, default=None), Key("dim", int), Key("vdim", int), Key("scale", float),
              Key("mask", dict, default=None), Key("v_mix", bool, default=False))
_LATENT = (Key("heads", int), Key("dim", int), Key("rot_dim", int), Key("vdim", int), Key("kv_rank", int),
           Key("scale", float), Key("mask", dict, default=None), Key("rot", dict))
_ROT = (Key("base", float), Key("dims", int))
_MLP = (Key("kind", str), Key("expert", dict), Key("router", dict), Key("shared", dict, default=None))
_ROUTER = (Key("experts", int), Key("top", int), Key("scale", float, default=1.0))


@dataclass(frozen=True)
class ChunkedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int | None          # mask.size: a row sees the keys of its own chunk; None: every earlier key
    v_mix: bool

    def to_dict(self) -> dict:
        body = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                "scale": self.scale, "v_mix": self.v_mix}
        if self.chunk is not None:
            body["mask"] = {"size": self.chunk}
        return body


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int | None         # mask.size: a row sees itself and the window - 1 keys before it; None: all
    rot_base: float
    rot_dims: int

    def to_dict(self) -> dict:
        body = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                "kv_rank": self.kv_rank, "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.window is not None:
            body["mask"] = {"size": self.window}
        return body


@dataclass(frozen=True)
class MoEConfig:
    experts: int
    top: int
    scale: float
    expert_ff: int
    shared_ff: int | None

    def to_dict(self) -> dict:
        return {"kind": "moe", "expert": {"ff": self.expert_ff},
                "router": {"experts": self.experts, "top": self.top, "scale": self.scale},
                "shared": None if self.shared_ff is None else {"ff": self.shared_ff}}


@dataclass(frozen=True)
class SovutarLayer:
    type: str                  # "attention" | "latent_attention"
    mixer: object
    mlp: MoEConfig | None

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


def _positive(where: str, **values) -> None:
    for name, v in values.items():
        if v <= 0:
            raise ConfigError(f"{where}: `{name}` must be positive")
        if v > 2 ** 31 - 1:
            raise ConfigError(f"{where}: `{name}` = {v} is beyond what a 32-bit index reaches")


def _sub(raw, keys, where: str) -> dict:
    try:
        return read_keys(raw, keys)
    except ConfigError as exc:
        raise ConfigError(f"{where}: {exc}") from None


def _mask_size(raw, where: str):
    if raw is None:
        return None
    size = _sub(raw, (Key("size", int),), where + ".mask")["size"]
    _positive(where, **{"mask.size": size})
    return size


def _read_mlp(raw, where: str):
    if raw is None:
        return None
    if not isinstance(raw, dict):
        raise ConfigError(f"{where}: null or an object with `kind`, `expert` and `router`")
    m = _sub(raw, _MLP, where)
    if m["kind"] != "moe":
        raise ConfigError(f"{where}: unknown kind {m['kind']!r} (known: moe)")
    r = _sub(m["router"], _ROUTER, where + ".router")
    ff = _sub(m["expert"], (Key("ff", int),), where + ".expert")["ff"]
    shared = _sub(m["shared"], (Key("ff", int),), where + ".shared")["ff"] if m["shared"] is not None else None
    _positive(where, experts=r["experts"], top=r["top"], **{"expert.ff": ff})
    if shared is not None:
        _positive(where, **{"shared.ff": shared})
    if r["top"] > r["experts"]:
        raise ConfigError(f"{where}: `top` = {r['top']} is more than the {r['experts']} experts")
    return MoEConfig(r["experts"], r["top"], r["scale"], ff, shared)


def _read_layer(i: int, raw) -> SovutarLayer:
    where = f"layers[{i}]"
    if not isinstance(raw, dict) or not isinstance(raw.get("mixer"), dict) or not isinstance(raw.get("type"), str):
        raise ConfigError(f"{where}: a layer is an object with `type`, `mixer` and `mlp`")
    kind, m = raw["type"], raw["mixer"]
    if kind == "attention":
        a = _sub(m, _ATTENTION, where + ".mixer")
        # without `kv_heads` every q head has key and value heads of its own
        mixer = ChunkedAttentionConfig(a["heads"], a["kv_heads"] if a["kv_heads"] is not None else a["heads"], a["dim"],
                                       a["vdim"], a["scale"],
                                       _mask_size(a["mask"], where + ".mixer"), a["v_mix"])
        _positive(where, heads=mixer.heads, kv_heads=mixer.kv_heads, dim=mixer.dim, vdim=mixer.vdim)
        if mixer.heads % mixer.kv_heads:
            raise ConfigError(f"{where}: heads must be divisible by kv_heads")
    elif kind == "latent_attention":
        a = _sub(m, _LATENT, where + ".mixer")
        rot = _sub(a["rot"], _ROT, where + ".mixer.rot")
        mixer = LatentAttentionConfig(a["heads"], a["dim"], a["rot_dim"], a["vdim"], a["kv_rank"], a["scale"],
                                      _mask_size(a["mask"], where + ".mixer"), rot["base"], rot["dims"])
        _positive(where, heads=mixer.heads, dim=mixer.dim, rot_dim=mixer.rot_dim, vdim=mixer.vdim,
                  kv_rank=mixer.kv_rank, **{"rot.dims": mixer.rot_dims})
        if mixer.rot_dims % 2 or mixer.rot_dims > mixer.rot_dim:
            raise ConfigError(f"{where}: `rot.dims` must be even and at most `rot_dim`")
        if not mixer.rot_base > 0:
            raise ConfigError(f"{where}: `rot.base` must be positive")
    else:
        raise ConfigError(f"{where}: unknown layer type {kind!r} (known: attention, latent_attention)")
    return SovutarLayer(kind, mixer, _read_mlp(raw.get("mlp"), where + ".mlp"))


@dataclass(frozen=True)
class SovutarConfig:
    vocab: int
    width: int
    eps: float
    logit_softcap: float       # 0: the logits are not capped
    layers: tuple

    architecture = ARCHITECTURE
    eos_token_id = None

    @classmethod
    def from_dict(cls, raw: dict) -> "SovutarConfig":
        top = read_keys(raw, _TOP)
        eps = _sub(top["norm"], (Key("eps", float),), "norm")["eps"]
        if len(top["layers"]) > 65535:
            raise ConfigError(f"{len(top['layers'])} layers: more than 65,535 are not taken")
        config = cls(top["vocab"], top["width"], eps, top["logit_softcap"],
                     tuple(_read_layer(i, layer) for i, layer in enumerate(top["layers"])))
        config.validate()
        return config

    def validate(self) -> None:
        _positive("config.json", vocab=self.vocab, width=self.width)
        if not self.eps >= 0.0:
            raise ConfigError("norm.eps must not be negative")
        if self.logit_softcap < 0.0:
            raise ConfigError("logit_softcap must not be negative")
        if not self.layers:
            raise ConfigError("`layers` must name at least one layer")
        first = self.first_value_mixer()
        if first is not None:
            a = self.layers[first].mixer
            for i, layer in enumerate(self.layers):
                m = layer.mixer
                if isinstance(m, ChunkedAttentionConfig) and m.v_mix and (m.kv_heads, m.vdim) != (a.kv_heads, a.vdim):
                    raise ConfigError(f"layers[{i}]: its values ({m.kv_heads} heads of {m.vdim}) cannot be mixed with "
                                      f"those of layer {first} ({a.kv_heads} heads of {a.vdim})")

    def first_value_mixer(self):
        """The first layer whose configuration says `v_mix`: the others mix its values into theirs."""
        for i, layer in enumerate(self.layers):
            if isinstance(layer.mixer, ChunkedAttentionConfig) and layer.mixer.v_mix:
                return i
        return None

    def to_dict(self) -> dict:
        """A config.json body that `from_dict` reads back to an equal object."""
        return {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "logit_softcap": self.logit_softcap, "layers": [layer.to_dict() for layer in self.layers]}
