"""Typed configuration of the Tazitar decoder: a list of pre-norm layers over one residual or several residual
streams, each with a mixer (an attention with q/k norm, rotation and capped scores; a pair of an attention and a
gated delta rule side by side; an attention with interleaved rotation, YaRN scaling and a learned sink) and an optional
gated feed-forward; a run of layers may be repeated with the same weights.

config.json names the design under `architecture` (one string).  Every size and every constant that can differ
between two models of the design is read here and nowhere else: `vocab`, `width`, `norm.eps`, `streams`, `loop`
(`start`, `stop`, `times`), and per layer `type`, `mixer.*` (with `rot.base`, `rot.dims`, `rot.scaling.*`) and `mlp`
(null, or `kind` and `ff`).
"""
from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, Key, read_keys

ARCHITECTURE = "Tazitar"

_TOP = (Key("vocab", int), Key("width", int), Key("norm", dict), Key("layers", list), Key("streams", int, default=None),
        Key("loop", dict, default=None))
_ATTENTION = (Key("heads", int), Key("kv_heads", int, default=None), Key("dim", int), Key("vdim", int),
              Key("scale", float), Key("softcap", float, default=0.0), Key("rot", dict, default=None))
_DELTA = (Key("heads", int), Key("kv_heads", int, default=None), Key("dim", int), Key("vdim", int), Key("conv", int))
_ROT = (Key("base", float), Key("dims", int), Key("scaling", dict, default=None))
_SCALING = (Key("factor", float), Key("original", float), Key("fast", float), Key("slow", float))
_LOOP = (Key("start", int), Key("stop", int), Key("times", int))
_MLP = (Key("kind", str), Key("ff", int))

LAYER_TYPES = ("attention", "parallel", "attention_2")


@dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int
    scaling: tuple | None      # (factor, original, fast, slow) of a YaRN scaling; None: plain frequencies

    def to_dict(self) -> dict:
        body = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            body["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        return body


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float             # 0: scores are not capped
    rot: RotaryConfig | None

    def to_dict(self) -> dict:
        body = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.softcap:
            body["softcap"] = self.softcap
        if self.rot is not None:
            body["rot"] = self.rot.to_dict()
        return body


@dataclass(frozen=True)
class DeltaRuleConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int                  # taps of the short convolutions

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class ParallelConfig:
    left: AttentionConfig
    right: DeltaRuleConfig

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class TazitarLayer:
    type: str                  # one of LAYER_TYPES
    mixer: object
    ff: int | None             # hidden size of the feed-forward; None: the layer has none

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


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


def _read_rot(raw, dim: int, where: str):
    if raw is None:
        return None
    r = _sub(raw, _ROT, where)
    _positive(where, dims=r["dims"])
    if r["dims"] % 2 or r["dims"] > dim:
        raise ConfigError(f"{where}: `dims` must be even and at most the head's `dim`")
    if not r["base"] > 0:
        raise ConfigError(f"{where}: `base` must be positive")
    scaling = None
    if r["scaling"] is not None:
        s = _sub(r["scaling"], _SCALING, where + ".scaling")
        if not (s["factor"] > 0 and s["original"] > 0 and s["fast"] > 0 and s["slow"] > 0) or r["base"] == 1.0:
            raise ConfigError(f"{where}.scaling: factor, original, fast and slow must be positive (and the base not 1)")
        scaling = (s["factor"], s["original"], s["fast"], s["slow"])
    return RotaryConfig(r["base"], r["dims"], scaling)


def _read_attention(raw, where: str) -> AttentionConfig:
    a = _sub(raw, _ATTENTION, where)
    kv = a["kv_heads"] if a["kv_heads"] is not None else a["heads"]
    _positive(where, heads=a["heads"], kv_heads=kv, dim=a["dim"], vdim=a["vdim"])
    if a["heads"] % kv:
        raise ConfigError(f"{where}: heads must be divisible by kv_heads")
    if a["softcap"] < 0:
        raise ConfigError(f"{where}: `softcap` must not be negative")
    return AttentionConfig(a["heads"], kv, a["dim"], a["vdim"], a["scale"], a["softcap"],
                           _read_rot(a["rot"], a["dim"], where + ".rot"))


def _read_delta(raw, where: str) -> DeltaRuleConfig:
    a = _sub(raw, _DELTA, where)
    kv = a["kv_heads"] if a["kv_heads"] is not None else a["heads"]
    _positive(where, heads=a["heads"], kv_heads=kv, dim=a["dim"], vdim=a["vdim"], conv=a["conv"])
    if a["heads"] % kv:
        raise ConfigError(f"{where}: heads must be divisible by kv_heads")
    return DeltaRuleConfig(a["heads"], kv, a["dim"], a["vdim"], a["conv"])


def _read_layer(i: int, raw) -> TazitarLayer:
    where = f"layers[{i}]"
    if not isinstance(raw, dict) or not isinstance(raw.get("mixer"), dict) or not isinstance(raw.get("type"), str):
        raise ConfigError(f"{where}: a layer is an object with `type`, `mixer` and `mlp`")
    kind, m = raw["type"], raw["mixer"]
    if kind in ("attention", "attention_2"):
        mixer = _read_attention(m, where + ".mixer")
    elif kind == "parallel":
        if not isinstance(m.get("left"), dict) or not isinstance(m.get("right"), dict):
            raise ConfigError(f"{where}.mixer: a parallel mixer names `left` and `right`")
        mixer = ParallelConfig(_read_attention(m["left"], where + ".mixer.left"),
                               _read_delta(m["right"], where + ".mixer.right"))
    else:
        raise ConfigError(f"{where}: unknown layer type {kind!r} (known: {', '.join(LAYER_TYPES)})")
    ff = None
    if raw.get("mlp") is not None:
        mlp = _sub(raw["mlp"], _MLP, where + ".mlp")
        if mlp["kind"] != "dense":
            raise ConfigError(f"{where}.mlp: unknown kind {mlp['kind']!r} (known: dense)")
        _positive(where + ".mlp", ff=mlp["ff"])
        ff = mlp["ff"]
    return TazitarLayer(kind, mixer, ff)


@dataclass(frozen=True)
class TazitarConfig:
    vocab: int
    width: int
    eps: float
    streams: int | None        # residual streams with learned connections; None: one plain residual
    loop: tuple | None         # (start, stop, times): layers start..stop-1 run `times` times in a row
    layers: tuple

    architecture = ARCHITECTURE
    eos_token_id = None

    @classmethod
    def from_dict(cls, raw: dict) -> "TazitarConfig":
        top = read_keys(raw, _TOP)
        eps = _sub(top["norm"], (Key("eps", float),), "norm")["eps"]
        if len(top["layers"]) > 65535:
            raise ConfigError(f"{len(top['layers'])} layers: more than 65,535 are not taken")
        loop = None
        if top["loop"] is not None:
            lp = _sub(top["loop"], _LOOP, "loop")
            loop = (lp["start"], lp["stop"], lp["times"])
        config = cls(top["vocab"], top["width"], eps, top["streams"], loop,
                     tuple(_read_layer(i, layer) for i, layer in enumerate(top["layers"])))
        config.validate()
        return config

    def validate(self) -> None:
        _positive("config.json", vocab=self.vocab, width=self.width)
        if not self.eps >= 0.0:
            raise ConfigError("norm.eps must not be negative")
        if not self.layers:
            raise ConfigError("`layers` must name at least one layer")
        if self.streams is not None and not 1 <= self.streams <= 16:
            raise ConfigError("`streams` must be between 1 and 16")
        if self.loop is not None:
            start, stop, times = self.loop
            if not 0 <= start <= stop <= len(self.layers):
                raise ConfigError("loop: `start` and `stop` must lie within the layers, start <= stop")
            if times < 0 or times * max(stop - start, 0) > 65535:
                raise ConfigError("loop: `times` must not be negative, and the passes at most 65,535 layer runs")

    def layer_order(self) -> list:
        """The layers in the order they run, a repeated one once for every pass."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        start, stop, times = self.loop
        return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))

    def to_dict(self) -> dict:
        """A config.json body that `from_dict` reads back to an equal object."""
        body = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "layers": [layer.to_dict() for layer in self.layers]}
        if self.streams is not None:
            body["streams"] = self.streams
        if self.loop is not None:
            body["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        return body
