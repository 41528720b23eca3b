"""Typed configuration of the Retudra decoder: a list of layers whose sublayers read the residual itself and whose
layer norms (weight and bias) stand on the sublayers' outputs, each added times one factor of the model.  A layer has
a mixer (a windowed attention that keeps the first keys, with q and k normed over the whole projection and a
rotate-half rotation; a latent attention with a gate on its heads' outputs; a gated delta rule with a decay for every
key channel), an optional feed-forward (gated dense, or a mixture of experts with a softmax router, grouped choice and
experts that hand back their input) and, where the model has one, a token-side input from a second embedding.

config.json names the design under `architecture` (one string).  Every size and every constant that can differ
between two models of the design is read here and nowhere else: `vocab`, `width`, `norm.eps`, `residual_mult`,
`token_side.dim`, `logit_softcap`, and per layer `type`, `mixer.*` (with `mask.size`, `mask.keep_first`, `rot.base`,
`rot.dims`) and `mlp` (null, or `kind` with `ff`, or with `expert.ff` and `router.experts|top|identity|groups.*`).
The widths of the narrow middles of the delta rule's decay and gate projections are the tensors' own; `decay_rank`
and `gate_rank` name them where a model is made from nothing.
"""
from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, Key, read_keys

ARCHITECTURE = "Retudra"

_TOP = (Key("vocab", int), Key("width", int), Key("norm", dict), Key("layers", list),
        Key("residual_mult", float, default=1.0), Key("token_side", dict, default=None),
        Key("logit_softcap", float, default=None))
_ROT = (Key("base", float), Key("dims", int))
_MASK = (Key("size", int), Key("keep_first", int, default=0))
_ATTENTION = (Key("heads", int), Key("kv_heads", int, default=None), Key("dim", int), Key("vdim", int),
              Key("scale", float), Key("rot", dict, default=None), Key("mask", dict, default=None))
_LATENT = (Key("heads", int), Key("dim", int), Key("rot_dim", int), Key("vdim", int), Key("kv_rank", int),
           Key("scale", float), Key("rot", dict))
_DELTA = (Key("heads", int), Key("kv_heads", int, default=None), Key("dim", int), Key("vdim", int), Key("conv", int),
          Key("decay_rank", int, default=None), Key("gate_rank", int, default=None))
_MLP = (Key("kind", str), Key("ff", int, default=None), Key("expert", dict, default=None), Key("router", dict, default=None))
_ROUTER = (Key("experts", int), Key("top", int), Key("identity", int, default=0), Key("groups", dict, default=None))
_GROUPS = (Key("count", int), Key("keep", int))

LAYER_TYPES = ("attention", "latent_attention", "channel_delta")
MLP_KINDS = ("dense", "moe")


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


@dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int

    def to_dict(self) -> dict:
        return {"base": self.base, "dims": self.dims}


def _read_rot(raw, most: int, where: str):
    if raw is None:
        return None
    r = _sub(raw, _ROT, where)
    _positive(where, dims=r["dims"])
    if r["dims"] % 2 or r["dims"] > most:
        raise ConfigError(f"{where}: `dims` must be even and at most the size of what is rotated ({most})")
    if not r["base"] > 0:
        raise ConfigError(f"{where}: `base` must be positive")
    return RotaryConfig(r["base"], r["dims"])


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotaryConfig | None
    window: int | None         # mask.size; None: every earlier key is seen
    keep_first: int            # mask.keep_first: the first keys that stay visible behind the window

    def to_dict(self) -> dict:
        body = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot is not None:
            body["rot"] = self.rot.to_dict()
        if self.window is not None:
            body["mask"] = {"size": self.window, "keep_first": self.keep_first}
        return body


@dataclass(frozen=True)
class LatentConfig:
    heads: int
    dim: int                   # unrotated query/key entries a head
    rot_dim: int               # rotated ones (the key's are shared by the heads)
    vdim: int
    kv_rank: int
    scale: float
    rot: RotaryConfig

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                "scale": self.scale, "rot": self.rot.to_dict()}


@dataclass(frozen=True)
class ChannelDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int                  # taps of the short convolutions
    decay_rank: int | None     # width of the decay projection's middle; None: what the tensors have
    gate_rank: int | None      # the same for the output gate

    def to_dict(self) -> dict:
        body = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}
        if self.decay_rank is not None:
            body["decay_rank"] = self.decay_rank
        if self.gate_rank is not None:
            body["gate_rank"] = self.gate_rank
        return body


@dataclass(frozen=True)
class DenseConfig:
    ff: int

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class MoEConfig:
    experts: int               # experts with tensors
    identity: int              # router outputs behind them: experts that hand back their input
    top: int
    expert_ff: int
    groups: tuple | None       # (count, keep); None: the choice is among all

    def to_dict(self) -> dict:
        router = {"experts": self.experts, "top": self.top, "identity": self.identity}
        if self.groups is not None:
            router["groups"] = {"count": self.groups[0], "keep": self.groups[1]}
        return {"kind": "moe", "expert": {"ff": self.expert_ff}, "router": router}


@dataclass(frozen=True)
class RetudraLayer:
    type: str                  # one of LAYER_TYPES
    mixer: object
    mlp: object                # DenseConfig, MoEConfig or None

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


def _read_attention(raw, where: str) -> AttentionConfig:
    a = _sub(raw, _ATTENTION, where)
    kv = a["kv_heads"] if a["kv_heads"] is not None else a["heads"]
    _positive(where, heads=a["heads"], kv_heads=kv, dim=a["dim"], vdim=a["vdim"])
    if a["heads"] % kv:
        raise ConfigError(f"{where}: heads must be divisible by kv_heads")
    window, keep = None, 0
    if a["mask"] is not None:
        m = _sub(a["mask"], _MASK, where + ".mask")
        _positive(where + ".mask", size=m["size"])
        if m["keep_first"] < 0:
            raise ConfigError(f"{where}.mask: `keep_first` must not be negative")
        window, keep = m["size"], m["keep_first"]
    return AttentionConfig(a["heads"], kv, a["dim"], a["vdim"], a["scale"], _read_rot(a["rot"], a["dim"], where + ".rot"),
                           window, keep)


def _read_latent(raw, where: str) -> LatentConfig:
    a = _sub(raw, _LATENT, where)
    _positive(where, heads=a["heads"], dim=a["dim"], rot_dim=a["rot_dim"], vdim=a["vdim"], kv_rank=a["kv_rank"])
    return LatentConfig(a["heads"], a["dim"], a["rot_dim"], a["vdim"], a["kv_rank"], a["scale"],
                        _read_rot(a["rot"], a["rot_dim"], where + ".rot"))


def _read_delta(raw, where: str) -> ChannelDeltaConfig:
    a = _sub(raw, _DELTA, where)
    kv = a["kv_heads"] if a["kv_heads"] is not None else a["heads"]
    _positive(where, heads=a["heads"], kv_heads=kv, dim=a["dim"], vdim=a["vdim"], conv=a["conv"])
    for name in ("decay_rank", "gate_rank"):
        if a[name] is not None:
            _positive(where, **{name: a[name]})
    if a["heads"] % kv:
        raise ConfigError(f"{where}: heads must be divisible by kv_heads")
    return ChannelDeltaConfig(a["heads"], kv, a["dim"], a["vdim"], a["conv"], a["decay_rank"], a["gate_rank"])


def _read_mlp(raw, where: str):
    if raw is None:
        return None
    m = _sub(raw, _MLP, where)
    if m["kind"] == "dense":
        if m["ff"] is None:
            raise ConfigError(f"{where}: missing or invalid config field `ff`")
        _positive(where, ff=m["ff"])
        return DenseConfig(m["ff"])
    if m["kind"] != "moe":
        raise ConfigError(f"{where}: unknown kind {m['kind']!r} (known: {', '.join(MLP_KINDS)})")
    if m["expert"] is None or m["router"] is None:
        raise ConfigError(f"{where}: a mixture of experts names `expert` and `router`")
    ff = _sub(m["expert"], (Key("ff", int),), where + ".expert")["ff"]
    r = _sub(m["router"], _ROUTER, where + ".router")
    _positive(where, ff=ff, experts=r["experts"], top=r["top"])
    if r["identity"] < 0:
        raise ConfigError(f"{where}.router: `identity` must not be negative")
    outputs = r["experts"] + r["identity"]
    groups = None
    if r["groups"] is not None:
        g = _sub(r["groups"], _GROUPS, where + ".router.groups")
        _positive(where + ".router.groups", count=g["count"], keep=g["keep"])
        if outputs % g["count"] or g["keep"] > g["count"]:
            raise ConfigError(f"{where}.router.groups: `count` must divide the router's {outputs} outputs, and `keep` "
                              "be at most `count`")
        groups = (g["count"], g["keep"])
    within = outputs if groups is None else groups[1] * (outputs // groups[0])
    if r["top"] > within:
        raise ConfigError(f"{where}.router: `top` = {r['top']} is more than the {within} outputs a token can choose among")
    return MoEConfig(r["experts"], r["identity"], r["top"], ff, groups)


def _read_layer(i: int, raw) -> RetudraLayer:
    where = f"layers[{i}]"
    if not isinstance(raw, dict) or not isinstance(raw.get("mixer"), dict) or not isinstance(raw.get("type"), str):
        raise ConfigError(f"{where}: a layer is an object with `type`, `mixer` and `mlp`")
    kind = raw["type"]
    readers = {"attention": _read_attention, "latent_attention": _read_latent, "channel_delta": _read_delta}
    if kind not in readers:
        raise ConfigError(f"{where}: unknown layer type {kind!r} (known: {', '.join(LAYER_TYPES)})")
    return RetudraLayer(kind, readers[kind](raw["mixer"], where + ".mixer"), _read_mlp(raw.get("mlp"), where + ".mlp"))


@dataclass(frozen=True)
class RetudraConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float       # the factor on every normed sublayer output that is added to the residual
    side_dim: int | None       # columns of the second embedding a layer reads; None: the model has no token-side input
    logit_softcap: float | None
    layers: tuple

    architecture = ARCHITECTURE
    eos_token_id = None

    @classmethod
    def from_dict(cls, raw: dict) -> "RetudraConfig":
        top = read_keys(raw, _TOP)
        eps = _sub(top["norm"], (Key("eps", float),), "norm")["eps"]
        side = None
        if top["token_side"] is not None:
            side = _sub(top["token_side"], (Key("dim", int),), "token_side")["dim"]
        if len(top["layers"]) > 65535:
            raise ConfigError(f"{len(top['layers'])} layers: more than 65,535 are not taken")
        config = cls(top["vocab"], top["width"], eps, top["residual_mult"], side, top["logit_softcap"],
                     tuple(_read_layer(i, layer) for i, layer in enumerate(top["layers"])))
        config.validate()
        return config

    def validate(self) -> None:
        _positive("config.json", vocab=self.vocab, width=self.width)
        if not self.eps >= 0.0:
            raise ConfigError("norm.eps must not be negative")
        if not self.layers:
            raise ConfigError("`layers` must name at least one layer")
        if self.side_dim is not None:
            _positive("token_side", dim=self.side_dim)
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError("`logit_softcap` must be positive")

    def to_dict(self) -> dict:
        """A config.json body that `from_dict` reads back to an equal object."""
        body = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "residual_mult": self.residual_mult, "layers": [layer.to_dict() for layer in self.layers]}
        if self.side_dim is not None:
            body["token_side"] = {"dim": self.side_dim}
        if self.logit_softcap is not None:
            body["logit_softcap"] = self.logit_softcap
        return body
