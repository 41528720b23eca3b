"""Recipe of the Retudra decoder: its configuration written out as a ModelSpec.

Every layer is a `post_norm` block: the mixer and the feed-forward read the residual itself, a layer norm with weight
and bias stands on each one's output, and what is added to the residual is that times the model's `residual_mult`
(the norms' `add_scale`).  Mixers: `wide_norm_attention` with a rotate-half rotation behind the whole-row norm, a
window and kept first keys; `latent_attention` with the same rotation on its rotated part and a sigmoid gate on the
heads' outputs; `gated_delta` with a decay for every key channel and a low-rank sigmoid gate.  Feed-forwards: `swiglu`,
or `sigmoid_moe` with a softmax router, grouped choice, unnormalised weights and identity experts.  A model with
`token_side` gives every layer a `token_side` part behind the feed-forward, RMS-normed (plain weight) on its way into
the residual.  The final norm is the same layer norm; the head caps its logits.  Tensor names: `embed`, `side.embed`,
`l<i>.norm1|norm2` (+ `.b`), `l<i>.mix.*`, `l<i>.mlp.*`, `l<i>.side.gate|proj|norm`, `final.norm` (+ `.b`), `head`.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.retudra import (ARCHITECTURE, AttentionConfig, ChannelDeltaConfig, DenseConfig, LatentConfig, MoEConfig,
                              RetudraConfig)
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

# the rotation's table is made for the longest request the engine is built for, not for a number of the model's
MAX_POSITIONS = 1 << 30
# inside the root of the delta rule's unit norms: a constant of the design
UNIT_EPS = 1e-6


def _rotation(head_dim: int, rot) -> PartSpec | None:
    if rot is None:
        return None
    return PartSpec("rope_neox", {"head_dim": head_dim, "rotary_dim": rot.dims, "theta": rot.base, "max_positions": 1})


def _attention(c: RetudraConfig, m: AttentionConfig, p: str) -> PartSpec:
    params = {"hidden_size": c.width, "num_q_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
              "value_dim": m.vdim, "qk_norm": True, "eps": c.eps, "scale": m.scale, "chunk": None, "window": m.window,
              "keep_first": m.keep_first, "position": _rotation(m.dim, m.rot), "value_mix": None}
    return PartSpec("wide_norm_attention", params,
                    {"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o", "q_norm": p + "q.norm", "k_norm": p + "k.norm"})


def _latent(c: RetudraConfig, m: LatentConfig, p: str) -> PartSpec:
    params = {"hidden_size": c.width, "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "value_dim": m.vdim,
              "rank": m.kv_rank, "eps": c.eps, "scale": m.scale, "window": None, "sink": False, "gate": True,
              "position": _rotation(m.rot_dim, m.rot)}
    return PartSpec("latent_attention", params,
                    {"q": p + "q", "dkv": p + "dkv", "c_norm": p + "dkv.norm", "uk": p + "uk", "uv": p + "uv",
                     "g": p + "g", "o": p + "o"})


def _delta(c: RetudraConfig, m: ChannelDeltaConfig, p: str) -> PartSpec:
    params = {"hidden_size": c.width, "heads": m.heads, "kv_heads": m.kv_heads, "key_dim": m.dim, "value_dim": m.vdim,
              "conv_taps": m.conv, "eps": c.eps, "unit_eps": UNIT_EPS, "decay": "channel", "gate": "sigmoid_low_rank",
              "decay_rank": m.decay_rank, "gate_rank": m.gate_rank}
    weights = {"q": p + "q", "k": p + "k", "v": p + "v", "q_conv": p + "q.conv", "k_conv": p + "k.conv",
               "v_conv": p + "v.conv", "b": p + "b", "a1": p + "a1", "a2": p + "a2", "A_log": p + "A_log",
               "dt_bias": p + "dt_bias", "g1": p + "g1", "g2": p + "g2", "norm": p + "norm", "o": p + "o"}
    return PartSpec("gated_delta", params, weights)


def _feed_forward(c: RetudraConfig, m, p: str) -> PartSpec:
    if isinstance(m, DenseConfig):
        return PartSpec("swiglu", {"hidden_size": c.width, "intermediate_size": m.ff, "float32_out": True},
                        {"gate": p + "gate", "up": p + "up", "down": p + "down"})
    assert isinstance(m, MoEConfig)
    params = {"hidden_size": c.width, "experts": m.experts, "identity": m.identity, "top": m.top, "expert_size": m.expert_ff,
              "scale": 1.0, "score": "softmax", "normalize": False, "correction": True, "shared_size": None,
              "groups": m.groups[0] if m.groups else 1, "keep_groups": m.groups[1] if m.groups else 1}
    weights = {"router": p + "router", "correction": p + "correction"}
    for e in range(m.experts):
        weights.update({f"gate{e}": f"{p}e{e}.gate", f"up{e}": f"{p}e{e}.up", f"down{e}": f"{p}e{e}.down"})
    return PartSpec("sigmoid_moe", params, weights)


_MIXERS = {AttentionConfig: _attention, LatentConfig: _latent, ChannelDeltaConfig: _delta}


def retudra_spec(config: RetudraConfig, stop_token_ids=()) -> ModelSpec:
    c = config

    def layer_norm(tensor: str, add_scale: float = 1.0) -> PartSpec:
        return PartSpec("layernorm", {"width": c.width, "eps": c.eps, "bias": True, "add_scale": add_scale},
                        {"weight": tensor, "bias": tensor + ".b"})

    layers = []
    for i, layer in enumerate(c.layers):
        p = f"l{i}."
        norms = {"mixer_out": layer_norm(p + "norm1", c.residual_mult)}
        ffn = None
        if layer.mlp is not None:
            norms["ffn_out"] = layer_norm(p + "norm2", c.residual_mult)
            ffn = _feed_forward(c, layer.mlp, p + "mlp.")
        parts = {}
        if c.side_dim is not None:
            side = PartSpec("token_side", {"hidden_size": c.width, "vocab_size": c.vocab, "dim": c.side_dim,
                                           "first": i * c.side_dim, "table_width": len(c.layers) * c.side_dim,
                                           "activation": "gelu_tanh"},
                            {"table": "side.embed", "gate": p + "side.gate", "proj": p + "side.proj"})
            parts["side"] = ("feed_forward", side)
            norms["side_out"] = PartSpec("rmsnorm", {"width": c.width, "eps": c.eps, "add_scale": c.residual_mult},
                                         {"weight": p + "side.norm"})
        layers.append(LayerSpec("post_norm", _MIXERS[type(layer.mixer)](c, layer.mixer, p + "mix."), ffn, norms, parts))
    sizes = {"vocab_size": c.vocab, "hidden_size": c.width}
    return ModelSpec(hidden_size=c.width, vocab_size=c.vocab, max_positions=MAX_POSITIONS,
                     embedding=PartSpec("token_table", sizes, {"table": "embed"}),
                     layers=layers, schedule=[ScheduleEntry(i) for i in range(len(layers))],
                     final_norm=layer_norm("final.norm"),
                     head=PartSpec("linear", dict(sizes, softcap=c.logit_softcap), {"weight": "head"}),
                     stop_token_ids=tuple(stop_token_ids))


register_architecture(ARCHITECTURE, RetudraConfig, retudra_spec)
