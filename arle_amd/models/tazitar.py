"""Recipe of the Tazitar decoder: its configuration written out as a ModelSpec.

Layers are pre-norm.  With `streams` in the configuration the residual is that many streams with a learned connection
for every sublayer (`hyper_pre_norm` blocks with `hyper_rmsnorm` norms; the last norm reads their sum); without, one
plain residual (`pre_norm`, `rmsnorm`).  Mixers, all on `rotary_attention`, `gated_delta` and `mixer_pair`:

* `attention`: q/k norm with a weight in front of a rotate-half rotation, tanh-capped scores, the ordinary softmax;
* `parallel`: an attention (rotate-half rotation, then unit-rms q and k, a sink of score 0) beside a gated delta rule,
  each output normed over the width, the mean of the two;
* `attention_2`: interleaved rotation with an optional YaRN scaling, then unit-rms q and k, a learned sink per head.

The feed-forward is gated with the tanh form of gelu.  `loop` repeats a run of layers: the schedule names them once a
pass, so the passes share weights and each has its own cache and state.  Tensor names: `embed`,
`l<i>.norm1|norm2`, `l<i>.hc1|hc2.in|out|mix`, `l<i>.mix.*`, `l<i>.mlp.gate|up|down`, `final.norm`, `head`.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.tazitar import ARCHITECTURE, AttentionConfig, DeltaRuleConfig, ParallelConfig, TazitarConfig
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

# the rotation's table is made for the longest request the engine is built for, not for a number of the model's
MAX_POSITIONS = 1 << 30


def _attention(c: TazitarConfig, m: AttentionConfig, p: str, qk_norm, sink, interleaved: bool) -> PartSpec:
    position = None
    if m.rot is not None:
        position = PartSpec("rope_interleaved" if interleaved else "rope_neox",
                            {"head_dim": m.dim, "rotary_dim": m.rot.dims, "theta": m.rot.base, "scaling": m.rot.scaling,
                             "max_positions": 1})
    params = {"hidden_size": c.width, "num_q_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
              "value_dim": m.vdim, "eps": c.eps, "scale": m.scale, "softcap": m.softcap, "qk_norm": qk_norm, "sink": sink,
              "position": position, "window": None}
    weights = {"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o"}
    if qk_norm == "weighted_before":
        weights.update(q_norm=p + "q.norm", k_norm=p + "k.norm")
    if sink == "learned":
        weights["sink"] = p + "sink"
    return PartSpec("rotary_attention", params, weights)


def _delta(c: TazitarConfig, m: DeltaRuleConfig, p: str) -> PartSpec:
    params = {"hidden_size": c.width, "heads": m.heads, "kv_heads": m.kv_heads, "key_dim": m.dim, "value_dim": m.vdim,
              "conv_taps": m.conv, "eps": c.eps, "unit_eps": 1e-6}
    weights = {"q": p + "q", "k": p + "k", "v": p + "v", "g": p + "g", "q_conv": p + "q.conv", "k_conv": p + "k.conv",
               "v_conv": p + "v.conv", "b": p + "b", "a": p + "a", "A_log": p + "A_log", "dt_bias": p + "dt_bias",
               "norm": p + "norm", "o": p + "o"}
    return PartSpec("gated_delta", params, weights)


def _mixer(c: TazitarConfig, kind: str, m, p: str) -> PartSpec:
    if kind == "attention":
        return _attention(c, m, p, "weighted_before", None, False)
    if kind == "attention_2":
        return _attention(c, m, p, "unit_after", "learned", True)
    assert isinstance(m, ParallelConfig)
    left = _attention(c, m.left, p + "left.", "unit_after", "zero", False)
    return PartSpec("mixer_pair", {"width": c.width, "eps": c.eps, "coef": 0.5, "left": left,
                                   "right": _delta(c, m.right, p + "right.")},
                    {"left_out": p + "left.out", "right_out": p + "right.out"})


def tazitar_spec(config: TazitarConfig, stop_token_ids=()) -> ModelSpec:
    c = config

    def norm(tensor: str, connection: str | None):
        if c.streams is None:
            return PartSpec("rmsnorm", {"width": c.width, "eps": c.eps}, {"weight": tensor})
        weights = {"weight": tensor}
        if connection is not None:
            weights.update({"in": connection + "in", "out": connection + "out", "mix": connection + "mix"})
        return PartSpec("hyper_rmsnorm", {"width": c.width, "eps": c.eps, "streams": c.streams,
                                          "connect": connection is not None}, weights)

    layers = []
    for i, layer in enumerate(c.layers):
        p = f"l{i}."
        norms = {"mixer_in": norm(p + "norm1", p + "hc1.")}
        ffn = None
        if layer.ff is not None:
            norms["ffn_in"] = norm(p + "norm2", p + "hc2.")
            ffn = PartSpec("swiglu", {"hidden_size": c.width, "intermediate_size": layer.ff, "activation": "gelu_tanh",
                                      "float32_out": True},
                           {"gate": p + "mlp.gate", "up": p + "mlp.up", "down": p + "mlp.down"})
        layers.append(LayerSpec("pre_norm" if c.streams is None else "hyper_pre_norm",
                                _mixer(c, layer.type, layer.mixer, p + "mix."), ffn, norms))
    sizes = {"vocab_size": c.vocab, "hidden_size": c.width}
    return ModelSpec(hidden_size=c.width, vocab_size=c.vocab, max_positions=MAX_POSITIONS,
                     embedding=PartSpec("token_table", sizes, {"table": "embed"}),
                     layers=layers, schedule=[ScheduleEntry(i) for i in c.layer_order()],
                     final_norm=norm("final.norm", None),
                     head=PartSpec("linear", sizes, {"weight": "head"}),
                     stop_token_ids=tuple(stop_token_ids))


register_architecture(ARCHITECTURE, TazitarConfig, tazitar_spec)
