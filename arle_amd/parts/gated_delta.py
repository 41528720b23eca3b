"""The gated delta rule mixer: a matrix state per head that decays, is corrected towards the current value along the
current key, and is read with the current query; q, k and v pass short causal convolutions first.

Per token, with h the mixer's input, H heads, G q/k heads (head j reads q/k head j // (H / G)), key size D, value size Dv:

    q, k = silu(conv(W_q h)), silu(conv(W_k h))  [G, D];   v = silu(conv(W_v h))  [H, Dv]
    q <- q / sqrt(sum q^2 + 1e-6) * D^(-1/2);   k <- k / sqrt(sum k^2 + 1e-6)            per head
    beta = sigmoid(W_b h);   g = exp(-exp(A_log) * softplus(W_a h + dt_bias))             per head
    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q                       per head, S [D, Dv]
    out = W_o ((o / rms(o) per head) * w_norm * silu(W_g h))

Two options.  `decay` "channel": a decay for every head and key entry, on the rows of S (S <- diag(g) S), from a
projection through a narrow middle, g = exp(-exp(A_log_h) * softplus(W_a2 (W_a1 h) + dt_bias)) laid out [H, D].
`gate` "sigmoid_low_rank": the output gate is sigmoid(W_g2 (W_g1 h)).  The widths of the narrow middles are the
tensors' own (`decay_rank`, `gate_rank` fix them where a model is made from nothing).

S starts at zero and lives in a 32-bit state slot `[H, D, Dv]` of the request; the convolutions' last taps - 1 inputs
are state too.  The gates' projections hand over 32-bit sums, and the unit norms, the gates, the recurrence and the head
norm are 32-bit in every mode; q, k, v, the output gate and the convolutions run in the activation type.
"""
from __future__ import annotations

import torch

from ..cache.manager import StateNeed
from ..kernels import ops
from .base import Part, WeightDecl, register
from .linear import Linear
from .short_conv import ShortConv


@register("mixer", "gated_delta")
class GatedDeltaMixer(Part):
    """params: hidden_size, heads, kv_heads, key_dim, value_dim, conv_taps, eps (of the head norm),
    unit_eps (inside the root of the unit norms; default 1e-6), decay ("head", the default, or "channel"),
    gate ("silu", the default, or "sigmoid_low_rank"), decay_rank, gate_rank (int, or None: whatever the tensors have)."""

    DECAYS = ("head", "channel")
    GATES = ("silu", "sigmoid_low_rank")

    graph_safe = True  # rows, slots and lengths are read on the GPU; launches depend on shapes only

    @classmethod
    def _widths(cls, params):
        qk = params["kv_heads"] * params["key_dim"]
        return qk, qk, params["heads"] * params["value_dim"]

    @classmethod
    def declare_weights(cls, params):
        w, h, dv, taps = params["hidden_size"], params["heads"], params["value_dim"], params["conv_taps"]
        qk, _, vw = cls._widths(params)
        decl = {"q": WeightDecl((qk, w)), "k": WeightDecl((qk, w)), "v": WeightDecl((vw, w)),
                "q_conv": WeightDecl((qk, taps)), "k_conv": WeightDecl((qk, taps)), "v_conv": WeightDecl((vw, taps)),
                "b": WeightDecl((h, w)), "A_log": WeightDecl((h,), init="zeros"),
                "norm": WeightDecl((dv,), init="ones"), "o": WeightDecl((w, vw))}
        if params.get("decay", "head") == "channel":
            r, n = params.get("decay_rank"), h * params["key_dim"]
            decl.update(a1=WeightDecl((r, w)), a2=WeightDecl((n, r)), dt_bias=WeightDecl((n,), init="normal"))
        else:
            decl.update(a=WeightDecl((h, w)), dt_bias=WeightDecl((h,), init="normal"))
        if params.get("gate", "silu") == "sigmoid_low_rank":
            r = params.get("gate_rank")
            decl.update(g1=WeightDecl((r, w)), g2=WeightDecl((vw, r)))
        else:
            decl["g"] = WeightDecl((vw, w))
        return decl

    @classmethod
    def declare_cache(cls, params):
        h, d, dv = int(params["heads"]), int(params["key_dim"]), int(params["value_dim"])
        need = {"S": StateNeed((h, d, dv), torch.float32)}
        conv = ShortConv.state_need(sum(cls._widths(params)), int(params["conv_taps"]))
        if conv is not None:
            need["conv"] = conv
        return need

    def cache_need(self):
        return self.declare_cache(self.params)

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.H, self.G = int(params["heads"]), int(params["kv_heads"])
        self.D, self.Dv = int(params["key_dim"]), int(params["value_dim"])
        if self.G < 1 or self.H % self.G:
            raise ValueError("heads must be a multiple of kv_heads")
        if not 0 < self.D <= ops.GATED_DELTA_MAX_KEY_DIM:
            raise ValueError(f"key_dim {self.D} is not supported: the gated delta rule's kernel takes 1..{ops.GATED_DELTA_MAX_KEY_DIM}")
        self.eps = float(params["eps"])
        self.unit_eps = float(params.get("unit_eps", 1e-6))
        self.decay, self.gate = params.get("decay", "head"), params.get("gate", "silu")
        if self.decay not in self.DECAYS or self.gate not in self.GATES:
            raise ValueError(f"decay is one of {self.DECAYS} and gate one of {self.GATES}")
        low_gate = self.gate == "sigmoid_low_rank"
        channel = self.decay == "channel"
        if low_gate and tensors["g1"].shape[0] != tensors["g2"].shape[1]:
            raise ValueError("the two projections of the output gate do not meet in one width")
        if channel and tensors["a1"].shape[0] != tensors["a2"].shape[1]:
            raise ValueError("the two projections of the decay do not meet in one width")
        # one product for q, k, v, the output gate (or its narrow middle) and, with a decay a channel, the decay's
        # narrow middle: all of them operands of what follows, in the activation type
        fused = [tensors[n] for n in ("q", "k", "v", "g1" if low_gate else "g")] + ([tensors["a1"]] if channel else [])
        if len({t.dtype for t in fused}) != 1:
            raise ValueError("q, k, v and gate projections must be stored in one type")
        self.gate_width = int(fused[3].shape[0])
        self.decay_rank = int(tensors["a1"].shape[0]) if channel else 0
        self.qkvg = Linear(torch.cat(fused, dim=0).contiguous(), rt.weight_tiles)
        self.gate_up = Linear(tensors["g2"], rt.weight_tiles) if low_gate else None
        self.gate_act = ops.GATES["sigmoid" if low_gate else "silu"]
        self.conv = ShortConv(torch.cat([tensors[n] for n in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous())
        # beta and the decay enter the recurrence: their projection hands over 32-bit sums whatever the mode.  In
        # bfloat16 it is a product of bfloat16 operands like every projection (rows padded with zeros to whole tiles
        # of 16 outputs), in float32 the fixed-order 32-bit product.  With a decay a channel it makes beta alone, and
        # the second projection of the decay (32-bit sums again) the channels' pre-activations from the narrow middle.
        gates = tensors["b"] if channel else torch.cat([tensors["b"], tensors["a"]], dim=0)
        if gates.dtype == torch.bfloat16 and not rt.is_f32:
            pad = -gates.shape[0] % 16
            gates = torch.cat([gates, gates.new_zeros((pad, gates.shape[1]))], dim=0) if pad else gates
            self.gates = Linear(gates.contiguous(), rt.weight_tiles)
            self.decay_up = Linear(tensors["a2"], rt.weight_tiles) if channel else None
        else:
            self.gates = Linear(gates.float().contiguous())
            self.decay_up = Linear(tensors["a2"].float().contiguous()) if channel else None
        self.a_log, self.dt_bias = tensors["A_log"].float().contiguous(), tensors["dt_bias"].float().contiguous()
        self.norm = tensors["norm"]
        self.o = Linear(tensors["o"], rt.weight_tiles)

    def products(self):
        if self.qkvg.weight.dtype != torch.bfloat16:
            return []
        return [("qkvg", self.qkvg.out_features, self.qkvg.in_features, False, None),
                ("o", self.o.out_features, self.o.in_features, False, "norm")]

    def forward(self, x, batch, cache):
        """x [T, W] -> float32 [T, W], or a float32 stack [S, T, W] to be added in order (see Linear)."""
        qk, _, vw = self._widths(self.params)
        p = self.qkvg(x)
        y = self.conv(p[:, :2 * qk + vw], batch, cache.get("conv"), silu=True)
        gates = self.gates(x, out_dtype=torch.float32)
        at = 2 * qk + vw
        gate, middle = p[:, at:at + self.gate_width], p[:, at + self.gate_width:]
        channel = None
        if self.decay_up is not None:
            channel = self.decay_up(middle, out_dtype=torch.float32)
        o = ops.gated_delta_scan(y[:, :qk], y[:, qk:2 * qk], y[:, 2 * qk:], gates, self.a_log, self.dt_bias,
                                 cache["S"].state, batch.seg_row0, batch.seg_slot, heads=self.H, kv_heads=self.G,
                                 key_dim=self.D, value_dim=self.Dv, unit_eps=self.unit_eps, channel_decay=channel)
        if self.gate_up is not None:
            gate = self.gate_up(gate)
        z = ops.gated_delta_output(o, gate, self.norm, self.eps, heads=self.H, value_dim=self.Dv, act=self.gate_act)
        return self.o(z, out_dtype=torch.float32, partials_ok=True)   # it goes into the 32-bit residual unrounded
