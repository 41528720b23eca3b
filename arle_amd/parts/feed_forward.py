"""Dense feed-forwards.  SwiGLU: down(silu(gate(x)) * up(x)), no biases; PolyNorm (below): one projection up
with a bias, a polynomial of row-normalised powers, one projection down with a bias.

infer/src/model/qwen3/prefill.rs:291-337.  gate and up are kept as one [2I, H] matrix
(gate rows first, as the reference's optional fusion does, weights.rs:111-121) so a step
runs one product for both.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, WeightDecl, register
from .linear import Linear


@register("feed_forward", "swiglu")
class SwiGLU(Part):
    """params: hidden_size, intermediate_size, float32_out (bool, default False: the down projection hands on its
    32-bit sums instead of rounding them to the activation type), activation ("silu", the default, or "gelu_tanh":
    what the gate passes through before it multiplies up)."""

    graph_safe = True  # launches depend on shapes only, never on the values of a step

    @classmethod
    def declare_weights(cls, params):
        h, i = params["hidden_size"], params["intermediate_size"]
        return {"gate": WeightDecl((i, h)), "up": WeightDecl((i, h)), "down": WeightDecl((h, i))}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.inter = int(params["intermediate_size"])
        self.float32_out = bool(params.get("float32_out", False))
        name = params.get("activation") or "silu"
        if name not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {name!r} (known: {', '.join(ops.ACTIVATIONS)})")
        self.act = ops.ACTIVATIONS[name]
        gate, up = tensors["gate"], tensors["up"]
        if gate.dtype != up.dtype:
            raise ValueError("gate and up projections must be stored in one type")
        # bfloat16: rows interleaved in blocks of 16 (16 gate rows, the 16 matching up rows, ...), so
        # that one tile of the decode kernel holds both halves of 16 outputs and applies the activation
        # itself.  Otherwise gate rows first, then up rows.
        self.block = 16 if (gate.dtype == torch.bfloat16 and self.inter % 16 == 0) else 0
        if self.block:
            h = gate.shape[1]
            fused = torch.stack([gate.view(-1, 16, h), up.view(-1, 16, h)], dim=1).reshape(2 * self.inter, h)
        else:
            fused = torch.cat([gate, up], dim=0)
        self.gate_up = Linear(fused.contiguous(), rt.weight_tiles)
        self.down = Linear(tensors["down"], rt.weight_tiles)

    def products(self):
        if self.gate_up.weight.dtype != torch.bfloat16:
            return []
        return [("gate_up", self.gate_up.out_features, self.gate_up.in_features, bool(self.block), None),
                ("down", self.down.out_features, self.down.in_features, False, "norm")]

    def forward(self, x):
        """x [T, H] -> [T, H], or a float32 stack [S, T, H] to be added in order (see Linear)."""
        if self.block:
            act = ops.gate_up_act(x, self.gate_up.weight, self.gate_up.tiles, self.act)   # one product with the activation, or two kernels
        else:
            gu = self.gate_up(x)
            act = ops.act_mul(gu[:, : self.inter], gu[:, self.inter:], self.act)
        return self.down(act, out_dtype=torch.float32 if self.float32_out else None, partials_ok=True)


@register("feed_forward", "polynorm")
class PolyNormFeedForward(Part):
    """down(act(up x + b_up)) + b_down with act(z) = a N(z) + b N(z^2) + c N(z^3) + e, powers element by element,
    N the division of a row of the hidden layer by its root mean square (eps inside the root).
    params: hidden_size, intermediate_size, eps.  The four numbers are a tensor of the checkpoint."""

    graph_safe = True  # launches depend on shapes only, never on the values of a step

    @classmethod
    def declare_weights(cls, params):
        h, i = params["hidden_size"], params["intermediate_size"]
        return {"up": WeightDecl((i, h)), "up_bias": WeightDecl((i,), init="normal"), "down": WeightDecl((h, i)),
                "down_bias": WeightDecl((h,), init="normal"), "coef": WeightDecl((4,), init="ones")}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.eps = float(params["eps"])
        self.up = Linear(tensors["up"], rt.weight_tiles)
        self.down = Linear(tensors["down"], rt.weight_tiles)
        self.up_bias, self.down_bias, self.coef = tensors["up_bias"], tensors["down_bias"], tensors["coef"]

    def products(self):
        if self.up.weight.dtype != torch.bfloat16:
            return []
        return [("up", self.up.out_features, self.up.in_features, False, None),
                ("down", self.down.out_features, self.down.in_features, False, "norm")]

    def forward(self, x):
        """x [T, H] -> (delta, bias of the down projection): the block's next norm adds both."""
        act = ops.polynorm(self.up(x), self.coef, self.eps, bias=self.up_bias)
        # float32 out: the sum goes into the 32-bit residual unrounded
        return self.down(act, out_dtype=torch.float32, partials_ok=True), self.down_bias
