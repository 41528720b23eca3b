"""A per-layer input from the token itself: a slice of a second embedding's row, gated by the residual.

    e = table[token][first : first + dim];   g = act(W_gate x) * e;   y = W_proj g

`table` is one tensor for the whole model, [vocab, layers * dim]; a layer's part reads its own `dim` columns from
`first` on.  The part is a feed-forward that also reads the step's token ids (`forward(x, batch)`), for a block that
runs it as a sublayer of its own and norms its output.  The projection back hands on its 32-bit sums.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, WeightDecl, register
from .linear import Linear


@register("feed_forward", "token_side")
class TokenSide(Part):
    """params: hidden_size, vocab_size, dim, first (column of the table where this layer's slice begins),
    table_width (columns of the whole table), activation (of the gate; default "gelu_tanh")."""

    graph_safe = True  # the token ids are read on the GPU; launches depend on shapes only

    @classmethod
    def declare_weights(cls, params):
        h, d = params["hidden_size"], params["dim"]
        return {"table": WeightDecl((params["vocab_size"], params["table_width"])), "gate": WeightDecl((d, h)),
                "proj": WeightDecl((h, d))}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.dim, self.first = int(params["dim"]), int(params["first"])
        if self.dim < 1 or self.first < 0 or self.first + self.dim > int(params["table_width"]):
            raise ValueError("a layer's slice must lie inside the table's columns")
        name = params.get("activation") or "gelu_tanh"
        if name not in ops.GATES:
            raise ValueError(f"unknown activation {name!r} (known: {', '.join(ops.GATES)})")
        self.act = ops.GATES[name]
        self.table = tensors["table"]
        self.gate = Linear(tensors["gate"], rt.weight_tiles)
        self.proj = Linear(tensors["proj"], rt.weight_tiles)

    def products(self):
        if self.gate.weight.dtype != torch.bfloat16:
            return []
        return [("side_gate", self.gate.out_features, self.gate.in_features, False, None),
                ("side_proj", self.proj.out_features, self.proj.in_features, False, "norm")]

    def forward(self, x, batch):
        """x [T, H] -> float32 [T, H], or a float32 stack [S, T, H] to be added in order (see Linear)."""
        g = ops.token_gate(self.gate(x), self.table, batch.token_ids, self.first, self.act)
        return self.proj(g, out_dtype=torch.float32, partials_ok=True)
