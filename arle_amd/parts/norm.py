"""Norms over the model width.  RMSNorm: x / sqrt(mean(x^2) + eps) * w with the plain weight w (not 1 + w);
LayerNorm with or without a bias of its own.

crates/cuda-kernels/csrc/misc/norm.cu:8,59,221-359; the residual add fused in as at :462-.
The weight keeps the type the checkpoint stores it in (bfloat16 or float32).
"""
from __future__ import annotations

from ..kernels import ops
from .base import Part, WeightDecl, register


@register("norm", "rmsnorm")
class RMSNorm(Part):
    """params: width, eps, one_plus (bool, default False: the checkpoint stores the weight around zero and the norm
    multiplies by 1 + w; the sum is formed in 32 bits, where it is exact or rounded once), add_scale (default 1: the
    factor on what `add_into` adds to the residual).

    Beside the norm of the residual (`forward`, `add_norm`) it can stand on a sublayer's output: `add_into` norms
    what the sublayer left and adds the result into the residual."""

    graph_safe = True  # launches depend on shapes only, never on the values of a step

    @classmethod
    def declare_weights(cls, params):
        return {"weight": WeightDecl((params["width"],), init="near_zero" if params.get("one_plus") else "ones")}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.one_plus = bool(params.get("one_plus", False))
        self.stored = tensors["weight"]
        self.weight = (1.0 + self.stored.float()) if self.one_plus else self.stored
        self.eps = float(params["eps"])
        self.width = int(params["width"])
        self.add_scale = float(params.get("add_scale", 1.0))

    def forward(self, x, rows=None):
        return ops.rmsnorm(x, self.weight, self.eps, self.rt.act_dtype, rows=rows)

    def add_into(self, residual, terms, want_rounded: bool = True):
        """residual (float32, in place) += norm(sum of `terms`): one or two of a tensor [T, W], a float32 stack
        [S, T, W] of partial sums, or (outputs [T, n, W], float32 weights [T, n]).  Returns the updated residual in
        the activation type: itself in a float32 engine, else a rounded copy from the same pass (None if not
        wanted)."""
        rounded = want_rounded and self.rt.act_dtype != residual.dtype
        out = ops.norm_add(residual, terms, self.stored, self.eps, one_plus=self.one_plus,
                           act_dtype=self.rt.act_dtype if rounded else None, mult=self.add_scale)
        return out if rounded else residual

    def add_norm(self, residual, delta, rows=None):
        """residual (float32) += delta, then the norm of it; delta None: just the norm."""
        if delta is None:
            return ops.rmsnorm(residual, self.weight, self.eps, self.rt.act_dtype, rows=rows)
        return ops.add_rmsnorm(residual, delta, self.weight, self.eps, self.rt.act_dtype, rows=rows)


@register("norm", "layernorm")
class LayerNorm(Part):
    """(x - mean) / sqrt(var + eps) * w (+ b), var the mean of the squared deviations.  params: width, eps, bias (bool,
    default False: the norm has a bias tensor of its own), add_scale (default 1: the factor on what `add_into` adds).

    Beside the norm of the residual it can stand on a sublayer's output: `add_into` norms what the sublayer left and
    adds the result, times add_scale, into the residual.

    `add_norm` takes what the block before has left to add as one tensor, one float32 stack of partial sums, or a
    `Pending` list of up to two of them, each with the bias of the projection that made it; with `also`, a second
    norm of the same sum (another weight, the same width and eps) comes out of the same pass: the two norms of a
    block whose mixer and feed-forward read the same residual."""

    graph_safe = True  # launches depend on shapes only, never on the values of a step

    @classmethod
    def declare_weights(cls, params):
        decl = {"weight": WeightDecl((params["width"],), init="ones")}
        if params.get("bias"):
            decl["bias"] = WeightDecl((params["width"],), init="normal")
        return decl

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.weight = tensors["weight"]
        self.bias = tensors.get("bias")
        if self.bias is not None and self.bias.dtype != self.weight.dtype:
            raise ValueError("a layer norm's weight and bias must be stored in one type")
        self.eps = float(params["eps"])
        self.width = int(params["width"])
        self.add_scale = float(params.get("add_scale", 1.0))

    def forward(self, x, rows=None):
        return self.add_norm(x, None, rows=rows)

    def add_into(self, residual, terms, want_rounded: bool = True):
        """residual (float32, in place) += add_scale * layer_norm(sum of `terms`): one or two of a tensor [T, W], a
        float32 stack [S, T, W] of partial sums, or (outputs [T, n, W], float32 weights [T, n]).  Returns the updated
        residual in the activation type: itself in a float32 engine, else a rounded copy from the same pass (None if
        not wanted)."""
        rounded = want_rounded and self.rt.act_dtype != residual.dtype
        out = ops.norm_add(residual, terms, self.weight, self.eps, center=True, bias=self.bias, mult=self.add_scale,
                           act_dtype=self.rt.act_dtype if rounded else None)
        return out if rounded else residual

    def add_norm(self, residual, delta, rows=None, also=None):
        terms = delta if isinstance(delta, list) else ([] if delta is None else [(delta, None)])
        if also is not None and (also.eps != self.eps or also.width != self.width):
            raise ValueError("two norms share a pass only with one width and one eps")
        return ops.add_layernorm(residual, terms, self.weight, self.eps, self.rt.act_dtype,
                                 weight_b=also.weight if also is not None else None, rows=rows, bias=self.bias,
                                 bias_b=also.bias if also is not None else None)
