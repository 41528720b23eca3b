"""Two mixers side by side: both read the same input, each one's output is RMS-normed over the model width with a
weight of its own, and the result is `coef` times their sum (the mean, by default).

    out = coef * (left(h) / rms(left(h)) * w_left + right(h) / rms(right(h)) * w_right)

Each keeps the cache or state it declares; the pair's need is the dictionary {"left": ..., "right": ...}.
"""
from __future__ import annotations

from ..kernels import ops
from .base import Part, WeightDecl, lookup, register


@register("mixer", "mixer_pair")
class MixerPair(Part):
    """params: width, eps, left (PartSpec of a mixer), right (PartSpec of a mixer), coef (default 0.5)."""

    @classmethod
    def declare_weights(cls, params):
        return {"left_out": WeightDecl((params["width"],), init="ones"), "right_out": WeightDecl((params["width"],), init="ones")}

    @classmethod
    def children(cls, params):
        return {"left": ("mixer", params["left"]), "right": ("mixer", params["right"])}

    @classmethod
    def _need(cls, left, right):
        need = {name: n for name, n in (("left", left), ("right", right)) if n is not None}
        return need or None

    @classmethod
    def declare_cache(cls, params):
        return cls._need(*(lookup("mixer", params[s].kind).declare_cache(params[s].params) for s in ("left", "right")))

    def cache_need(self):
        return self._need(self.left.cache_need(), self.right.cache_need())

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.left, self.right = children["left"], children["right"]
        self.eps = float(params["eps"])
        self.coef = float(params.get("coef", 0.5))
        self.w_left = tensors["left_out"].float().contiguous()
        self.w_right = tensors["right_out"].float().contiguous()
        self.graph_safe = all(bool(getattr(m, "graph_safe", False)) for m in (self.left, self.right))

    def products(self):
        return self.left.products() + self.right.products()

    def decode_launch_class(self, rows, max_context):
        found = tuple(m.decode_launch_class(rows, max_context) for m in (self.left, self.right))
        return None if all(f is None for f in found) else found

    def forward(self, x, batch, cache):
        """x [T, W] -> float32 [T, W]."""
        cache = cache or {}
        a = self.left.forward(x, batch, cache.get("left"))
        b = self.right.forward(x, batch, cache.get("right"))
        return ops.pair_norm(a, b, self.w_left, self.w_right, self.eps, self.coef)
