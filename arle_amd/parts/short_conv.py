"""A short causal convolution over time on every channel, continued across steps, and a mixer wrapper that
puts one in front of any other mixer.

`ShortConv` is the mechanism: y_t = sum_j w[:, j] u_(t - taps + 1 + j) per channel with zeros before a sequence's
start (optionally u_t + that sum), where the last taps - 1 inputs of every request live in a state slot
`[taps - 1, channels]` of the activation type, so that a row's result is the same bits whether its predecessors
came in the same step or in an earlier one.  `input_conv` (mixer): h <- h + conv(h) on what the inner mixer
reads; its cache need is a dictionary of its own state and the inner mixer's need.
"""
from __future__ import annotations

from ..cache.manager import StateNeed
from ..kernels import ops
from .base import Part, WeightDecl, register


class ShortConv:
    """One convolution weight [channels, taps] (None: no convolution) with an optional bias on its input."""

    def __init__(self, weight, bias=None):
        self.weight = weight
        self.bias = bias
        self.taps = int(weight.shape[1]) if weight is not None else 1

    @staticmethod
    def state_need(channels: int, taps: int):
        """The state of a convolution of `taps` taps: its last taps - 1 inputs, in the activation type."""
        return StateNeed((taps - 1, channels), None) if taps > 1 else None

    def __call__(self, u, batch, state_view, add_input: bool = False, silu: bool = False):
        """The convolution of the step's rows (with `silu`, its silu); the requests' states move on by the rows they brought."""
        state = state_view.state if (state_view is not None and self.taps > 1) else None
        y = ops.causal_conv(u, self.weight, state, batch.slot_of_token, bias=self.bias, add_input=add_input, silu=silu)
        if state is not None:
            ops.conv_state_update(u, state, batch.seg_row0, batch.seg_slot, bias=self.bias)
        return y


@register("mixer", "input_conv")
class InputConvMixer(Part):
    """params: width, taps, inner (PartSpec of the mixer that reads h + conv(h))."""

    @classmethod
    def declare_weights(cls, params):
        return {"weight": WeightDecl((params["width"], params["taps"]))}

    @classmethod
    def children(cls, params):
        return {"inner": ("mixer", params["inner"])}

    @classmethod
    def _need(cls, params, inner_need):
        need = {"inner": inner_need} if inner_need is not None else {}
        own = ShortConv.state_need(int(params["width"]), int(params["taps"]))
        if own is not None:
            need["input_conv"] = own
        return need or None

    @classmethod
    def declare_cache(cls, params):
        from .base import lookup

        return cls._need(params, lookup("mixer", params["inner"].kind).declare_cache(params["inner"].params))

    @classmethod
    def declare_reader_cache(cls, params):
        from .base import lookup

        return cls._need(params, lookup("mixer", params["inner"].kind).declare_reader_cache(params["inner"].params))

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.conv = ShortConv(tensors["weight"])
        self.inner = children["inner"]
        self.graph_safe = bool(getattr(self.inner, "graph_safe", False))

    def cache_need(self):
        return self._need(self.params, self.inner.cache_need())

    def reader_cache_need(self):
        return self._need(self.params, self.inner.reader_cache_need())

    def products(self):
        return self.inner.products()

    def decode_launch_class(self, rows, max_context):
        return self.inner.decode_launch_class(rows, max_context)

    def forward(self, x, batch, cache):
        cache = cache or {}
        h = self.conv(x, batch, cache.get("input_conv"), add_input=True)
        return self.inner.forward(h, batch, cache.get("inner"))
