"""Residual streams with learned connections (hyper-connections): instead of one residual a token carries S copies
x_1..x_S, all equal to the embedding's output at the start, and every sublayer has a connection of its own:

    reads    N(sum_s a_s x_s)                                   a [S], N an RMS norm with a plain weight
    writes   x_t <- sum_s M[s, t] x_s + b_t y                   M [S, S] indexed [from, to], b [S], y its output

all streams at once from the old ones.  Behind the last layer the model's norm reads the plain sum of the streams.

`hyper_rmsnorm` (a norm) holds one sublayer's connection and norm weight.  `hyper_pre_norm` (a block) runs
mixer and feed-forward through two of them.  What a sublayer has put out is not written at once: it travels on as a
`StreamWrite`, and the kernel that reads for the next sublayer (of this block, of the next one, or the model's last
norm) writes it in the same pass.  The streams are float32 `[T, S, W]`; a block that receives the embedding's
`[T, W]` makes them.
"""
from __future__ import annotations

from ..kernels import ops
from .base import Part, WeightDecl, register


class StreamWrite:
    """A sublayer's output (a tensor [T, W] or a float32 stack [P, T, W]) and the connection it is written through."""

    def __init__(self, y, connection):
        self.y = y
        self.connection = connection

    def settled(self, streams):
        """float32 [T, W]: the sum of the streams once this write is done (for a debugging dump; torch arithmetic)."""
        c = self.connection
        y = (self.y.float().sum(0) if self.y.dim() == 3 else self.y.float())
        x = streams if streams.dim() == 3 else streams.unsqueeze(1).expand(-1, c.streams, -1)
        new = (x.unsqueeze(2) * c.mix[None, :, :, None]).sum(1) + c.out_w[None, :, None] * y[:, None, :]
        return new.sum(1)


@register("norm", "hyper_rmsnorm")
class HyperRMSNorm(Part):
    """params: width, eps, streams, connect (bool, default True; False: no connection of its own, it reads the plain
    sum of the streams: the norm behind the last layer)."""

    graph_safe = True  # launches depend on shapes only, never on the values of a step

    @classmethod
    def declare_weights(cls, params):
        s = int(params["streams"])
        decl = {"weight": WeightDecl((params["width"],), init="ones")}
        if params.get("connect", True):
            decl.update({"in": WeightDecl((s,), init="stream_in"), "out": WeightDecl((s,), init="ones"),
                         "mix": WeightDecl((s, s), init="stream_mix")})
        return decl

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.streams = int(params["streams"])
        self.eps = float(params["eps"])
        self.width = int(params["width"])
        self.weight = tensors["weight"].float().contiguous()
        self.connect = bool(params.get("connect", True))
        self.in_w = tensors["in"].float().contiguous() if self.connect else None
        self.out_w = tensors["out"].float().contiguous() if self.connect else None
        self.mix = tensors["mix"].float().contiguous() if self.connect else None

    def read(self, streams, pending=None, rows=None):
        """(streams [T, S, W], what the sublayer reads [T or rows, W] in the activation type); `pending`, the
        `StreamWrite` of the sublayer before, is written first."""
        if pending is not None and not isinstance(pending, StreamWrite):
            raise ValueError("between sublayers of residual streams travels a StreamWrite")
        c = pending.connection if pending is not None else None
        return ops.hyper_step(streams, pending.y if c else None, c.mix if c else None, c.out_w if c else None,
                              self.in_w, self.weight, self.eps, self.rt.act_dtype, num_streams=self.streams, rows=rows)

    # the model's last norm is asked like any norm
    def add_norm(self, residual, delta, rows=None):
        return self.read(residual, delta, rows=rows)[1]

    def forward(self, x, rows=None):
        return self.read(x, None, rows=rows)[1]


@register("block", "hyper_pre_norm")
class HyperPreNormBlock:
    """The pre-norm layer over residual streams.  norm roles: "mixer_in", "ffn_in" (the second only with a
    feed-forward), both `hyper_rmsnorm`.  It hands on the streams and the `StreamWrite` of its last sublayer."""

    norm_roles = ("mixer_in", "ffn_in")

    def __init__(self, mixer, feed_forward, norms: dict):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms
        self.norm_mixer = norms["mixer_in"]
        self.norm_ffn = norms.get("ffn_in") if feed_forward is not None else None

    def forward(self, residual, delta, batch, cache_view):
        streams, a = self.norm_mixer.read(residual, delta)
        pending = StreamWrite(self.mixer.forward(a, batch, cache_view), self.norm_mixer)
        if self.norm_ffn is not None:
            streams, b = self.norm_ffn.read(streams, pending)
            pending = StreamWrite(self.feed_forward.forward(b), self.norm_ffn)
        return streams, pending
