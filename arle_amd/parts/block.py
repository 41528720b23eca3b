"""Arrangements of a mixer, a feed-forward and norms in one layer.

`pre_norm`: h += mixer(norm(h)); h += ffn(norm(h))  (infer/src/model/qwen3/prefill.rs:618-776).
The residual stream is float32.  A block receives the residual and the delta its
predecessor has not added yet, so that every add is fused into the norm that follows it
(the reference's fused_add_rms_norm chain, infer/src/model/qwen3/batch_decode.rs:2411-2456).
"""
from __future__ import annotations

from .base import register


@register("block", "pre_norm")
class PreNormBlock:
    """norm roles: "mixer_in", "ffn_in" (the second only with a feed-forward; without one the mixer's output is what
    the next block adds)."""

    norm_roles = ("mixer_in", "ffn_in")

    def __init__(self, mixer, feed_forward, norms: dict):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms
        self.norm_mixer = norms["mixer_in"]
        self.norm_ffn = norms["ffn_in"] if feed_forward is not None else None

    def forward(self, residual, delta, batch, cache_view):
        a = self.norm_mixer.add_norm(residual, delta)
        m = self.mixer.forward(a, batch, cache_view)
        if self.norm_ffn is None:
            return residual, m
        b = self.norm_ffn.add_norm(residual, m)
        return residual, self.feed_forward.forward(b)


@register("block", "post_norm")
class PostNormBlock:
    """h += norm_a(mixer(h)); h += norm_b(ffn(h)): the sublayers read the residual itself, the norms stand on their
    outputs (a norm's `add_scale` is the model's factor on what is added).  norm roles: "mixer_out", "ffn_out" (the
    second only with a feed-forward), "side_out" (with a further part "side").  The residual is float32;
    what a sublayer reads is the residual in the activation type, which the norm's kernel writes beside the sum it
    updates (`add_into`), and which goes from block to block in `batch.carry`.  Nothing is left for the next block
    to add.

    A further part named "side" (a feed-forward that also reads the step's tokens: `forward(x, batch)`) runs behind
    the feed-forward as a third sublayer of the same kind: h += norm_c(side(h, tokens))."""

    norm_roles = ("mixer_out", "ffn_out", "side_out")
    CARRY = "residual_rounded"     # batch.carry[CARRY] = (the residual tensor, its copy in the activation type)

    def __init__(self, mixer, feed_forward, norms: dict, extra: dict | None = None):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms
        self.norm_mixer = norms.get("mixer_out") if mixer is not None else None
        self.norm_ffn = norms.get("ffn_out") if feed_forward is not None else None
        self.side = (extra or {}).get("side")
        self.norm_side = norms.get("side_out") if self.side is not None else None
        if self.side is not None and self.norm_side is None:
            raise ValueError("a post_norm block with a side part needs the norm on its output (side_out)")

    def _reads(self, residual, batch):
        kept = batch.carry.get(self.CARRY)
        if kept is not None and kept[0] is residual:
            return kept[1]
        act = next(iter(self.norms.values())).rt.act_dtype
        if act == residual.dtype:
            return residual
        from ..kernels import ops
        return ops.sum_partials(residual.unsqueeze(0), act)     # one part: a rounding pass

    def forward(self, residual, delta, batch, cache_view):
        if delta is not None:
            raise ValueError("a post_norm block stands behind blocks that leave nothing to add")
        x = self._reads(residual, batch)
        if self.mixer is not None:
            x = self.norm_mixer.add_into(residual, self.mixer.forward(x, batch, cache_view))
        if self.feed_forward is not None:
            x = self.norm_ffn.add_into(residual, self.feed_forward.forward(x))
        if self.side is not None:
            x = self.norm_side.add_into(residual, self.side.forward(x, batch))
        batch.carry[self.CARRY] = (residual, x)
        return residual, None


@register("block", "parallel")
class ParallelBlock:
    """h += mixer(norm_a(h)) + ffn(norm_b(h)): both read the same residual.  norm roles: "mixer_in", "ffn_in" (the
    second only with a feed-forward).  The two outputs go on, unadded, to the next block's norms (or the final one),
    which add them in the pass that computes their statistics; the two norms of this block come out of one pass too.
    A mixer or feed-forward may hand back (delta, bias): the bias of its last projection, added with the delta."""

    norm_roles = ("mixer_in", "ffn_in")

    def __init__(self, mixer, feed_forward, norms: dict):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms
        self.norm_mixer = norms["mixer_in"]
        self.norm_ffn = norms.get("ffn_in") if feed_forward is not None else None

    def forward(self, residual, delta, batch, cache_view):
        from .base import Pending

        if self.norm_ffn is not None:
            a, b = self.norm_mixer.add_norm(residual, delta, also=self.norm_ffn)
        else:
            a = self.norm_mixer.add_norm(residual, delta)
        left = Pending()
        for out in (self.mixer.forward(a, batch, cache_view),
                    self.feed_forward.forward(b) if self.norm_ffn is not None else None):
            if out is not None:
                left.append(out if isinstance(out, tuple) else (out, None))
        return residual, left
