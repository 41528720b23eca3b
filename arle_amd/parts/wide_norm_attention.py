"""Grouped-query attention whose q and k are RMS-normed over the whole projection, with or without a rotation behind
the norm, over the keys of the row's own chunk or of a window that may keep the request's first keys, with values that
may be mixed with those of another layer.

Per token, with h the mixer's input, nq query heads over nkv key/value heads, key size Dk, value size Dv:

    q, k, v = W_q h, W_k h, W_v h                        (no biases)
    q <- q / rms(q) * wq,  k <- k / rms(k) * wk           over all heads' entries at once, plain weights
    q, k <- rotated per head by the position part (optional; `rope_neox` pairs (i, i + R/2), `rope_interleaved`
            (2i, 2i + 1), on the first R entries of a head)
    v <- (1 - lambda) v + lambda v_first                  (`value_mix` "mix"; v_first: the unmixed values that the
                                                           layer with `value_mix` "source" computed for the same token)
    s_ij = scale (q_i . k_j)   for j <= i with floor(i / chunk) = floor(j / chunk)   (chunk None: every j <= i)
                               and (i - j < window or j < keep_first)                 (window None: every j <= i)
    out  = W_o concat_h(softmax_j(s) v)

Chunks are counted from position 0 of the request.  Keys (after the norm) and values (after the mixing) go to pages
`[nkv, page, Dk]` and `[nkv, Dv, page]`.  The source layer hands its values on through `batch.carry[carry_key]`, a view
of its own projection, for the pass that computed them.  The attention itself is the kernel family of
`softcap_attention` (no cap, no penalty), which knows the chunk rule.
"""
from __future__ import annotations

import torch

from ..cache.manager import PAGE, PagedNeed, PageTensor
from ..kernels import ops
from .base import Part, WeightDecl, register
from .linear import Linear
from .softcap_attention import softcap_attention


@register("mixer", "wide_norm_attention")
class WideNormAttention(Part):
    """params: hidden_size, num_q_heads, num_kv_heads, key_dim, value_dim, qk_norm (bool), eps, scale,
    chunk (int | None), window (int | None), keep_first (int, default 0: with a window, the request's first so many keys
    stay visible behind it, at their true positions), position (PartSpec of a rotation, or None),
    value_mix (None | "source" | "mix"), carry_key (str)."""

    graph_safe = True  # positions, slots and lengths are read on the GPU; launches depend on shapes only

    @classmethod
    def _widths(cls, params):
        return (params["num_q_heads"] * params["key_dim"], params["num_kv_heads"] * params["key_dim"],
                params["num_kv_heads"] * params["value_dim"])

    @classmethod
    def declare_weights(cls, params):
        h = params["hidden_size"]
        qw, kw, vw = cls._widths(params)
        decl = {"q": WeightDecl((qw, h)), "k": WeightDecl((kw, h)), "v": WeightDecl((vw, h)),
                "o": WeightDecl((h, params["num_q_heads"] * params["value_dim"]))}
        if params.get("qk_norm"):
            decl.update(q_norm=WeightDecl((qw,), init="ones"), k_norm=WeightDecl((kw,), init="ones"))
        if params.get("value_mix") == "mix":
            decl["mix"] = WeightDecl((), init="normal")
        return decl

    @classmethod
    def children(cls, params):
        return {"position": ("position", params["position"])} if params.get("position") is not None else {}

    @classmethod
    def declare_cache(cls, params):
        nkv, dk, dv = int(params["num_kv_heads"]), int(params["key_dim"]), int(params["value_dim"])
        return PagedNeed(window=params.get("window"), chunk=params.get("chunk"),
                         keep_first=int(params.get("keep_first") or 0) if params.get("window") else 0,
                         tensors=(PageTensor("k", (nkv, PAGE, dk)), PageTensor("v", (nkv, dv, PAGE))))

    def cache_need(self):
        return self.declare_cache(self.params)

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.nq, self.nkv = int(params["num_q_heads"]), int(params["num_kv_heads"])
        self.Dk, self.Dv = int(params["key_dim"]), int(params["value_dim"])
        if self.nkv < 1 or self.nq % self.nkv:
            raise ValueError("num_q_heads must be a multiple of num_kv_heads")
        if not (0 < self.Dk <= ops.MAX_HEAD_DIM and 0 < self.Dv <= ops.MAX_HEAD_DIM):
            raise ValueError(f"head sizes {self.Dk}, {self.Dv} are not supported: the attention kernels take 1..{ops.MAX_HEAD_DIM}")
        self.eps = float(params.get("eps", 0.0))
        self.scale = float(params["scale"])
        self.chunk = int(params.get("chunk") or 0)
        self.window = int(params.get("window") or 0)
        self.keep_first = int(params.get("keep_first") or 0) if self.window else 0
        if self.keep_first < 0:
            raise ValueError("keep_first must not be negative")
        self.position = (children or {}).get("position")
        self.value_mix = params.get("value_mix")
        if self.value_mix not in (None, "source", "mix"):
            raise ValueError(f"value_mix is None, 'source' or 'mix', not {self.value_mix!r}")
        self.carry_key = params.get("carry_key", "first_values")
        mats = [tensors[n] for n in ("q", "k", "v")]
        if len({t.dtype for t in mats}) != 1:
            raise ValueError("q, k and v projections must be stored in one type")
        self.widths = self._widths(params)
        self.proj = Linear(torch.cat(mats, dim=0).contiguous(), rt.weight_tiles)
        self.q_norm, self.k_norm = tensors.get("q_norm"), tensors.get("k_norm")
        self.mix = tensors.get("mix")
        self.o = Linear(tensors["o"], rt.weight_tiles)

    def products(self):
        if self.proj.weight.dtype != torch.bfloat16:
            return []
        return [("qkv", self.proj.out_features, self.proj.in_features, False, None),
                ("o", self.o.out_features, self.o.in_features, False, "norm")]

    def forward(self, x, batch, cache):
        """x [T, H] -> float32 [T, H], or a float32 stack [S, T, H] to be added in order (see Linear)."""
        if not cache.writes:
            raise ValueError("this attention keeps keys and values of its own")
        Q, K, _ = self.widths
        y = self.proj(x)
        q, k, v = y[:, :Q], y[:, Q:Q + K], y[:, Q + K:]
        v_first = None
        if self.value_mix == "source":
            batch.carry[self.carry_key] = v
        elif self.value_mix == "mix":
            v_first = batch.carry.get(self.carry_key)
            if v_first is None:
                raise ValueError("a layer that mixes values runs behind the layer whose values it mixes in")
        cos = sin = None
        rotary_dim, interleaved = 0, False
        if self.position is not None:
            self.position.ensure_positions(batch.max_position + 1)
            cos, sin, rotary_dim = self.position.fused_rotary()
            interleaved = self.position.kind == "rope_interleaved"
        ops.wide_norm_store(q, k, v, num_q_heads=self.nq, num_kv_heads=self.nkv, key_dim=self.Dk, value_dim=self.Dv,
                            eps=self.eps, q_weight=self.q_norm, k_weight=self.k_norm, v_first=v_first, mix=self.mix,
                            positions=batch.positions, slot_of_token=batch.slot_of_token, block_table=cache.block_table,
                            k_pages=cache.pages["k"], v_pages=cache.pages["v"], page_size=cache.page_size, cos=cos,
                            sin=sin, rotary_dim=rotary_dim or 0, interleaved=interleaved)
        out = torch.empty((x.shape[0], self.nq * self.Dv), dtype=x.dtype, device=x.device)
        softcap_attention(q, out, cache, batch, num_q_heads=self.nq, num_kv_heads=self.nkv, key_dim=self.Dk,
                          value_dim=self.Dv, scale=self.scale, softcap=0.0, r1=None, r2=None, window=self.window,
                          chunk=self.chunk, keep_first=self.keep_first)
        return self.o(out, out_dtype=torch.float32, partials_ok=True)   # it goes into the 32-bit residual unrounded
