"""Grouped-query attention over a paged cache with rotary positions, per-head q/k norms in front of or behind the
rotation, tanh-capped scores and a sink in the softmax; key and value heads may differ in size.

Per token, with h the mixer's input, nq query heads over nkv key/value heads, key size Dk, value size Dv:

    q, k, v = W_q h, W_k h, W_v h                                   (one fused product, no biases)
    qk_norm "weighted_before":  q, k <- per-head RMS norm with a weight of Dk (one for all heads), then the rotation
    qk_norm "unit_after":       the rotation, then q, k <- divided by their root mean square per head
    rotation: the position part's (`rope_neox` pairs (i, i + R/2), `rope_interleaved` pairs (2i, 2i + 1), either with
              a YaRN scaling) on the first R entries of a head
    s_ij    = scale (q_i . k_j);  s <- cap tanh(s / cap)  (softcap > 0);   j <= i, or the last `window` keys
    p_ij    = exp(s_ij) / (sum_j exp(s_ij) + exp(sink_h))            sink "learned": a tensor [nq]; "zero": sink_h = 0,
              one more in the denominator; None: the ordinary softmax
    out     = W_o concat_h(sum_j p_ij v_j)

Keys go to pages `[nkv, page, Dk]` as the kernel reads them (normed and rotated), values to `[nkv, Dv, page]`.  Norms,
angles, scores, the cap, the sink and the softmax are 32-bit; the output projection hands on its 32-bit sums.
"""
from __future__ import annotations

import torch

from ..cache.manager import PAGE, PagedNeed, PageTensor
from ..kernels import ops
from .base import Part, WeightDecl, register
from .linear import Linear
from .softcap_attention import softcap_attention

QK_NORMS = (None, "weighted_before", "unit_after")
SINKS = (None, "zero", "learned")


@register("mixer", "rotary_attention")
class RotaryAttention(Part):
    """params: hidden_size, num_q_heads, num_kv_heads, key_dim, value_dim, eps, scale, softcap (0: none),
    qk_norm (one of QK_NORMS), sink (one of SINKS), position (PartSpec of a position part, or None),
    window (int | None)."""

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
        if params.get("qk_norm") == "weighted_before":
            decl.update(q_norm=WeightDecl((params["key_dim"],), init="ones"), k_norm=WeightDecl((params["key_dim"],), init="ones"))
        if params.get("sink") == "learned":
            decl["sink"] = WeightDecl((params["num_q_heads"],), init="normal")
        return decl

    @classmethod
    def children(cls, params):
        return {"position": ("position", params["position"])} if params.get("position") is not None else {}

    @classmethod
    def declare_cache(cls, params):
        nkv, dk, dv = int(params["num_kv_heads"]), int(params["key_dim"]), int(params["value_dim"])
        return PagedNeed(window=params.get("window"),
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
        self.softcap = float(params.get("softcap") or 0.0)
        self.window = int(params.get("window") or 0)
        self.qk_norm, self.sink_kind = params.get("qk_norm"), params.get("sink")
        if self.qk_norm not in QK_NORMS or self.sink_kind not in SINKS:
            raise ValueError(f"qk_norm is one of {QK_NORMS} and sink one of {SINKS}")
        mats = [tensors[n] for n in ("q", "k", "v")]
        if len({t.dtype for t in mats}) != 1:
            raise ValueError("q, k and v projections must be stored in one type")
        self.widths = self._widths(params)
        self.proj = Linear(torch.cat(mats, dim=0).contiguous(), rt.weight_tiles)
        self.q_norm, self.k_norm = tensors.get("q_norm"), tensors.get("k_norm")
        self.sink = None
        if self.sink_kind == "learned":
            self.sink = tensors["sink"].float().contiguous()
        elif self.sink_kind == "zero":
            self.sink = torch.zeros(self.nq, dtype=torch.float32, device=rt.device)
        self.position = (children or {}).get("position")
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
        cos = sin = None
        rotary_dim, interleaved = 0, False
        if self.position is not None:
            cos, sin, rotary_dim = self.position.fused_rotary()
            interleaved = self.position.kind == "rope_interleaved"
        ops.rotary_qkv_store(q, k, v, num_q_heads=self.nq, num_kv_heads=self.nkv, key_dim=self.Dk, value_dim=self.Dv,
                             eps=self.eps, q_weight=self.q_norm, k_weight=self.k_norm,
                             unit_after=self.qk_norm == "unit_after", cos=cos, sin=sin, rotary_dim=rotary_dim or 0,
                             interleaved=interleaved, positions=batch.positions, slot_of_token=batch.slot_of_token,
                             block_table=cache.block_table, k_pages=cache.pages["k"], v_pages=cache.pages["v"],
                             page_size=cache.page_size)
        out = torch.empty((x.shape[0], self.nq * self.Dv), dtype=x.dtype, device=x.device)
        softcap_attention(q, out, cache, batch, num_q_heads=self.nq, num_kv_heads=self.nkv, key_dim=self.Dk,
                          value_dim=self.Dv, scale=self.scale, softcap=self.softcap, r1=None, r2=None,
                          window=self.window, sink=self.sink)
        return self.o(out, out_dtype=torch.float32, partials_ok=True)   # it goes into the 32-bit residual unrounded
