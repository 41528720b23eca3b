"""Grouped-query attention over a sliding window of a paged cache, without rotation: positions enter through a
query temperature and a penalty on distance.

Per token, with h the mixer's input, nq query heads over nkv key/value heads, key size Dk, value size Dv:

    q, k, v = projections with biases -> short causal convolution over time on every channel (its own state)
    q, k    <- per-head RMS norm over Dk (one weight for all heads)
    q       <- q * (1 + coef ln(floor((p + 1) / every) + 1))                       at position p
    s_ij    = cap tanh(scale (q_i . k_j) / cap) - r1_h ln(1 + r2_h (i - j))         for i - window < j <= i
    out     = W_o concat_h(softmax_j(s) v)

Keys (after convolution and norm) and values (after convolution) go to pages `[nkv, page, Dk]` and
`[nkv, Dv, page]`.  With `shares_kv` the layer has no key and value tensors: the schedule makes it read the pages
of the layer that owns them, with its own queries, window, cap and penalty; its own state is then the
convolution's last inputs of q alone.  The owner keeps keys for the widest window among its readers
(`cache_window`).  Every option can be left out: no biases, no convolution (taps 0), no norm, no temperature
(coef 0), no cap (0), no penalty, no window (None).
"""
from __future__ import annotations

import torch

from ..cache.manager import PAGE, PagedNeed, PageTensor
from ..kernels import ops
from .base import Part, WeightDecl, register
from .linear import Linear
from .short_conv import ShortConv


@register("mixer", "softcap_attention")
class SoftcapAttention(Part):
    """params: hidden_size, num_q_heads, num_kv_heads, key_dim, value_dim, bias (bool), conv_taps (0: none),
    qk_norm (bool), eps, temp_coef, temp_every, scale, softcap (0: none), distance_penalty (bool),
    window (int | None), cache_window (int | None; default window), shares_kv (bool)."""

    graph_safe = True  # positions, slots and lengths are read on the GPU; launches depend on shapes only

    @classmethod
    def _widths(cls, params):
        q = params["num_q_heads"] * params["key_dim"]
        return q, params["num_kv_heads"] * params["key_dim"], params["num_kv_heads"] * params["value_dim"]

    @classmethod
    def declare_weights(cls, params):
        h, dk = params["hidden_size"], params["key_dim"]
        qw, kw, vw = cls._widths(params)
        taps = int(params.get("conv_taps") or 0)
        decl = {"q": WeightDecl((qw, h)), "o": WeightDecl((h, params["num_q_heads"] * params["value_dim"]))}
        names = [("q", qw)]
        if not params.get("shares_kv"):
            decl.update(k=WeightDecl((kw, h)), v=WeightDecl((vw, h)))
            names += [("k", kw), ("v", vw)]
        for name, width in names:
            if params.get("bias"):
                decl[name + "_bias"] = WeightDecl((width,), init="normal")
            if taps:
                decl[name + "_conv"] = WeightDecl((width, taps))
        if params.get("qk_norm"):
            decl["q_norm"] = WeightDecl((dk,), init="ones")
            if not params.get("shares_kv"):
                decl["k_norm"] = WeightDecl((dk,), init="ones")
        if params.get("distance_penalty"):
            decl.update(r1=WeightDecl((params["num_q_heads"],), init="ones"),
                        r2=WeightDecl((params["num_q_heads"],), init="ones"))
        return decl

    @classmethod
    def _conv_need(cls, params, channels):
        return ShortConv.state_need(channels, int(params.get("conv_taps") or 0))

    @classmethod
    def declare_cache(cls, params):
        nkv, dk, dv = int(params["num_kv_heads"]), int(params["key_dim"]), int(params["value_dim"])
        keep = params.get("cache_window", params.get("window"))
        need = {"kv": PagedNeed(window=keep, tensors=(PageTensor("k", (nkv, PAGE, dk)), PageTensor("v", (nkv, dv, PAGE))))}
        conv = cls._conv_need(params, sum(cls._widths(params)))
        if conv is not None:
            need["conv"] = conv
        return need

    @classmethod
    def declare_reader_cache(cls, params):
        conv = cls._conv_need(params, cls._widths(params)[0])
        return {"conv": conv} if conv is not None else None

    def cache_need(self):
        return self.declare_reader_cache(self.params) if self.shares_kv else self.declare_cache(self.params)

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.nq, self.nkv = int(params["num_q_heads"]), int(params["num_kv_heads"])
        self.Dk, self.Dv = int(params["key_dim"]), int(params["value_dim"])
        if self.nkv < 1 or self.nq % self.nkv:
            raise ValueError("num_q_heads must be a multiple of num_kv_heads")
        if not (0 < self.Dk <= ops.MAX_HEAD_DIM and 0 < self.Dv <= ops.MAX_HEAD_DIM):
            raise ValueError(f"head sizes {self.Dk}, {self.Dv} are not supported: the attention kernels take 1..{ops.MAX_HEAD_DIM}")
        self.shares_kv = bool(params.get("shares_kv"))
        self.eps = float(params.get("eps", 0.0))
        self.scale = float(params["scale"])
        self.softcap = float(params.get("softcap") or 0.0)
        self.window = params.get("window")
        self.temp_coef = float(params.get("temp_coef") or 0.0)
        self.temp_every = int(params.get("temp_every") or 1)
        names = ["q"] if self.shares_kv else ["q", "k", "v"]
        mats = [tensors[n] for n in names]
        if len({t.dtype for t in mats}) != 1:
            raise ValueError("q, k and v projections must be stored in one type")
        self.widths = [int(t.shape[0]) for t in mats]
        self.proj = Linear(torch.cat(mats, dim=0).contiguous() if len(mats) > 1 else mats[0], rt.weight_tiles)
        cat = lambda suffix: (torch.cat([tensors[n + suffix] for n in names], dim=0).contiguous()
                              if (names[0] + suffix) in tensors else None)
        self.conv = ShortConv(cat("_conv"), cat("_bias"))
        self.q_norm, self.k_norm = tensors.get("q_norm"), tensors.get("k_norm")
        self.r1, self.r2 = tensors.get("r1"), tensors.get("r2")
        self.o = Linear(tensors["o"], rt.weight_tiles)

    def reader_cache_need(self):
        return self.declare_reader_cache(self.params)

    def products(self):
        if self.proj.weight.dtype != torch.bfloat16:
            return []
        return [("qkv", self.proj.out_features, self.proj.in_features, False, None),
                ("o", self.o.out_features, self.o.in_features, False, "norm")]

    def forward(self, x, batch, cache):
        """x [T, H] -> [T, H], or a float32 stack [S, T, H] to be added in order (see Linear)."""
        kv = cache["kv"]
        if kv.writes == self.shares_kv:
            raise ValueError("a layer that shares keys and values must read another entry's pages, and only such a layer")
        y = self.conv(self.proj(x), batch, cache.get("conv"))
        Q = self.widths[0]
        q = y[:, :Q]
        if self.shares_kv:
            ops.qkv_norm_store(q, None, None, num_q_heads=self.nq, num_kv_heads=0, key_dim=self.Dk, value_dim=self.Dv,
                               eps=self.eps, q_weight=self.q_norm, temp_coef=self.temp_coef, temp_every=self.temp_every,
                               positions=batch.positions)
        else:
            K = self.widths[1]
            ops.qkv_norm_store(q, y[:, Q:Q + K], y[:, Q + K:], num_q_heads=self.nq, num_kv_heads=self.nkv,
                               key_dim=self.Dk, value_dim=self.Dv, eps=self.eps, q_weight=self.q_norm,
                               k_weight=self.k_norm, temp_coef=self.temp_coef, temp_every=self.temp_every,
                               positions=batch.positions, slot_of_token=batch.slot_of_token,
                               block_table=kv.block_table, k_pages=kv.pages["k"], v_pages=kv.pages["v"],
                               page_size=kv.page_size)
        out = torch.empty((x.shape[0], self.nq * self.Dv), dtype=x.dtype, device=x.device)
        softcap_attention(q, out, kv, batch, num_q_heads=self.nq, num_kv_heads=self.nkv, key_dim=self.Dk,
                          value_dim=self.Dv, scale=self.scale, softcap=self.softcap, r1=self.r1, r2=self.r2,
                          window=self.window or 0)
        return self.o(out, out_dtype=torch.float32, partials_ok=True)   # it goes into the 32-bit residual unrounded


def softcap_attention(q, out, kv, batch, *, num_q_heads, num_kv_heads, key_dim, value_dim, scale, softcap, r1, r2,
                      window, chunk=0, sink=None, keep_first=0):
    """Attention of every row of the packed step over its request's pages: bfloat16 pages of sizes the matrix-core
    kernel takes run there; float32 pages, and every other shape, run the fixed-order kernel (the true 32-bit path).
    chunk > 0: a row sees the keys of its own chunk of so many positions only; sink [heads]: a term exp(sink_h) in the
    softmax's denominator; keep_first (with a window): the request's first so many keys stay visible to rows whose
    window has passed them, at their true positions."""
    common = dict(keep_first=keep_first, num_q_heads=num_q_heads, num_kv_heads=num_kv_heads, key_dim=key_dim, value_dim=value_dim,
                  page_size=kv.page_size, scale=scale, softcap=softcap, r1=r1, r2=r2, window=window, chunk=chunk, sink=sink)
    if (ops.attn_softcap_mfma_supported(q.dtype, key_dim, value_dim, kv.page_size, num_q_heads // num_kv_heads)
            and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0
            and not (keep_first and chunk)
            and ops.attn_softcap_mfma_fits(ops.mask_span(window, chunk), kv.block_table.shape[1], kv.page_size, keep_first)):
        ops.attn_softcap_mfma(q, out, kv.pages["k"], kv.pages["v"], kv.block_table, batch.seg_row0, batch.seg_slot,
                              batch.seg_start, max_qlen=batch.max_qlen, **common)
    else:
        ops.attn_softcap_simt(q, out, kv.pages["k"], kv.pages["v"], kv.block_table, batch.positions,
                              batch.slot_of_token, **common)
