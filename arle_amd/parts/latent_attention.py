"""Latent attention: every token caches one compressed vector c and one rotated key part shared by all heads.

Per token, with h the mixer's input, H heads, per head D unrotated and R rotated query/key entries, value size Dv,
latent size C:

    q = W_q h, head by head [D unrotated | R rotated];     W_dkv h = [C entries | R entries]
    c = rms_norm(first C entries) * w_c;                    k_rot = rotate(last R entries)        (one for all heads)
    k_h = W_uk,h c,  v_h = W_uv,h c
    s_ij,h = scale (q_h,i . k_h,j + rotate(q_rot,h,i) . k_rot,j)    for 0 <= i - j < window  (None: every j <= i)
    p = exp(s) / (sum_j exp(s_ij) + exp(sink_h))            (sink: a learned number a head, optional)
    out = W_o (concat_h(sum_j p_j v_h,j) * sigmoid(W_g h))          (the gate: optional)

The maps W_uk and W_uv are folded into the query and the output: q'_h = W_uk,h^T q_h, so that
s = scale (q'_h . c + q_rot . k_rot), and out_h = W_uv,h (sum_j p_j c_j).  The attention is then one of H query heads
over a single key/value head with keys [c | k_rot] and values c, which is what the pages hold
(`[1, page, C + R]`, and c once more d-major `[1, C, page]` as the second operand of the matrix cores); keys and
values of the heads are never formed.  The rotation is a position part (`rope_interleaved`, pairs (2i, 2i + 1), or
`rope_neox`, pairs (i, i + R'/2) over the first R' rotated entries) whose table the preparation kernel reads.
"""
from __future__ import annotations

import torch

from ..cache.manager import PAGE, PagedNeed, PageTensor
from ..kernels import ops
from .base import Part, WeightDecl, register
from .linear import Linear
from .softcap_attention import softcap_attention


@register("mixer", "latent_attention")
class LatentAttention(Part):
    """params: hidden_size, heads, dim, rot_dim, value_dim, rank, eps, scale, window (int | None), sink (bool),
    gate (bool: a sigmoid gate on the heads' outputs, a projection of the mixer's input), position (PartSpec of the
    rotation over the rot_dim part)."""

    graph_safe = True  # positions, slots and lengths are read on the GPU; launches depend on shapes only

    @classmethod
    def declare_weights(cls, params):
        h, H = params["hidden_size"], params["heads"]
        D, R, Dv, C = params["dim"], params["rot_dim"], params["value_dim"], params["rank"]
        decl = {"q": WeightDecl((H * (D + R), h)), "dkv": WeightDecl((C + R, h)), "c_norm": WeightDecl((C,), init="ones"),
                "uk": WeightDecl((H * D, C)), "uv": WeightDecl((H * Dv, C)), "o": WeightDecl((h, H * Dv))}
        if params.get("sink"):
            decl["sink"] = WeightDecl((H,), init="normal")
        if params.get("gate"):
            decl["g"] = WeightDecl((H * Dv, h))
        return decl

    @classmethod
    def children(cls, params):
        return {"position": ("position", params["position"])}

    @classmethod
    def declare_cache(cls, params):
        C, R = int(params["rank"]), int(params["rot_dim"])
        return PagedNeed(window=params.get("window"),
                         tensors=(PageTensor("k", (1, PAGE, C + R)), PageTensor("v", (1, C, PAGE))))

    def cache_need(self):
        return self.declare_cache(self.params)

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.H, self.D, self.R = int(params["heads"]), int(params["dim"]), int(params["rot_dim"])
        self.Dv, self.C = int(params["value_dim"]), int(params["rank"])
        if not (0 < self.C + self.R <= ops.CAP_SIMT_MAX_DIM):
            raise ValueError(f"latent and rotated sizes {self.C} + {self.R} are not supported: the attention kernels "
                             f"take keys of 1..{ops.CAP_SIMT_MAX_DIM}")
        if max(self.D, self.C) > ops.HEAD_PROJ_MAX_K:
            raise ValueError(f"head and latent sizes up to {ops.HEAD_PROJ_MAX_K} are taken")
        self.eps = float(params.get("eps", 0.0))
        self.scale = float(params["scale"])
        self.window = int(params.get("window") or 0)
        self.position = children["position"]
        wq, wd = tensors["q"], tensors["dkv"]
        self.gated = bool(params.get("gate"))
        fused = [wq, wd] + ([tensors["g"]] if self.gated else [])
        if len({t.dtype for t in fused} | {tensors["uk"].dtype, tensors["uv"].dtype}) != 1:
            raise ValueError("the projections of a latent attention must be stored in one type")
        self.q_width = self.H * (self.D + self.R)
        self.dkv_width = self.C + self.R
        self.proj = Linear(torch.cat(fused, dim=0).contiguous(), rt.weight_tiles)
        self.c_norm = tensors["c_norm"]
        # a matrix a head, stored [inner, outer]: q'_h = q_h W_uk,h (W_uk,h is [D, C] as it lies), out_h = lat_h W_uv,h^T
        # (the matrix-core form of the product reads the other layout, [outer, inner]; only the one that runs is kept)
        uk, uv = tensors["uk"].view(self.H, self.D, self.C), tensors["uv"].view(self.H, self.Dv, self.C)
        self.on_matrix_cores = (uk.dtype == torch.bfloat16 and self.D % 8 == 0 and self.C % 8 == 0 and self.R % 8 == 0
                                and self.q_width % 8 == 0 and (self.C + self.R) % 8 == 0)
        if self.on_matrix_cores:
            self.uk_nk, self.uv_nk = uk.transpose(1, 2).contiguous(), uv
        else:
            self.uk, self.uv_t = uk, uv.transpose(1, 2).contiguous()
        self.sink = tensors.get("sink")
        self.o = Linear(tensors["o"], rt.weight_tiles)

    def products(self):
        if self.proj.weight.dtype != torch.bfloat16:
            return []
        return [("q_dkv_g" if self.gated else "q_dkv", self.proj.out_features, self.proj.in_features, False, None),
                ("o", self.o.out_features, self.o.in_features, False, "norm")]

    def _per_head(self, x, which, out, *, in_head, out_head):
        """out[:, head] = x[:, head] . (W_uk,h or W_uv,h^T), a matrix a head."""
        if self.on_matrix_cores and ops.head_proj_mfma_supported(x, self.H, in_head, self.D if which == "uk" else self.C):
            ops.head_proj_mfma(x, self.uk_nk if which == "uk" else self.uv_nk, out, heads=self.H, in_head=in_head, out_head=out_head)
        elif self.on_matrix_cores:      # operands that are not aligned for it after all: the plain kernel, from a turned copy
            w = (self.uk_nk if which == "uk" else self.uv_nk).transpose(1, 2).contiguous()
            ops.head_proj(x, w, out, heads=self.H, in_head=in_head, out_head=out_head)
        else:
            ops.head_proj(x, self.uk if which == "uk" else self.uv_t, out, heads=self.H, in_head=in_head, out_head=out_head)

    def forward(self, x, batch, cache):
        """x [T, H] -> float32 [T, H], or a float32 stack [S, T, H] to be added in order (see Linear)."""
        if not cache.writes:
            raise ValueError("a latent attention keeps a cache of its own")
        H, D, R, C, Dv = self.H, self.D, self.R, self.C, self.Dv
        self.position.ensure_positions(batch.max_position + 1)
        cos, sin, rot = self.position.fused_rotary()
        y = self.proj(x)
        q, dkv = y[:, :self.q_width], y[:, self.q_width:self.q_width + self.dkv_width]
        q_full = torch.empty((x.shape[0], H * (C + R)), dtype=x.dtype, device=x.device)
        ops.latent_prep(q, dkv, q_full, heads=H, dim=D, rot_dim=R, rank=C, c_weight=self.c_norm, eps=self.eps, cos=cos,
                        sin=sin, rotary_dims=rot, positions=batch.positions, slot_of_token=batch.slot_of_token,
                        block_table=cache.block_table, k_pages=cache.pages["k"], v_pages=cache.pages["v"],
                        page_size=cache.page_size, halves=self.position.kind != "rope_interleaved")
        self._per_head(q, "uk", q_full, in_head=D + R, out_head=C + R)
        latent = torch.empty((x.shape[0], H * C), dtype=x.dtype, device=x.device)
        softcap_attention(q_full, latent, cache, batch, num_q_heads=H, num_kv_heads=1, key_dim=C + R, value_dim=C,
                          scale=self.scale, softcap=0.0, r1=None, r2=None, window=self.window, sink=self.sink)
        heads_out = torch.empty((x.shape[0], H * Dv), dtype=x.dtype, device=x.device)
        self._per_head(latent, "uv", heads_out, in_head=C, out_head=Dv)
        if self.gated:
            heads_out = ops.gate_mul(y[:, self.q_width + self.dkv_width:], heads_out, ops.ACT_SIGMOID)
        return self.o(heads_out, out_dtype=torch.float32, partials_ok=True)   # into the 32-bit residual unrounded
