"""Position encodings applied to queries and keys.

`rope_neox`: half-split rotary encoding over the first `rotary_dim` dims of a head
(all of them for Qwen3): inv_freq_i = theta^(-2i/rotary_dim), angle = pos * inv_freq_i,
pairs (i, i + rotary_dim/2).  infer/src/weight_loader.rs:955-989 builds the same table
(and then narrows it to bf16, which this engine does not: angles, cos and sin stay
32-bit); rotation as crates/cuda-kernels/csrc/attention/prefill_attention_paged_prep.cu:60-76.
`rope_interleaved`: the same angles with entry 2i paired with entry 2i + 1; it only keeps the table, which the
kernel of the mixer that names it applies.
Both take an optional `scaling` (YaRN): the frequencies of the slowly turning pairs are divided by a factor, those of
the fast ones kept, with a linear ramp between two border pairs, and cos and sin are multiplied by 0.1 ln(factor) + 1.
`none`: no position encoding.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, register


def yarn_ramp(rotary_dim: int, theta: float, original: float, fast: float, slow: float):
    """float32 [rotary_dim/2]: 0 for the pairs that keep their frequency, 1 for those that are slowed down by the
    whole factor.  A pair that turns t times over `original` positions has the index
    dim(t) = rotary_dim ln(original / (2 pi t)) / (2 ln theta); the ramp rises from lo = max(floor(dim(fast)), 0) to
    hi = min(ceil(dim(slow)), rotary_dim - 1), at least 0.001 apart."""
    import math

    at = lambda turns: rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))
    lo = max(math.floor(at(fast)), 0)
    hi = min(math.ceil(at(slow)), rotary_dim - 1)
    i = torch.arange(rotary_dim // 2, dtype=torch.float32)
    return torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)


def rope_table(rotary_dim: int, theta: float, positions: int, scaling=None):
    """(cos, sin), each float32 [positions, rotary_dim/2] on the CPU: angle(pos, i) = pos * theta^(-2i/rotary_dim).
    scaling = (factor, original, fast, slow): frequency f_i / factor * ramp_i + f_i (1 - ramp_i), and cos and sin times
    0.1 ln(factor) + 1.

    float32 throughout, as the reference computes it on the host (infer/src/weight_loader.rs:963-981).
    """
    import math

    half = rotary_dim // 2
    base = torch.tensor(float(theta), dtype=torch.float32)
    exponent = torch.arange(half, dtype=torch.float32) * 2.0 / float(rotary_dim)
    inv_freq = 1.0 / torch.pow(base, exponent)
    magnitude = 1.0
    if scaling is not None:
        factor, original, fast, slow = (float(x) for x in scaling)
        ramp = yarn_ramp(rotary_dim, float(theta), original, fast, slow)
        inv_freq = inv_freq / factor * ramp + inv_freq * (1.0 - ramp)
        magnitude = 0.1 * math.log(factor) + 1.0
    angle = torch.arange(positions, dtype=torch.float32)[:, None] * inv_freq[None, :]
    cos, sin = torch.cos(angle), torch.sin(angle)
    if magnitude != 1.0:
        cos, sin = cos * magnitude, sin * magnitude
    return cos.contiguous(), sin.contiguous()


@register("position", "rope_neox")
class RopeNeox(Part):
    """params: head_dim, rotary_dim (default head_dim), theta, max_positions, scaling (None, or the YaRN numbers
    (factor, original, fast, slow))."""

    fusable = True  # the q/k preparation kernel applies this encoding itself

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.head_dim = int(params["head_dim"])
        self.rotary_dim = int(params.get("rotary_dim", self.head_dim))
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError("rotary_dim must be even and in 1..head_dim")
        self.theta = float(params["theta"])
        self.scaling = tuple(float(x) for x in params["scaling"]) if params.get("scaling") else None
        self.cos, self.sin = self._table(int(params["max_positions"]))

    # layers with the same encoding share one table: (device, rotary_dim, theta, positions) -> (cos, sin)
    _shared: dict = {}

    def _table(self, positions: int):
        key = (str(self.rt.device), self.rotary_dim, self.theta, positions, self.scaling)
        if key not in RopeNeox._shared:
            RopeNeox._shared[key] = self._make_table(positions)
        return RopeNeox._shared[key]

    def _make_table(self, positions: int):
        cos, sin = rope_table(self.rotary_dim, self.theta, positions, self.scaling)
        return cos.to(self.rt.device), sin.to(self.rt.device)

    def ensure_positions(self, n: int) -> None:
        """Grow the table if a request runs past what it was sized for."""
        if n > self.cos.shape[0]:
            self.cos, self.sin = self._table(max(n, 2 * self.cos.shape[0]))

    def prepare(self, max_positions: int) -> None:
        self.ensure_positions(max_positions)

    def fused_rotary(self):
        return self.cos, self.sin, self.rotary_dim

    def apply(self, q, k, positions, num_q_heads, num_kv_heads):
        ops.qk_prep(q, k, k, num_q_heads=num_q_heads, num_kv_heads=num_kv_heads,
                    head_dim=self.head_dim, eps=0.0, cos=self.cos, sin=self.sin,
                    rotary_dim=self.rotary_dim, positions=positions)


@register("position", "rope_interleaved")
class RopeInterleaved(RopeNeox):
    """params: head_dim (size of the vector that is rotated), rotary_dim (its first entries that rotate; default all),
    theta, max_positions.  The pair (u, v) = (x[2i], x[2i+1]) at position p becomes (u cos a - v sin a,
    v cos a + u sin a), a = p theta^(-2i/rotary_dim).  The q/k preparation of the rotate-half layout does not know
    this pairing, so `fusable` is False and `apply` refuses: a mixer reads `fused_rotary()` and rotates itself."""

    fusable = False

    def apply(self, q, k, positions, num_q_heads, num_kv_heads):
        raise NotImplementedError("rope_interleaved is applied by the kernels of the mixer that names it")


@register("position", "none")
class NoPosition(Part):
    fusable = True  # nothing to apply
    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)

    def ensure_positions(self, n: int) -> None:
        pass

    def fused_rotary(self):
        return None, None, 0

    def apply(self, q, k, positions, num_q_heads, num_kv_heads):
        pass
