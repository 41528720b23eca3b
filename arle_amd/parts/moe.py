"""A mixture of experts with a sigmoid or softmax router, and an optional shared expert that every token uses.

    z = W_r h (32-bit),  s = sigmoid(z) or softmax(z);  the `top` experts with the largest s + correction are chosen,
    with `groups`: only among the experts of the `keep_groups` groups of neighbours that hold the largest such numbers;
    weight_e = s_e / (sum of the chosen s + 1e-20) * scale, or without `normalize` s_e * scale;
    expert: down(silu(gate h) * (up h)), no biases; the last `identity` outputs of the router stand for experts without
    tensors that hand back h itself;
    out = sum over the chosen experts of weight_e expert_e(h)  +  shared(h)

The router's kernel leaves the chosen experts and their weights on the GPU; the experts' kernel finds, workgroup by
workgroup, the rows that chose its expert, so no step sorts rows or reads anything back and its launches follow the
number of rows alone.  The experts' outputs stay apart, one row a (token, choice), in float32: the norm behind the
feed-forward weighs and adds them in the order of the choices, in the pass that computes its statistics
(`forward` returns the addends, not their sum).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, PartSpec, WeightDecl, register


@register("feed_forward", "sigmoid_moe")
class SigmoidMoE(Part):
    """params: hidden_size, experts (those with tensors), top, expert_size, scale, correction (bool),
    shared_size (int | None), score ("sigmoid", the default, or "softmax"), normalize (bool, default True),
    groups (default 1), keep_groups (default 1), identity (default 0: router outputs behind the experts' that stand
    for experts which hand back their input; groups and the softmax run over experts and these together)."""

    graph_safe = True  # launches depend on shapes only; what a token chose is read on the GPU

    @classmethod
    def declare_weights(cls, params):
        h, i, E = params["hidden_size"], params["expert_size"], params["experts"]
        outputs = E + int(params.get("identity") or 0)
        decl = {"router": WeightDecl((outputs, h))}
        if params.get("correction"):
            decl["correction"] = WeightDecl((outputs,), init="normal")
        for e in range(E):
            decl.update({f"gate{e}": WeightDecl((i, h)), f"up{e}": WeightDecl((i, h)), f"down{e}": WeightDecl((h, i))})
        return decl

    @classmethod
    def children(cls, params):
        if not params.get("shared_size"):
            return {}
        shared = PartSpec("swiglu", {"hidden_size": params["hidden_size"], "intermediate_size": params["shared_size"],
                                     "float32_out": True}, params["shared_weights"])
        return {"shared": ("feed_forward", shared)}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.E, self.top = int(params["experts"]), int(params["top"])
        self.identity = int(params.get("identity") or 0)
        outputs = self.E + self.identity
        self.score = params.get("score") or "sigmoid"
        self.normalize = bool(params.get("normalize", True))
        self.groups, self.keep_groups = int(params.get("groups") or 1), int(params.get("keep_groups") or 1)
        if self.score not in ("sigmoid", "softmax"):
            raise ValueError("a router's scores are sigmoid or softmax")
        if self.E < 1 or self.identity < 0 or not 1 <= self.top <= outputs:
            raise ValueError("a token chooses between 1 and all of the experts")
        if outputs > ops.MOE_MAX_EXPERTS or self.top > ops.MOE_MAX_TOP:
            raise ValueError(f"up to {ops.MOE_MAX_EXPERTS} experts and {ops.MOE_MAX_TOP} choices a token are taken")
        if (self.groups < 1 or outputs % self.groups or not 1 <= self.keep_groups <= self.groups
                or self.top > self.keep_groups * (outputs // self.groups)):
            raise ValueError("groups divide the router's outputs evenly, and the kept groups hold at least `top` of them")
        self.scale = float(params.get("scale", 1.0))
        self.router = tensors["router"]
        self.correction = tensors.get("correction")
        E = self.E
        kinds = {tensors[f"{n}{e}"].dtype for n in ("gate", "up", "down") for e in range(E)}
        if len(kinds) != 1:
            raise ValueError("the experts' projections must be stored in one type")
        # one tensor for all experts: [E, 2I, H] (an expert's gate rows, then its up rows) and [E, H, I]
        self.gate_up = torch.stack([torch.cat([tensors[f"gate{e}"], tensors[f"up{e}"]], dim=0) for e in range(E)]).contiguous()
        self.down = torch.stack([tensors[f"down{e}"] for e in range(E)]).contiguous()
        self.shared = (children or {}).get("shared")

    def forward(self, x):
        """x [T, H] -> the addends of the output: [(outputs float32 [T, top, H], weights float32 [T, top])] and, with
        a shared expert, its output (float32 [T, H] or a float32 stack of partial sums)."""
        w_dtype = self.gate_up.dtype
        xe = x if x.dtype == w_dtype else x.to(w_dtype)
        ids, weights = ops.moe_route(x, self.router, self.correction, top=self.top, scale=self.scale, score=self.score,
                                     groups=self.groups, keep_groups=self.keep_groups, normalize=self.normalize)
        act = ops.moe_expert(xe, self.gate_up, ids, gate_up=True)
        outs = ops.moe_expert(act, self.down, ids, gate_up=False)
        if self.identity:
            ops.moe_identity(x, ids, outs, self.E)
        terms = [(outs.view(x.shape[0], self.top, -1), weights)]
        if self.shared is not None:
            terms.append(self.shared.forward(x))
        return terms
