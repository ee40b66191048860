"""A feed-forward of routed experts.

    z = W_router f;   the ``top`` largest z are chosen (ties to the lower number), their weights
    are the softmax over the chosen z alone;   y = sum over the chosen e of weight_e expert_e(f)
    (+ sigmoid(w_sg . f) shared(f), an expert that every row takes, when the spec has one)

    expert(f) = W_down (g' sigmoid(alpha g') (u' + 1)),  g' = min(W_gate f, limit),
    u' = W_up f cut to [-limit, limit]                                  ("swish_clamp")
    expert(f) = W_down (silu(W_gate f) W_up f)                          ("silu")
    expert(f) = W_down max(W_up f, 0)^2, an expert without a gate       ("relu_sq")

With ``router_score`` "sigmoid" the scores are s = sigmoid(z), the ``top`` largest s are chosen and
their weights are s times ``router_scale``, not renormalized; "softmax_all": the same with s the
softmax of z over all experts.  With ``groups`` > 1 the experts lie in that many equal groups of
neighbours, a group's score is its best expert's, and only experts of the ``keep_groups`` best groups
can be chosen.  ``shared_gate`` false: the expert
that every row takes is added as it is (no sigmoid gate, no tensor for it).

The router runs in float32 whatever the model's type (its matrix, with the shared expert's gate
row under it, is kept in float32; one kernel makes the scores and the choice).  Choice and weights
are made on the device, and the experts' products find their rows there too: nothing of a step
depends on a value the host has seen, so a decode step can be recorded and replayed.  The experts'
matrices are stacked when the part is built: [experts, 2 * inner, width] (gate over up) and
[experts, width, inner].  The expert that every row takes is a dense feed-forward: its two products
are the framework's own, with the clamped pair applied to the float32 result of the stacked one.

Every (row, choice) pair has its own row of the intermediate and of the result; the pass that
ends the sublayer adds a row's pairs in the order of the choice, times their weights.  A pair's
numbers depend on its row and its expert alone, never on which other rows chose the same expert.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Branch, Part, register_part
from .linear import Linear
from .spec import PartSpec, TensorSpec

EXPERT_ACTIVATIONS = ("swish_clamp", "silu", "relu_sq")
UNGATED = ("relu_sq",)            # experts of two matrices: W_down act(W_up f)
ROUTER_SCORES = ("softmax_chosen", "sigmoid", "softmax_all")


def moe_ffn_spec(prefix: str, width: int, experts: int, top: int, inner: int, limit: float, alpha: float = 1.702,
                 shared_inner: int = 0, shared_limit: float = 0.0, activation: str = "swish_clamp",
                 names=("gate", "up", "down"), expert_prefix: str = "e{}.", router_name: str = "router",
                 shared_prefix: str = "shared.", shared_gate_name: str = "shared.sg", router_score: str = "softmax_chosen",
                 router_scale: float = 1.0, shared_gate: bool = True, groups: int = 1, keep_groups: int = 1) -> PartSpec:
    """``shared_inner`` > 0: an expert of that inner width that every row takes, times the sigmoid of
    one more router row (``shared_gate_name``) unless ``shared_gate`` is false.  Experts without a gate
    (``activation`` one of ``UNGATED``) have no tensor of the first of ``names``."""
    gated = activation not in UNGATED
    tensors = {"router": TensorSpec(prefix + router_name, (experts, width))}
    for e in range(experts):
        ep = prefix + expert_prefix.format(e)
        if gated:
            tensors[f"e{e}.gate"] = TensorSpec(ep + names[0], (inner, width))
        tensors[f"e{e}.up"] = TensorSpec(ep + names[1], (inner, width))
        tensors[f"e{e}.down"] = TensorSpec(ep + names[2], (width, inner))
    if shared_inner:
        sp = prefix + shared_prefix
        if gated:
            tensors["shared.gate"] = TensorSpec(sp + names[0], (shared_inner, width))
        tensors["shared.up"] = TensorSpec(sp + names[1], (shared_inner, width))
        tensors["shared.down"] = TensorSpec(sp + names[2], (width, shared_inner))
        if shared_gate:
            tensors["shared.sg"] = TensorSpec(prefix + shared_gate_name, (1, width))
    return PartSpec("ffn", "moe", {"width": width, "experts": experts, "top": top, "inner": inner, "limit": float(limit),
                                   "alpha": float(alpha), "shared_inner": int(shared_inner),
                                   "shared_limit": float(shared_limit), "activation": activation,
                                   "router_score": router_score, "router_scale": float(router_scale),
                                   "shared_gate": bool(shared_gate), "groups": int(groups),
                                   "keep_groups": int(keep_groups)}, tensors)


def _stack(mats):
    if any(m.dtype != mats[0].dtype for m in mats):
        mats = [m.float() for m in mats]
    return torch.stack(mats, dim=0).contiguous()


@register_part("ffn", "moe")
class MoEFFN(Part):
    category = "ffn"
    graph_safe = True     # its launches depend on device buffers only

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.width, self.experts, self.top, self.inner = int(p["width"]), int(p["experts"]), int(p["top"]), int(p["inner"])
        self.limit, self.alpha = float(p["limit"]), float(p.get("alpha", 1.702))
        self.shared_inner, self.shared_limit = int(p.get("shared_inner", 0)), float(p.get("shared_limit", 0.0))
        self.activation = p.get("activation", "swish_clamp")
        if self.activation not in EXPERT_ACTIVATIONS:
            raise ValueError(f"unknown expert activation {p.get('activation')!r}; known: {EXPERT_ACTIVATIONS}")
        self.router_score, self.router_scale = p.get("router_score", "softmax_chosen"), float(p.get("router_scale", 1.0))
        if self.router_score not in ROUTER_SCORES:
            raise ValueError(f"unknown kind of router score {self.router_score!r}; known: {ROUTER_SCORES}")
        self.shared_gate = bool(p.get("shared_gate", True)) and bool(int(p.get("shared_inner", 0)))
        if not 0 < self.top <= self.experts:
            raise ValueError(f"{self.top} choices of {self.experts} experts")
        self.groups, self.keep_groups = int(p.get("groups", 1) or 1), int(p.get("keep_groups", 1) or 1)
        if self.groups > 1:
            if self.experts % self.groups or not 0 < self.keep_groups <= self.groups:
                raise ValueError(f"{self.keep_groups} of {self.groups} groups do not fit {self.experts} experts")
            if self.keep_groups * (self.experts // self.groups) < self.top:
                raise ValueError(f"{self.keep_groups} groups of {self.experts // self.groups} experts hold fewer than the "
                                 f"{self.top} a row chooses")
        self.gated = self.activation not in UNGATED
        if self.top > ops.MOE_MAX_TOP:
            raise ValueError(f"{self.top} choices a row are more than the router kernel's {ops.MOE_MAX_TOP}")
        rows = [tensors["router"].float()]
        if self.shared_gate:
            rows.append(tensors["shared.sg"].float().reshape(1, self.width))
        self.router = torch.cat(rows, dim=0).contiguous()        # float32, the shared expert's gate row last
        if self.gated:
            self.w_in = ops.MoEWeight(_stack([torch.cat([tensors[f"e{e}.gate"], tensors[f"e{e}.up"]], dim=0)
                                              for e in range(self.experts)]), gated=True, fast=rt.fast_kernels)
        else:
            self.w_in = ops.MoEWeight(_stack([tensors[f"e{e}.up"] for e in range(self.experts)]), fast=rt.fast_kernels)
        self.w_out = ops.MoEWeight(_stack([tensors[f"e{e}.down"] for e in range(self.experts)]), fast=rt.fast_kernels)
        # the expert that every row takes is a dense feed-forward: the framework's own products, with the
        # clamped pair applied to the float32 result of the stacked one
        self.s_in = self.s_out = None
        if self.shared_inner and not self.gated:
            self.s_in = Linear(tensors["shared.up"], None, rt.fast_kernels)
            self.s_out = Linear(tensors["shared.down"], None, rt.fast_kernels)
        elif self.shared_inner:
            g, u = tensors["shared.gate"], tensors["shared.up"]
            if g.dtype != u.dtype:
                g, u = g.float(), u.float()
            # (the plain silu pair is the gated product of the dense feed-forwards, applied in the product's epilogue)
            self.s_in = Linear(torch.cat([g, u], dim=0), None, rt.fast_kernels, gated=self.activation == "silu")
            self.s_out = Linear(tensors["shared.down"], None, rt.fast_kernels)

    def produce(self, h, ctx):
        """The pairs' results [rows, top, width] with their weights, and the shared expert's with its
        gate, for the pass that adds them up."""
        act = self.rt.act_dtype
        n = h.shape[0]
        ids, weights = ops.moe_router(h, self.router, self.experts, self.top, has_gate=self.shared_gate,
                                      score=self.router_score, score_scale=self.router_scale, groups=self.groups,
                                      keep_groups=self.keep_groups)
        plan = ops.moe_plan(ids, self.experts)
        if self.gated:
            mid = ops.moe_product(h, self.w_in, plan, self.top, act, self.limit, self.alpha, pair=self.activation)   # [n * top, inner]
        else:
            mid = ops.moe_product(h, self.w_in, plan, self.top, act, single=self.activation)
        out = ops.moe_product(mid, self.w_out, plan, 1, torch.float32)                         # [n * top, width]
        branch = Branch(out.view(n, self.top, self.width), by_row=True, part_weights=weights[:, : self.top])
        if self.shared_inner:
            if not self.gated:
                smid = ops.activate(self.s_in(h, torch.float32), act, self.activation)
            elif self.activation == "silu":
                smid = self.s_in.gated_product(h, act)
            else:
                smid = ops.swish_clamp_mul(self.s_in(h, torch.float32), act, self.shared_limit, self.alpha)
            branch.extra = self.s_out(smid, torch.float32)
            branch.extra_weights = weights[:, self.top:] if self.shared_gate else None
        return branch

    def forward(self, h, x, ctx, then_norm=None):
        """x += moe(h)."""
        b = self.produce(h, ctx)
        ops.norm_add(x, b.part, None, 0.0, 0.0, None, part_weights=b.part_weights, extra=b.extra,
                     extra_weights=b.extra_weights, by_row=True, norm=False)
        return None
