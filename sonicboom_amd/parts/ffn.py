"""Dense feed-forwards, gated and plain.

``gated_dense``: y = W_down (act(W_gate f) * (W_up f)).

/root/reference/core/src/model/emit.cpp:364-374; the activation is a parameter
of the spec: "silu", g / (1 + exp(-g)) (/root/reference/core/src/nn/activation.cpp:41-50),
"gelu_tanh", 0.5 g (1 + tanh(sqrt(2/pi) g (1 + 0.044715 g^2))) (:27-36), or "relu", max(g, 0); the product
kernels apply either in their epilogue.  The gate and up matrices
are stacked into one [2*inner, width] matrix when the part is built, so a
step runs one product for both; its float32 result feeds the activation
kernel, whose output is rounded once to the activation type.

``dense``: y = W_down act(W_up f + b_up) + b_down (biases when the spec names them), the activation one
of ``ops.ACTIVATIONS`` ("gelu_erf": z Phi(z) by the error function; "relu_sq": max(z, 0)^2); "xielu" reads its two
numbers (p, q) from a tensor of the layer: softplus(p) z^2 + z/2 for z > 0 and
(1/2 + softplus(q)) (exp(z) - 1 - z) + z/2 else.  The up product leaves in float32, the activation
kernel rounds once to the activation type.

Both add ``out_scale`` times their result into the stream (1 unless the spec says otherwise).
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Part, register_part
from .linear import Linear
from .spec import PartSpec, TensorSpec

ACTIVATIONS = ("silu", "gelu_tanh", "relu")    # the gates the product kernels apply in their epilogue


def gated_ffn_spec(prefix: str, width: int, inner: int, activation: str = "silu", out_scale: float = 1.0,
                   names=("gate_proj.weight", "up_proj.weight", "down_proj.weight")) -> PartSpec:
    """``names``: what the file calls the gate, up and down matrices after ``prefix``."""
    return PartSpec("ffn", "gated_dense", {"width": width, "inner": inner, "activation": activation,
                                           "out_scale": float(out_scale)}, {
        "gate_weight": TensorSpec(prefix + names[0], (inner, width)),
        "up_weight": TensorSpec(prefix + names[1], (inner, width)),
        "down_weight": TensorSpec(prefix + names[2], (width, inner)),
    })


@register_part("ffn", "gated_dense")
class GatedDenseFFN(Part):
    category = "ffn"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.width, self.inner = int(p["width"]), int(p["inner"])
        self.activation = p.get("activation", "silu")
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r}; known: {ACTIVATIONS}")
        g, u = tensors["gate_weight"], tensors["up_weight"]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.gate_up = Linear(torch.cat([g, u], dim=0), None, rt.fast_kernels, gated=True,
                              activation=self.activation)
        self.down = Linear(tensors["down_weight"], None, rt.fast_kernels)
        self.out_scale = float(p.get("out_scale", 1.0))

    fuses_norm = True
    graph_safe = True     # its launches depend on device buffers only

    def forward(self, h, x, ctx, then_norm=None):
        """x += out_scale * ffn(h).  Returns then_norm(x) when the down projection could apply the
        norm in its last pass, else None."""
        mid = self.gate_up.gated_product(h, self.rt.act_dtype)
        return self.down.add_into(mid, x, then_norm, self.rt.act_dtype, scale=self.out_scale)

    def produce(self, h, ctx):
        """ffn(h) in float32 (whole, or in K slices), for a block that adds it up itself."""
        if self.out_scale != 1.0:
            raise ValueError("a feed-forward that hands its result over has no multiplier of its own")
        return self.down.raw(self.gate_up.gated_product(h, self.rt.act_dtype))


def dense_ffn_spec(up_name: str, down_name: str, width: int, inner: int, activation: str,
                   act_name: str = None, out_scale: float = 1.0, up_bias_name: str = None,
                   down_bias_name: str = None) -> PartSpec:
    """``act_name``: the tensor that holds the activation's numbers (xIELU's two); ``up_bias_name``,
    ``down_bias_name``: the biases of the two products, for feed-forwards that have them."""
    tensors = {"up_weight": TensorSpec(up_name, (inner, width)), "down_weight": TensorSpec(down_name, (width, inner))}
    if act_name is not None:
        tensors["act_params"] = TensorSpec(act_name, (2,), init=(0.0, 0.5))
    if up_bias_name is not None:
        tensors["up_bias"] = TensorSpec(up_bias_name, (inner,), init=(0.0, 0.02))
    if down_bias_name is not None:
        tensors["down_bias"] = TensorSpec(down_bias_name, (width,), init=(0.0, 0.02))
    return PartSpec("ffn", "dense", {"width": width, "inner": inner, "activation": activation,
                                     "out_scale": float(out_scale)}, tensors)


@register_part("ffn", "dense")
class DenseFFN(Part):
    category = "ffn"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.width, self.inner = int(p["width"]), int(p["inner"])
        self.activation = p["activation"]
        if self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r}; known: {sorted(ops.ACTIVATIONS)}")
        self.act_params = tensors.get("act_params")
        if self.activation == "xielu" and self.act_params is None:
            raise ValueError("xIELU needs the tensor with its two numbers")
        up_b, down_b = tensors.get("up_bias"), tensors.get("down_bias")
        self.up = Linear(tensors["up_weight"], None if up_b is None else up_b.float(), rt.fast_kernels)
        self.down = Linear(tensors["down_weight"], None if down_b is None else down_b.float(), rt.fast_kernels)
        self.out_scale = float(p.get("out_scale", 1.0))

    fuses_norm = True
    graph_safe = True     # its launches depend on device buffers only

    def forward(self, h, x, ctx, then_norm=None):
        """x += out_scale * (W_down act(W_up h + b_up) + b_down).  Returns then_norm(x) when the down projection could
        apply the norm in its last pass, else None."""
        mid = ops.activate(self.up(h, torch.float32), self.rt.act_dtype, self.activation, self.act_params)
        return self.down.add_into(mid, x, then_norm, self.rt.act_dtype, scale=self.out_scale)
