"""Token embedding and the output head.

Embedding: a row lookup into the float32 residual stream, no scale
(/root/reference/core/src/model/emit.cpp:237-248).  Head: logits = W h in
float32; the matrix is the embedding table when the spec says the model ties
them (/root/reference/core/src/model/exec.cpp:516-517).
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Part, register_part
from .linear import Linear
from .spec import PartSpec, TensorSpec


def embedding_spec(name: str, vocab: int, width: int) -> PartSpec:
    return PartSpec("embedding", "lookup", {"vocab": vocab, "width": width},
                    {"table": TensorSpec(name, (vocab, width))})


def head_spec(name: str, vocab: int, width: int, scale: float = 1.0, softcap: float = 0.0) -> PartSpec:
    """``name`` may be the embedding table's name: the head then shares it.  ``scale`` multiplies the logits;
    ``softcap`` > 0: they then become softcap * tanh(logits / softcap)."""
    return PartSpec("head", "linear", {"vocab": vocab, "width": width, "scale": float(scale), "softcap": float(softcap)},
                    {"weight": TensorSpec(name, (vocab, width))})


def positional_embedding_spec(name: str, vocab: int, width: int, scale: float = 1.0, positions_name: str = None,
                              n_positions: int = 0, norm_name: str = None, eps: float = 0.0,
                              norm_offset: float = 0.0) -> PartSpec:
    """x = table[id] * scale (+ positions[p], a learned row per position, not scaled), then, with
    ``norm_name``, the RMS norm of that row times (norm_offset + weight)."""
    tensors = {"table": TensorSpec(name, (vocab, width))}
    if positions_name is not None:
        tensors["positions"] = TensorSpec(positions_name, (n_positions, width))
    if norm_name is not None:
        tensors["norm_weight"] = TensorSpec(norm_name, (width,), init=(1.0 - float(norm_offset), 0.02))
    return PartSpec("embedding", "positional", {"vocab": vocab, "width": width, "scale": float(scale),
                                                "n_positions": int(n_positions), "eps": float(eps),
                                                "norm_offset": float(norm_offset)}, tensors)


@register_part("embedding", "lookup")
class Embedding(Part):
    category = "embedding"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        self.table = tensors["table"]
        self.vocab, self.width = self.table.shape

    def forward(self, ids: torch.Tensor, ctx=None) -> torch.Tensor:
        """``ctx``: the step's context, for embeddings that look at more than the ids (the
        rows' positions, say); this one does not."""
        return ops.embed(self.table, ids)


@register_part("embedding", "positional")
class PositionalEmbedding(Part):
    """Token rows times a multiplier, plus a learned row per position, then optionally normed: one kernel."""
    category = "embedding"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        self.table = tensors["table"]
        self.vocab, self.width = self.table.shape
        self.positions = tensors.get("positions")
        self.norm_weight = tensors.get("norm_weight")
        p = spec.params
        self.scale, self.eps, self.norm_offset = float(p.get("scale", 1.0)), float(p.get("eps", 0.0)), float(p.get("norm_offset", 0.0))
        self.n_positions = self.positions.shape[0] if self.positions is not None else 0

    def forward(self, ids: torch.Tensor, ctx=None) -> torch.Tensor:
        row_pos = ctx.row_pos if self.positions is not None else None
        x, copy = ops.embed_pos_norm(self.table, ids, self.scale, self.positions, row_pos, self.norm_weight, self.eps,
                                     self.norm_offset, norm=self.norm_weight is not None, copy_dtype=self.rt.act_dtype)
        shared = getattr(ctx, "shared", None)
        if copy is not None and shared is not None:
            shared["stream"] = (x, copy)        # the stream in the activation type, for a first block that reads it as it is
        return x


@register_part("head", "linear")
class LinearHead(Part):
    category = "head"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        self.proj = Linear(tensors["weight"], None, rt.fast_kernels)
        self.vocab = int(spec.params["vocab"])
        self.scale = float(spec.params.get("scale", 1.0))
        self.softcap = float(spec.params.get("softcap", 0.0) or 0.0)
        if self.softcap < 0:
            raise ValueError("the logits' cap must not be negative")

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        logits = self.proj(h, torch.float32)
        if self.scale != 1.0:
            logits = ops.scale_(logits, self.scale)
        return ops.softcap_(logits, self.softcap) if self.softcap else logits
