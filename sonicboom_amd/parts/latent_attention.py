"""Latent attention: keys and values of all heads come from one small latent per token.

    q = W_q h, head a = [dim plain numbers | rot_dim rotated numbers]
    W_dkv h = [kv_rank numbers | rot_dim numbers]:  c = rmsnorm(first part) * w_c (the latent),
                                                     r = rotate(second part) (one key part for all heads)
    head a:  key [W_uk,a c | r],  value W_uv,a c,  score = scale * (q_a . key_a),
    softmax over the positions s with 0 <= t - s < window (window 0: all up to t),
    x += out_scale * W_o ((heads' results side by side) * sigmoid(W_g h))

The cache holds the row [c | r] per token (a cache of rows, one "head" for all query heads), and
the kernels work in that space: W_uk,a carries head a's plain query part into the latent space,
attention runs over the cached rows, and W_uv,a (with the output gate) brings the result back
(csrc/attention_latent.hip).  The input projections (queries, output gate, and the latent's
projection when the layer has one) are one stacked matrix.  A layer may read the rows another
layer stores (an order entry that does not write its cache): it then has no W_dkv, and its own
queries, W_uk, W_uv, window and scale.  The rotation is a nested position part of a rotary kind;
its pairing (neighbours or halves) and its magnitude go to the kernel as arguments.

With ``q_rank`` > 0 the queries pass a latent of their own: cq = rmsnorm(W_dq h) * w_q (eps of the
layer), q = W_uq cq; W_dq then takes W_q's place in the stacked product and W_uq is a second product.
With ``gate_per_head`` the output gate is one number a head, sigmoid((W_g h)_a), and W_g has a row a head.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops
from .base import Mixer, RowsSpec, register_part
from .linear import Linear
from .spec import PartSpec, TensorSpec


def latent_attention_spec(prefix: str, width: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                          scale: float, position: PartSpec, window: int = 0, eps: float = 1e-6,
                          own_latent: bool = True, out_scale: float = 1.0, q_rank: int = 0,
                          gate_per_head: bool = False) -> PartSpec:
    """Tensors ``<prefix>q`` (or, with ``q_rank``, ``dq``, ``dq.norm`` and ``uq``), ``g``, ``o``, ``uk``, ``uv`` and,
    with ``own_latent``, ``dkv`` and ``dkv.norm``."""
    if q_rank:
        tensors = {"dq_weight": TensorSpec(prefix + "dq", (q_rank, width)),
                   "dq_norm": TensorSpec(prefix + "dq.norm", (q_rank,), init=(1.0, 0.02)),
                   "uq_weight": TensorSpec(prefix + "uq", (heads * (dim + rot_dim), q_rank))}
    else:
        tensors = {"q_weight": TensorSpec(prefix + "q", (heads * (dim + rot_dim), width))}
    tensors.update({
        "uk_weight": TensorSpec(prefix + "uk", (heads * dim, kv_rank)),
        "uv_weight": TensorSpec(prefix + "uv", (heads * vdim, kv_rank)),
        "g_weight": TensorSpec(prefix + "g", (heads if gate_per_head else heads * vdim, width)),
        "o_weight": TensorSpec(prefix + "o", (width, heads * vdim)),
    })
    if own_latent:
        tensors["dkv_weight"] = TensorSpec(prefix + "dkv", (kv_rank + rot_dim, width))
        tensors["dkv_norm"] = TensorSpec(prefix + "dkv.norm", (kv_rank,), init=(1.0, 0.02))
    return PartSpec("mixer", "latent_attention", {
        "width": width, "heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
        "scale": float(scale), "window": int(window), "eps": float(eps), "own_latent": bool(own_latent),
        "out_scale": float(out_scale), "q_rank": int(q_rank), "gate_per_head": bool(gate_per_head)},
        tensors, {"position": position})


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    fuses_norm = True
    graph_safe = True     # its launches depend on device buffers only

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.width, self.heads = int(p["width"]), int(p["heads"])
        self.dim, self.rot_dim, self.vdim, self.rank = int(p["dim"]), int(p["rot_dim"]), int(p["vdim"]), int(p["kv_rank"])
        self.latent = self.rank + self.rot_dim
        self.window = int(p.get("window") or 0)
        self.eps = float(p["eps"])
        self.own_latent = bool(p.get("own_latent", True))
        self.out_scale = float(p.get("out_scale", 1.0))
        self.position = parts["position"]
        tables = self.position.rotary_tables()
        if tables is None:
            raise ValueError("latent attention takes a rotary position encoding (or 'none')")
        self.inv_freq, factors, self.rot_dims = tables
        if factors is not None:
            raise ValueError("latent attention does not take per-pair divisors of the rotation")
        if self.inv_freq is None:
            self.rot_dims = 0
        if self.rot_dims > self.rot_dim:
            raise ValueError(f"{self.rot_dims} numbers rotate, a head has {self.rot_dim} for it")
        self.scale = float(p["scale"]) * float(self.position.score_scale)
        self.magnitude = float(getattr(self.position, "magnitude", 1.0))
        H = self.heads
        self.q_rank = int(p.get("q_rank", 0) or 0)
        self.gate_per_head = bool(p.get("gate_per_head", False))
        self.gate_cols = H if self.gate_per_head else H * self.vdim
        first = tensors["dq_weight"] if self.q_rank else tensors["q_weight"]
        ws = [first, tensors["g_weight"]] + ([tensors["dkv_weight"]] if self.own_latent else [])
        if not all(w.dtype == ws[0].dtype for w in ws):
            ws = [w.float() for w in ws]
        # the stacked product's columns: queries (or their latent), gate, and the latent's part when the layer has one
        self.q_off, self.g_off = 0, first.shape[0]
        self.kv_off = self.g_off + self.gate_cols if self.own_latent else -1
        self.proj = Linear(torch.cat(ws, dim=0), None, rt.fast_kernels)
        self.q_norm_weight = tensors.get("dq_norm") if self.q_rank else None
        self.uq = Linear(tensors["uq_weight"], None, rt.fast_kernels) if self.q_rank else None
        self.c_weight = tensors.get("dkv_norm")
        # per head a small matrix [out, in]: keys are W_uk c, so W_uk,a^T [rank, dim] carries head a's plain
        # query part into the latent space; W_uv,a [vdim, rank] as the file has it brings a result back
        wdt = rt.act_dtype
        self.uk = tensors["uk_weight"].to(wdt).reshape(H, self.dim, self.rank).transpose(1, 2).contiguous()
        self.uv = tensors["uv_weight"].to(wdt).reshape(H, self.vdim, self.rank).contiguous()
        # the matrix-core attention kernel takes a prompt step's rows in runs of this many
        if rt.fast_kernels and ops.latent_attention_mfma_ok(rt.act_dtype, rt.cache_dtype, self.rank, self.rot_dim):
            self.row_tile = ops.LATENT_ROW_TILE
        self.out = Linear(tensors["o_weight"], None, rt.fast_kernels)

    def cache_spec(self) -> RowsSpec:
        return RowsSpec((self.latent,), self.window)

    def forward(self, h, x, ctx, binding, then_norm=None):
        """x += out_scale * attention(h).  Returns then_norm(x) when the output projection could apply
        the norm in its last pass, else None."""
        rt = self.rt
        writes = binding.writes_cache
        if writes != self.own_latent:
            raise RuntimeError("a latent-attention layer stores rows exactly when it has a latent projection of its own")
        pre = self.proj(h, torch.float32)                 # [rows, q | g | (c, r)]
        table = ctx.page_table(binding.group)
        cache = binding.k_cache
        queries, kv_rows = pre, None
        if self.q_rank:
            # the queries' own latent is normed where it lies in the stacked product's rows, then carried up
            cq, _ = ops.rmsnorm_pair(pre[:, :self.q_rank], self.q_norm_weight, None, self.eps, rt.act_dtype, second=False)
            queries, kv_rows = self.uq(cq, torch.float32), pre
        q_plain, q_lat = ops.latent_prepare(
            queries, self.q_off, self.kv_off, rt.act_dtype, self.c_weight, self.eps, self.inv_freq, self.rot_dims,
            bool(self.position.interleaved), ctx.row_pos, ctx.row_seq, cache if writes else None,
            table if writes else None, self.heads, self.dim, self.rot_dim, self.rank, kv_rows=kv_rows,
            magnitude=self.magnitude)
        ops.head_product(q_plain, self.uk, q_lat, fast=rt.fast_kernels)     # the first rank numbers of every head's query
        a_lat = ops.latent_attention(q_lat, cache, table, ctx, self.rank, self.scale, self.window, fast=rt.fast_kernels)
        a = torch.empty((a_lat.shape[0], self.heads, self.vdim), dtype=rt.act_dtype, device=a_lat.device)
        gate = pre[:, self.g_off:self.g_off + self.gate_cols]
        ops.head_product(a_lat, self.uv, a, gate=gate, fast=rt.fast_kernels, gate_per_head=self.gate_per_head)
        return self.out.add_into(a.view(a.shape[0], -1), x, then_norm, rt.act_dtype, scale=self.out_scale)
