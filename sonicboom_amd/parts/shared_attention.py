"""Grouped-query attention whose heads share their softmax weights.

    q = W_q h + b_q,  k = W_k h + b_k;  with ``values_from_keys`` the values are k as projected
    (there is no W_v and v_dim = head_dim);
    q and k are RMS-normed over the whole projection (all heads at once) with weights of that size;
    q is multiplied by 1 + temp_coef ln(floor((p + 1) / temp_every) + 1) at position p;
    score(p, j) = scale q_p . k_j - r1_a ln(1 + r2_a (p - j)) for j <= p, a number pair (r1, r2) a head;
    P_a = softmax over j;  P'_a = sum_b T[a, b] P_b with T [heads, heads];
    head a applies P'_a to the values of its own key/value head;  x += out_scale * W_o (heads).

Since the mixing is linear, head a's result is sum_b T[a, b] (P_b V_c) with c its key/value head: the
attention kernel computes O[b, c] = P_b V_c for every query head b against the values of every
key/value head c (the scores and the softmax once a head), and a small pass mixes them with T.  No
mixed weight matrix is ever built.  Keys (normed) and values go into the framework's paged cache, in
its layout; positions enter through the temperature and the distance only.

Switches of the spec: ``qk_bias``, ``temp_coef`` (0: none), ``distance_bias``, ``head_mix``, ``values_from_keys``
(the only form built so far: a model with a W_v of its own is refused when the part is built).
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from .. import ops
from .base import KVSpec, Mixer, register_part
from .linear import Linear
from .spec import PartSpec, TensorSpec

NAMES = {"q": "q", "k": "k", "q_bias": "q.b", "k_bias": "k.b", "q_norm": "q.norm", "k_norm": "k.norm", "r1": "r1", "r2": "r2",
         "mix": "talk", "out": "o"}


def shared_attention_spec(prefix: str, width: int, heads_q: int, heads_kv: int, head_dim: int, eps: float,
                          scale: Optional[float] = None, qk_bias: bool = True, temp_coef: float = 0.0, temp_every: int = 1,
                          distance_bias: bool = True, head_mix: bool = True, values_from_keys: bool = True,
                          out_scale: float = 1.0, names: Optional[dict] = None) -> PartSpec:
    nm = dict(NAMES, **(names or {}))
    qw, kw = heads_q * head_dim, heads_kv * head_dim
    tensors = {"q": TensorSpec(prefix + nm["q"], (qw, width)), "k": TensorSpec(prefix + nm["k"], (kw, width)),
               "q_norm": TensorSpec(prefix + nm["q_norm"], (qw,), init=(1.0, 0.02)),
               "k_norm": TensorSpec(prefix + nm["k_norm"], (kw,), init=(1.0, 0.02)),
               "out": TensorSpec(prefix + nm["out"], (width, qw))}
    if qk_bias:
        tensors["q_bias"] = TensorSpec(prefix + nm["q_bias"], (qw,))
        tensors["k_bias"] = TensorSpec(prefix + nm["k_bias"], (kw,))
    if distance_bias:
        tensors["r1"] = TensorSpec(prefix + nm["r1"], (heads_q,), init=(0.5, 0.1))
        tensors["r2"] = TensorSpec(prefix + nm["r2"], (heads_q,), init=(0.5, 0.1))
    if head_mix:
        tensors["mix"] = TensorSpec(prefix + nm["mix"], (heads_q, heads_q), init=(0.15, 0.2))
    return PartSpec("mixer", "shared_attention", {
        "width": width, "heads_q": heads_q, "heads_kv": heads_kv, "head_dim": head_dim, "eps": float(eps), "scale": scale,
        "qk_bias": bool(qk_bias), "temp_coef": float(temp_coef), "temp_every": int(temp_every),
        "distance_bias": bool(distance_bias), "head_mix": bool(head_mix), "values_from_keys": bool(values_from_keys),
        "out_scale": float(out_scale)}, tensors)


@register_part("mixer", "shared_attention")
class SharedAttention(Mixer):
    # a step's context lists its rows in runs of this many for the matrix-core kernel
    row_tile = ops.CAPPED_ROW_TILE
    fuses_norm = True
    graph_safe = True     # its launches depend on device buffers only

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.heads_q, self.heads_kv, self.head_dim = int(p["heads_q"]), int(p["heads_kv"]), int(p["head_dim"])
        if self.heads_q % self.heads_kv:
            raise ValueError(f"{self.heads_q} query heads are not a multiple of {self.heads_kv} key/value heads")
        if not p.get("values_from_keys", True):
            raise ValueError("attention with shared weights is built for values taken from the keys")
        self.v_dim = self.head_dim
        self.eps = float(p["eps"])
        scale = p.get("scale")
        self.scale = float(np.float32(1.0) / np.sqrt(np.float32(self.head_dim))) if scale is None else float(scale)
        self.temp_coef, self.temp_every = float(p.get("temp_coef", 0.0)), int(p.get("temp_every", 1))
        if self.temp_coef and self.temp_every <= 0:
            raise ValueError("the query temperature's period must be positive")
        self.out_scale = float(p.get("out_scale", 1.0))
        ws = [tensors["q"], tensors["k"]]
        if ws[0].dtype != ws[1].dtype:
            ws = [w.float() for w in ws]
        bias = None
        if p.get("qk_bias", True):
            bias = torch.cat([tensors["q_bias"].float(), tensors["k_bias"].float()], dim=0)
        self.qk = Linear(torch.cat(ws, dim=0), bias, rt.fast_kernels)         # one product for q | k
        self.q_norm, self.k_norm = tensors["q_norm"].contiguous(), tensors["k_norm"].contiguous()
        if self.q_norm.dtype != self.k_norm.dtype:
            self.q_norm, self.k_norm = self.q_norm.float(), self.k_norm.float()
        self.r1 = tensors["r1"].float().contiguous() if p.get("distance_bias", True) else None
        self.r2 = tensors["r2"].float().contiguous() if p.get("distance_bias", True) else None
        self.mix = tensors["mix"].float().contiguous() if p.get("head_mix", True) else None
        self.out = Linear(tensors["out"], None, rt.fast_kernels)

    def cache_spec(self) -> KVSpec:
        return KVSpec(self.heads_kv, self.head_dim, 0, self.v_dim)

    def forward(self, h, x, ctx, binding, then_norm=None):
        rt = self.rt
        if not binding.writes_cache:
            raise ValueError("attention with shared weights stores its own keys")
        qk = self.qk(h, torch.float32)                                 # [rows, q | k], biases added
        page_table = ctx.page_table(binding.group)
        q = ops.qk_rownorm_store(qk, rt.act_dtype, self.q_norm, self.k_norm, self.eps, self.temp_coef, self.temp_every,
                                 ctx.row_pos, ctx.row_seq, binding.k_cache, binding.v_cache, page_table, self.heads_q,
                                 self.heads_kv, self.head_dim)
        a = ops.attention_shared(q, binding.k_cache, binding.v_cache, page_table, ctx, self.heads_q, self.heads_kv,
                                 self.head_dim, self.v_dim, self.scale, self.r1, self.r2, self.mix, rt.act_dtype,
                                 fast=rt.fast_kernels)
        return self.out.add_into(a, x, then_norm, rt.act_dtype, scale=self.out_scale)
