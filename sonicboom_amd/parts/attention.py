"""Grouped-query self-attention over the paged cache.

Order of work, from /root/reference/core/src/model/emit.cpp:255-308: project
q, k and v, add their biases, rotate q and k (the bias precedes the rotation,
v is not rotated), store k and v, attend, project the result.  The scale is
1/sqrt(head_dim) unless the spec gives another, times the position encoding's
multiplier (/root/reference/core/src/model/recipe.cpp:65-70, :165-167).
Every size and switch is a parameter of the spec:

    heads_q, heads_kv, head_dim, window (0 = all keys), scale (None = 1/sqrt),
    qkv_bias, out_bias, out_scale (the multiplier of the branch, 1 unless given),
    v_dim (the values' size per head when it is not the keys'), qk_norm (every head of q and k
    divided by its root mean square, eps ``qk_norm_eps`` inside the root, times a weight of the head's
    size that the heads share), softcap (scores become softcap * tanh(score / softcap); 0: not),
    sink (one more key of score 0 without a value in every softmax: the weights are
    exp(s_j) / (1 + sum exp(s_j))), value_mix ("first": the values of this step's rows are kept
    for later layers under ``value_mix_key``; "mix": v <- (1 - lam) v + lam v_first with the layer's
    own number lam; what is mixed is what the cache keeps), sink_scores (the sink's score is a number of
    the query head's own, a tensor of heads_q numbers, as it is: weights exp(s_j) / (exp(sink_a) + sum
    exp(s_j))), out_gate (the heads' results side by side times sigmoid(W_g h), number by number, before
    the output product; W_g is stacked under q, k and v)

and the position encoding is a nested part.  The three input projections are
packed into one matrix when the mixer is built, so a step runs one product
for q, k and v.  An order entry that only reads another entry's cache runs
the query rows of that matrix alone.
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from .. import ops
from .base import KVSpec, Mixer, register_part
from .linear import Linear
from .spec import PartSpec, TensorSpec


NAMES = {"q_weight": "q_proj.weight", "k_weight": "k_proj.weight", "v_weight": "v_proj.weight",
         "o_weight": "o_proj.weight", "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias",
         "o_bias": "o_proj.bias", "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", "value_mix": "value_mix",
         "sink": "sink", "g_weight": "g"}


def attention_spec(prefix: str, width: int, heads_q: int, heads_kv: int, head_dim: int,
                   position: PartSpec, window: int = 0, scale: Optional[float] = None,
                   qkv_bias: bool = True, out_bias: bool = False, out_scale: float = 1.0,
                   v_dim: Optional[int] = None, qk_norm: bool = False, qk_norm_eps: float = 0.0,
                   softcap: float = 0.0, sink: bool = False, value_mix: Optional[str] = None,
                   value_mix_key: str = "values", names: Optional[dict] = None, sink_scores: bool = False,
                   out_gate: bool = False) -> PartSpec:
    """``names``: what the file calls a role's tensor after ``prefix``, where that is not what
    ``NAMES`` says."""
    nm = dict(NAMES, **(names or {}))
    v_dim = head_dim if v_dim is None else int(v_dim)
    qw, kw, vw = heads_q * head_dim, heads_kv * head_dim, heads_kv * v_dim
    tensors = {
        "q_weight": TensorSpec(prefix + nm["q_weight"], (qw, width)),
        "k_weight": TensorSpec(prefix + nm["k_weight"], (kw, width)),
        "v_weight": TensorSpec(prefix + nm["v_weight"], (vw, width)),
        "o_weight": TensorSpec(prefix + nm["o_weight"], (width, heads_q * v_dim)),
    }
    if qkv_bias:
        tensors["q_bias"] = TensorSpec(prefix + nm["q_bias"], (qw,))
        tensors["k_bias"] = TensorSpec(prefix + nm["k_bias"], (kw,))
        tensors["v_bias"] = TensorSpec(prefix + nm["v_bias"], (vw,))
    if out_bias:
        tensors["o_bias"] = TensorSpec(prefix + nm["o_bias"], (width,))
    if qk_norm:
        tensors["q_norm"] = TensorSpec(prefix + nm["q_norm"], (head_dim,), init=(1.0, 0.02))
        tensors["k_norm"] = TensorSpec(prefix + nm["k_norm"], (head_dim,), init=(1.0, 0.02))
    if sink_scores:
        if not sink:
            raise ValueError("scores of a sink belong to a mixer that has one")
        tensors["sink"] = TensorSpec(prefix + nm["sink"], (heads_q,), init=(0.0, 0.5))
    if out_gate:
        tensors["g_weight"] = TensorSpec(prefix + nm["g_weight"], (heads_q * v_dim, width))
    if value_mix not in (None, "first", "mix"):
        raise ValueError(f"value_mix is None, 'first' or 'mix', not {value_mix!r}")
    if value_mix is not None:
        # the first mixing layer's number is in the file too, and is not used
        tensors["value_mix"] = TensorSpec(prefix + nm["value_mix"], (), init=(0.5, 0.1))
    return PartSpec("mixer", "attention", {
        "width": width, "heads_q": heads_q, "heads_kv": heads_kv, "head_dim": head_dim,
        "window": int(window), "scale": scale, "qkv_bias": qkv_bias, "out_bias": out_bias,
        "out_scale": float(out_scale), "v_dim": v_dim, "qk_norm": bool(qk_norm), "qk_norm_eps": float(qk_norm_eps),
        "softcap": float(softcap), "sink": bool(sink), "value_mix": value_mix, "value_mix_key": value_mix_key,
        "sink_scores": bool(sink_scores), "out_gate": bool(out_gate),
    }, tensors, {"position": position})


@register_part("mixer", "attention")
class Attention(Mixer):
    # a step's context lists its rows in runs of this many for the mixer's prefill kernel
    row_tile = ops.ATTENTION_ROW_TILE

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.width = int(p["width"])
        self.heads_q, self.heads_kv, self.head_dim = int(p["heads_q"]), int(p["heads_kv"]), int(p["head_dim"])
        if self.heads_q % self.heads_kv:
            raise ValueError(f"{self.heads_q} query heads are not a multiple of {self.heads_kv} kv heads")
        self.window = int(p.get("window") or 0)
        self.position = parts["position"]
        base_scale = p.get("scale")
        if base_scale is None:
            base_scale = float(np.float32(1.0) / np.sqrt(np.float32(self.head_dim)))
        self.scale = float(np.float32(base_scale) * np.float32(self.position.score_scale))
        self.q_width = self.heads_q * self.head_dim
        self.kv_width = self.heads_kv * self.head_dim
        self.v_dim = int(p.get("v_dim") or self.head_dim)
        self.qk_norm = bool(p.get("qk_norm", False))
        self.qk_norm_eps = float(p.get("qk_norm_eps", 0.0))
        self.q_norm, self.k_norm = tensors.get("q_norm"), tensors.get("k_norm")
        self.softcap = float(p.get("softcap", 0.0) or 0.0)
        self.sink = bool(p.get("sink", False))
        self.value_mix = p.get("value_mix")
        self.value_mix_key = p.get("value_mix_key", "values")
        self.lam = tensors.get("value_mix") if self.value_mix == "mix" else None
        self.sink_scores = tensors["sink"].float().contiguous() if p.get("sink_scores") else None
        self.out_gate = bool(p.get("out_gate", False))
        # head norms, capped scores, a sink, values of their own size or mixed values, an output gate: the path
        # whose kernels take them.  Head norms and mixed values go with mixers that do not rotate (one kernel
        # norms, mixes and stores); the others rotate and store with the kernel of the plain path.
        self.extended = bool(self.qk_norm or self.softcap or self.sink or self.value_mix or self.v_dim != self.head_dim
                             or self.out_gate)
        self.head_norm_path = bool(self.qk_norm or self.value_mix)
        if self.extended:
            if self.head_norm_path and self.position.rotary_tables() != (None, None, 0):
                raise ValueError("head norms and mixed values are built for mixers without a rotation")
            if self.position.rotary_tables() is None:
                raise ValueError("capped scores, sinks, gates and values of their own size take a rotary position "
                                 "encoding, or none")
            if self.head_norm_path and p.get("qkv_bias", True):
                raise ValueError("head norms and mixed values are built for mixers without biases on q, k and v")
        if rt.fast_kernels and not self.extended:
            # (groups of one and two heads per kv head take higher tiles on the matrix cores)
            self.row_tile = ops.attention_row_tiles(self.heads_q, self.heads_kv, self.head_dim, rt.act_dtype)

        ws = [tensors["q_weight"], tensors["k_weight"], tensors["v_weight"]]
        self.g_off = sum(int(w.shape[0]) for w in ws)        # where the output gate's columns start in the stacked product
        if self.out_gate:
            ws.append(tensors["g_weight"])
        w_qkv = torch.cat(ws, dim=0) if all(w.dtype == ws[0].dtype for w in ws) \
            else torch.cat([w.float() for w in ws], dim=0)
        b_qkv = None
        if p.get("qkv_bias", True):
            bs = [tensors["q_bias"], tensors["k_bias"], tensors["v_bias"]]
            b_qkv = torch.cat([b.float() for b in bs], dim=0)
            if self.out_gate:
                b_qkv = torch.cat([b_qkv, torch.zeros(tensors["g_weight"].shape[0], dtype=torch.float32, device=b_qkv.device)])
        self.qkv = Linear(w_qkv, b_qkv, rt.fast_kernels)
        # an order entry that reads another entry's cache projects queries only: the model asks for
        # that projection (query_only) before finish_build() drops the separate query weight
        self._q_parts = (tensors["q_weight"], None if b_qkv is None else b_qkv[: self.q_width])
        self._q_only = None
        self.out = Linear(tensors["o_weight"], tensors.get("o_bias"), rt.fast_kernels)
        self.out_scale = float(p.get("out_scale", 1.0))      # x += out_scale * attention(h)

    def query_only(self) -> None:
        """Build the queries-only projection (for run-order entries that read another entry's cache)."""
        if self._q_only is None:
            if self._q_parts is None:
                raise RuntimeError("the queries-only projection must be asked for while the model is built")
            self._q_only = Linear(self._q_parts[0], self._q_parts[1], self.rt.fast_kernels)

    def finish_build(self) -> None:
        self._q_parts = None

    def cache_spec(self) -> KVSpec:
        return KVSpec(self.heads_kv, self.head_dim, self.window, self.v_dim)

    fuses_norm = True
    graph_safe = True     # its launches depend on device buffers only
    fold_rotation = True  # decode steps: rotate and store inside the attention kernel where it takes the sizes

    def forward(self, h, x, ctx, binding, then_norm=None):
        """x += attention(h).  Returns then_norm(x) when the output projection could apply the
        norm in its last pass, else None."""
        a = self._attend(h, ctx, binding)
        return self.out.add_into(a, x, then_norm, self.rt.act_dtype, scale=self.out_scale)

    def produce(self, h, ctx, binding):
        """attention(h) in float32 (whole, or in K slices of the output product), for a block that
        adds it up itself."""
        if self.out_scale != 1.0:
            raise ValueError("a mixer that hands its result over has no multiplier of its own")
        return self.out.raw(self._attend(h, ctx, binding))

    def _attend_rotating(self, h, ctx, binding):
        """The extended path of mixers that rotate (or have no position encoding and no head norms): the plain path's
        rotate-and-store kernel with the values' own size, attention with the sink's scores, the output gate."""
        rt = self.rt
        if not binding.writes_cache:
            raise RuntimeError("this mixer stores the keys and values it reads")
        # (with a gate the product is taken whole: the gate's columns are read where they lie)
        qkv = None if self.out_gate else self.qkv.partial(h)
        bias = None
        if qkv is not None:
            bias = self.qkv.bias
        else:
            qkv = self.qkv(h, torch.float32)
        inv_freq, freq_factors, rot_dims = self.position.rotary_tables()
        page_table = ctx.page_table(binding.group)
        q = ops.rope_kv_store(qkv, rt.act_dtype, inv_freq, freq_factors, rot_dims, ctx.row_pos, ctx.row_seq,
                              binding.k_cache, binding.v_cache, page_table, self.heads_q, self.heads_kv, self.head_dim,
                              bias=bias, v_dim=self.v_dim, magnitude=float(getattr(self.position, "magnitude", 1.0)))
        # the gate rides in the attention kernel's last pass (or, when a row's pages are shared out, in the merge)
        gate = qkv[:, self.g_off:self.g_off + self.heads_q * self.v_dim] if self.out_gate else None
        a = ops.attention_capped(q, binding.k_cache, binding.v_cache, page_table, ctx, self.heads_q, self.heads_kv,
                                 self.head_dim, self.v_dim, self.scale, self.window, self.softcap, self.sink,
                                 fast=rt.fast_kernels, sink_scores=self.sink_scores, gate=gate)
        return a

    def _attend_extended(self, h, ctx, binding):
        if not self.head_norm_path:
            return self._attend_rotating(h, ctx, binding)
        rt = self.rt
        writes = binding.writes_cache
        if not writes:
            self.query_only()
        proj = self.qkv if writes else self._q_only
        qkv = proj.partial(h)
        if qkv is None:
            qkv = proj(h, torch.float32)
        v_first = v_out = None
        if writes and self.value_mix is not None:
            shared = ctx.shared
            if self.value_mix == "first":
                v_out = torch.empty((ctx.n_rows, self.heads_kv * self.v_dim), dtype=torch.float32, device=h.device)
                shared[self.value_mix_key] = v_out
            else:
                v_first = shared.get(self.value_mix_key)
                if v_first is None:
                    raise RuntimeError(f"no earlier layer of this step has left its values under {self.value_mix_key!r}")
        page_table = ctx.page_table(binding.group)
        q = ops.headnorm_kv_store(qkv, rt.act_dtype, self.q_norm, self.k_norm, self.qk_norm_eps, ctx.row_pos, ctx.row_seq,
                                  binding.k_cache, binding.v_cache, page_table, self.heads_q, self.heads_kv,
                                  self.head_dim, self.v_dim, store=writes, v_first=v_first, lam=self.lam, v_out=v_out)
        return ops.attention_capped(q, binding.k_cache, binding.v_cache, page_table, ctx, self.heads_q, self.heads_kv,
                                    self.head_dim, self.v_dim, self.scale, self.window, self.softcap, self.sink,
                                    fast=rt.fast_kernels, sink_scores=self.sink_scores)

    def _attend(self, h, ctx, binding):
        """The heads' results [rows, heads_q * v_dim] in the activation type; keys and values of the
        step's rows are in the cache afterwards."""
        if self.extended:
            return self._attend_extended(h, ctx, binding)
        rt = self.rt
        writes = binding.writes_cache
        if not writes:
            self.query_only()
        proj = self.qkv if writes else self._q_only
        # q, k, v stay float32 until they have been rotated: one rounding on the way to the cache.
        tables = self.position.rotary_tables()
        bias = None
        qkv = proj.partial(h) if tables is not None else None
        if qkv is not None:
            bias = proj.bias          # the rotate-and-store kernel adds the K slices and the bias
        else:
            qkv = proj(h, torch.float32)
        if tables is None:
            self.position.apply(qkv, ctx, self.heads_q, self.heads_kv if writes else 0, self.head_dim)
            tables = (None, None, 0)
        inv_freq, freq_factors, rot_dims = tables
        page_table = ctx.page_table(binding.group)
        if ctx.is_decode and rt.fast_kernels and self.fold_rotation and ops.attention_decode_rope_ok(
                qkv, rt.act_dtype, binding.k_cache.dtype, self.heads_q, self.heads_kv, self.head_dim,
                rot_dims if inv_freq is not None else 0):
            # one token per sequence: rotation, store and attention in one kernel
            return ops.attention_decode_rope(qkv, inv_freq, freq_factors, rot_dims, binding.k_cache, binding.v_cache,
                                             page_table, ctx.row_pos, self.heads_q, self.heads_kv, self.head_dim,
                                             self.scale, self.window, bias=bias, store=writes)
        q = ops.rope_kv_store(
            qkv, rt.act_dtype, inv_freq, freq_factors, rot_dims, ctx.row_pos, ctx.row_seq,
            binding.k_cache if writes else None, binding.v_cache if writes else None,
            page_table if writes else None, self.heads_q, self.heads_kv if writes else 0, self.head_dim,
            bias=bias)
        return ops.attention(q, binding.k_cache, binding.v_cache, page_table, ctx, self.heads_q, self.heads_kv,
                             self.head_dim, self.scale, self.window, fast=rt.fast_kernels, row_tile=self.row_tile)
