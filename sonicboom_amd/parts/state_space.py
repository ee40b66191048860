"""Recurrent mixers whose memory of a sequence is a float32 matrix per head, fed through short
causal convolutions over time.

``ssd`` (a selective state space in its state-space-duality form; heads of ``v_dim`` channels, a
state of ``n_state`` x ``v_dim`` a head, B and C shared by the heads of a group):

    W_in h = [z | xs | B | C | dt];  (xs, B, C) <- silu(tconv(xs, B, C) + b_conv);
    dt <- softplus(dt + dt_bias);    S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t xs_t^T;
    y_t = S_t^T C_t + D xs_t;        x += out_scale * W_o gnorm(y * silu(z))

with gnorm the RMS norm over ``norm_groups`` equal parts of the row (the gate comes before it).

``channel_delta`` (the delta rule with a decay per head and key channel; ``kv_heads`` heads of
queries and keys of ``head_dim`` numbers shared by groups of the ``heads`` value heads of ``v_dim``):

    q, k, v <- silu(tconv(W_q h)), silu(tconv(W_k h)), silu(tconv(W_v h)); q, k unit vectors a head,
    q also times head_dim^(-1/2);  beta = sigmoid(W_b h);
    g = exp(-exp(A_log) softplus(W_a2 W_a1 h + dt_bias))  (a number per head and key channel);
    S <- g * S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;
    x += out_scale * W_o (o / rms(o) * w * sigmoid(W_g2 W_g1 h))

Everything that enters the recurrences after the projections and convolutions is float32 in both
precisions: the projections leave in float32, the convolutions and their SiLU run on those rows,
and the scan kernels take softplus, exponentials, sigmoids, unit vectors and the output norm from
there.  The matrices and the convolutions' last inputs are per-sequence state of the cache (a row per
slot, zeroed when the slot is handed out, moved on by every step), so prompts cut into steps,
batches and decoding all run the same recurrence, to the bit in the 32-bit path.

With bfloat16 activations a step that brings a sequence more than two chunks of rows takes the
scans' chunked form (every chunk from an empty matrix, the results carried along the sequence, every
chunk again from the matrix that comes in; float32 throughout), which spreads a long prompt over
the whole chip; it differs from the walk by rounding.  The 32-bit path always walks.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Mixer, StateSpec, register_part
from .linear import Linear
from .spec import PartSpec, TensorSpec

UNIT_EPS = 1e-6          # inside the root of the delta rule's unit vectors

SSD_NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "a_log": "A_log", "d_skip": "D",
             "norm": "norm", "out": "o"}
DELTA_NAMES = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "beta": "b",
               "a_log": "A_log", "norm": "norm", "decay_down": "a1", "decay_up": "a2", "dt_bias": "dt_bias",
               "gate_down": "g1", "gate_up": "g2", "out": "o"}


def _vec(t: torch.Tensor) -> torch.Tensor:
    return t.float().contiguous()


def _chunk_rows(rt, tensor: torch.Tensor) -> int:
    """The chunk of the scans' chunked form, 0 where the mixer always walks."""
    return ops.state_scan_chunk_rows() if rt.act_dtype != torch.float32 and tensor.is_cuda else 0


def _chunks(chunk: int, ctx):
    return ctx.row_tiles(chunk) if chunk and ctx.max_new > 2 * chunk else None


def _check_taps(taps: int) -> None:
    if not 2 <= taps <= ops.time_conv_max_taps():
        raise ValueError(f"{taps} taps are not between 2 and the convolution kernel's {ops.time_conv_max_taps()}")


def ssd_spec(prefix: str, width: int, heads: int, v_dim: int, n_state: int, groups: int, taps: int, norm_groups: int,
             eps: float, out_scale: float = 1.0, names: dict = None) -> PartSpec:
    nm = dict(SSD_NAMES, **(names or {}))
    inner, bc = heads * v_dim, 2 * groups * n_state
    return PartSpec("mixer", "ssd", {
        "width": width, "heads": heads, "v_dim": v_dim, "n_state": n_state, "groups": groups, "taps": taps,
        "norm_groups": norm_groups, "eps": float(eps), "out_scale": float(out_scale)}, {
        "in": TensorSpec(prefix + nm["in"], (2 * inner + bc + heads, width)),
        "conv": TensorSpec(prefix + nm["conv"], (inner + bc, taps), init=(0.0, 0.3)),
        "conv_bias": TensorSpec(prefix + nm["conv_bias"], (inner + bc,), init=(0.0, 0.1)),
        "dt_bias": TensorSpec(prefix + nm["dt_bias"], (heads,), init=(0.0, 0.5)),
        "a_log": TensorSpec(prefix + nm["a_log"], (heads,), init=(0.0, 0.5)),
        "d_skip": TensorSpec(prefix + nm["d_skip"], (heads,), init=(1.0, 0.1)),
        "norm": TensorSpec(prefix + nm["norm"], (inner,), init=(1.0, 0.02)),
        "out": TensorSpec(prefix + nm["out"], (width, inner)),
    })


@register_part("mixer", "ssd")
class SSD(Mixer):
    fuses_norm = True
    graph_safe = True     # its launches depend on device buffers only

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.heads, self.v_dim, self.n_state, self.groups = int(p["heads"]), int(p["v_dim"]), int(p["n_state"]), int(p["groups"])
        self.taps, self.norm_groups, self.eps = int(p["taps"]), int(p["norm_groups"]), float(p["eps"])
        self.out_scale = float(p.get("out_scale", 1.0))
        self.inner = self.heads * self.v_dim
        self.bc = self.groups * self.n_state
        if self.heads % self.groups:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.groups} groups")
        if self.inner % self.norm_groups:
            raise ValueError(f"{self.norm_groups} norm groups do not divide {self.inner} channels")
        _check_taps(self.taps)
        rows, cols = ops.state_scan_limits()
        if self.n_state > rows or self.v_dim > cols:
            raise ValueError(f"a state of {self.n_state} x {self.v_dim} a head is more than the scan kernel's {rows} x {cols}")
        self.inp = Linear(tensors["in"], None, rt.fast_kernels)
        self.conv, self.conv_bias = tensors["conv"].contiguous(), tensors["conv_bias"].contiguous()
        self.dt_bias, self.a_log, self.d_skip = _vec(tensors["dt_bias"]), _vec(tensors["a_log"]), _vec(tensors["d_skip"])
        self.norm = tensors["norm"].contiguous()
        self.out = Linear(tensors["out"], None, rt.fast_kernels)
        self.chunk = _chunk_rows(rt, self.norm)
        self.row_tile = self.chunk or None

    def state_spec(self):
        return {"conv": StateSpec((self.taps - 1, self.inner + 2 * self.bc), torch.float32),
                "matrix": StateSpec((self.heads, self.n_state, self.v_dim), torch.float32)}

    def forward(self, h, x, ctx, binding, then_norm=None):
        inner, bc = self.inner, self.bc
        proj = self.inp(h, torch.float32)                              # [rows, z | xs | B | C | dt]
        xbc = ops.time_conv(proj, self.conv, self.conv_bias, binding.states["conv"], ctx, torch.float32, activation="silu",
                            columns=(inner, inner + 2 * bc))
        y = ops.ssd_scan(proj[:, :inner], xbc[:, :inner], xbc[:, inner:inner + bc], xbc[:, inner + bc:],
                         proj[:, 2 * inner + 2 * bc:], self.dt_bias, self.a_log, self.d_skip, binding.states["matrix"], ctx,
                         self.heads, self.groups, self.n_state, self.v_dim, _chunks(self.chunk, ctx))
        y = ops.rmsnorm(y, self.norm, self.eps, self.rt.act_dtype, groups=self.norm_groups)
        return self.out.add_into(y, x, then_norm, self.rt.act_dtype, scale=self.out_scale)


def channel_delta_spec(prefix: str, width: int, heads: int, kv_heads: int, head_dim: int, v_dim: int, taps: int, eps: float,
                       decay_rank: int = -1, gate_rank: int = -1, out_scale: float = 1.0, names: dict = None) -> PartSpec:
    """``decay_rank``, ``gate_rank``: the inner sizes of the two-step projections of the decays and of the
    output gate; -1 takes what the file's tensors have."""
    nm = dict(DELTA_NAMES, **(names or {}))
    qk, vw = kv_heads * head_dim, heads * v_dim
    return PartSpec("mixer", "channel_delta", {
        "width": width, "heads": heads, "kv_heads": kv_heads, "head_dim": head_dim, "v_dim": v_dim, "taps": taps,
        "eps": float(eps), "out_scale": float(out_scale)}, {
        "q": TensorSpec(prefix + nm["q"], (qk, width)), "k": TensorSpec(prefix + nm["k"], (qk, width)),
        "v": TensorSpec(prefix + nm["v"], (vw, width)),
        "q_conv": TensorSpec(prefix + nm["q_conv"], (qk, taps), init=(0.0, 0.3)),
        "k_conv": TensorSpec(prefix + nm["k_conv"], (qk, taps), init=(0.0, 0.3)),
        "v_conv": TensorSpec(prefix + nm["v_conv"], (vw, taps), init=(0.0, 0.3)),
        "beta": TensorSpec(prefix + nm["beta"], (heads, width)),
        "a_log": TensorSpec(prefix + nm["a_log"], (heads,), init=(-1.0, 0.5)),
        "norm": TensorSpec(prefix + nm["norm"], (v_dim,), init=(1.0, 0.02)),
        "decay_down": TensorSpec(prefix + nm["decay_down"], (decay_rank, width)),
        "decay_up": TensorSpec(prefix + nm["decay_up"], (heads * head_dim, decay_rank)),
        "dt_bias": TensorSpec(prefix + nm["dt_bias"], (heads * head_dim,), init=(0.0, 0.5)),
        "gate_down": TensorSpec(prefix + nm["gate_down"], (gate_rank, width)),
        "gate_up": TensorSpec(prefix + nm["gate_up"], (vw, gate_rank)),
        "out": TensorSpec(prefix + nm["out"], (width, vw)),
    })


@register_part("mixer", "channel_delta")
class ChannelDelta(Mixer):
    fuses_norm = True
    graph_safe = True     # its launches depend on device buffers only

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.heads, self.kv_heads, self.head_dim, self.v_dim = int(p["heads"]), int(p["kv_heads"]), int(p["head_dim"]), int(p["v_dim"])
        self.taps, self.eps = int(p["taps"]), float(p["eps"])
        self.out_scale = float(p.get("out_scale", 1.0))
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.kv_heads} query/key heads")
        _check_taps(self.taps)
        rows, cols = ops.state_scan_limits()
        if self.head_dim > rows or self.v_dim > cols:
            raise ValueError(f"a state of {self.head_dim} x {self.v_dim} a head is more than the scan kernel's {rows} x {cols}")
        self.qkv_width = 2 * self.kv_heads * self.head_dim + self.heads * self.v_dim
        ws = [tensors["q"], tensors["k"], tensors["v"], tensors["beta"]]
        if not all(w.dtype == ws[0].dtype for w in ws):
            ws = [w.float() for w in ws]
        self.qkvb = Linear(torch.cat(ws, dim=0), None, rt.fast_kernels)          # one product for q | k | v | beta
        convs = [tensors["q_conv"], tensors["k_conv"], tensors["v_conv"]]
        if not all(c.dtype == convs[0].dtype for c in convs):
            convs = [c.float() for c in convs]
        self.conv = torch.cat(convs, dim=0).contiguous()
        self.decay_down = Linear(tensors["decay_down"], None, rt.fast_kernels)
        self.decay_up = Linear(tensors["decay_up"], None, rt.fast_kernels)
        self.gate_down = Linear(tensors["gate_down"], None, rt.fast_kernels)
        self.gate_up = Linear(tensors["gate_up"], None, rt.fast_kernels)
        self.dt_bias, self.a_log = _vec(tensors["dt_bias"]), _vec(tensors["a_log"])
        self.norm = tensors["norm"].contiguous()
        self.out = Linear(tensors["out"], None, rt.fast_kernels)
        self.chunk = _chunk_rows(rt, self.norm)
        self.row_tile = self.chunk or None

    def state_spec(self):
        return {"conv": StateSpec((self.taps - 1, self.qkv_width), torch.float32),
                "matrix": StateSpec((self.heads, self.head_dim, self.v_dim), torch.float32)}

    def forward(self, h, x, ctx, binding, then_norm=None):
        act = self.rt.act_dtype
        proj = self.qkvb(h, torch.float32)                             # [rows, q | k | v | beta]
        qkv = ops.time_conv(proj, self.conv, None, binding.states["conv"], ctx, torch.float32, activation="silu",
                            columns=(0, self.qkv_width))
        decay = self.decay_up(self.decay_down(h, act), torch.float32)
        gate = self.gate_up(self.gate_down(h, act), torch.float32)
        y = ops.delta_scan(qkv, proj[:, self.qkv_width:], decay, gate, self.dt_bias, self.a_log, self.norm,
                           binding.states["matrix"], ctx, self.heads, self.kv_heads, self.head_dim, self.v_dim, self.eps,
                           UNIT_EPS, act, _chunks(self.chunk, ctx))
        return self.out.add_into(y, x, then_norm, act, scale=self.out_scale)
