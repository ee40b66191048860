"""A plain, slow implementation of the Nalasun decoder.

Whole sequences, no cache, one function per mechanism, NumPy in float64 throughout.  It shares no
code with ``sonicboom_amd``: the configuration is the dict of config.json and the weights a dict of
arrays by the file's tensor names.

The design in this file's notation (``n`` tokens, position t = 0 .. n-1, stream x [n, width]):

* start: x = table[token] + pos[t].
* rms(v, w) = v / sqrt(mean(v^2) + eps) * w.
* a layer: h = rms(x, norm1); h <- h + tconv(h, canon1) (a causal convolution over time, channel
  by channel, the last tap on the current token, zeros before the sequence); x += mixer(h);
  and, if the layer has a feed-forward, x += ff(rms(x, norm2)).
* mixer ``mamba2``: W_in h = [z | xs | B | C | dt]; (xs, B, C) pass a causal convolution with bias
  and silu; dt = softplus(dt + dt_bias); per head a, with group a // (heads / groups):
  S_t = exp(-exp(A_log_a) dt_t) S_(t-1) + dt_t B_t xs_t^T, y_t = S_t^T C_t + D_a xs_t; y times silu(z),
  divided part by part (``norm_groups`` equal parts) by its root mean square, times a weight; W_o.
* mixer ``channel_delta``: q, k (kv_heads x dim) and v (heads x vdim) pass a causal convolution
  without bias and silu; every head of q and k becomes a unit vector (1e-6 inside the root), q also
  times dim^(-1/2); beta = sigmoid(W_b h) a head; a decay per head and key channel
  g = exp(-exp(A_log_a) softplus(W_a2 W_a1 h + dt_bias)); per head: S <- g * S (rows of S are key
  channels), u = beta (v - S^T k), S <- S + k u^T, o = S^T q; o divided by its root mean square a
  head, times a weight of vdim numbers that heads share, times sigmoid(W_g2 W_g1 h); W_o.
* mixer ``attention``: q = W_q h + b_q, k = W_k h + b_k, the values are k as projected; q and k
  are RMS-normed over the whole projection (all heads at once) with weights of that size; q times
  1 + coef ln(floor((t + 1) / every) + 1); score(t, j) = scale q_t . k_j - r1_a ln(1 + r2_a (t - j))
  for j <= t; softmax; the heads' weights are mixed, P'_a = sum_b T[a, b] P_b; head a applies P'_a to
  the values of its own key/value head; W_o.
* feed-forward ``moe``: z = W_router f, s = sigmoid(z), the ``top`` largest s are chosen, their
  weights are s times router.scale (not renormalized); expert(f) = W_down (silu(W_gate f) W_up f);
  a shared expert of the same form is added for every token.
* logits: rms(x, final.norm) times the table.
"""
from __future__ import annotations

import numpy as np

F64 = np.float64
UNIT_EPS = 1e-6          # inside the root of the unit vectors of the delta rule


def sigmoid(a):
    a = np.asarray(a, dtype=F64)
    return 1.0 / (1.0 + np.exp(-a))


def silu(a):
    a = np.asarray(a, dtype=F64)
    return a * sigmoid(a)


def softplus(a):
    a = np.asarray(a, dtype=F64)
    return np.logaddexp(0.0, a)


def linear(x, weight, bias=None):
    y = np.asarray(x, dtype=F64) @ np.asarray(weight, dtype=F64).T
    return y if bias is None else y + np.asarray(bias, dtype=F64)


def rms_divide(v, eps: float):
    v = np.asarray(v, dtype=F64)
    return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps)


def rms_norm(v, weight, eps: float):
    return rms_divide(v, eps) * np.asarray(weight, dtype=F64)


def grouped_rms_norm(v, weight, eps: float, groups: int):
    n, width = v.shape
    parts = rms_divide(np.asarray(v, dtype=F64).reshape(n, groups, width // groups), eps)
    return parts.reshape(n, width) * np.asarray(weight, dtype=F64)


def time_conv(h, taps_weight, bias=None):
    """Causal convolution over time, channel by channel: y_t = sum_j w[:, j] h_(t - taps + 1 + j),
    zeros before the first row.  h [n, channels], taps_weight [channels, taps]."""
    h = np.asarray(h, dtype=F64)
    w = np.asarray(taps_weight, dtype=F64)
    n, taps = h.shape[0], w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, h.shape[1]), dtype=F64), h], axis=0)
    y = np.zeros_like(h)
    for j in range(taps):
        y += padded[j:j + n] * w[:, j]
    return y if bias is None else y + np.asarray(bias, dtype=F64)


def start(cfg, w, tokens):
    t = np.arange(len(tokens))
    return np.asarray(w["embed"], dtype=F64)[np.asarray(tokens)] + np.asarray(w["pos"], dtype=F64)[t]


# ---- mamba2 ----------------------------------------------------------------------------------
def mamba2_scan(xs, B, C, dt, a_log, d_skip, heads_per_group: int):
    """xs [n, heads, vdim], B and C [n, groups, N], dt [n, heads] (after softplus) -> y [n, heads, vdim]."""
    n, H, P = xs.shape
    N = B.shape[-1]
    rate = np.exp(np.asarray(a_log, dtype=F64))
    d_skip = np.asarray(d_skip, dtype=F64)
    y = np.empty((n, H, P), dtype=F64)
    S = np.zeros((H, N, P), dtype=F64)
    for t in range(n):
        for a in range(H):
            g = a // heads_per_group
            S[a] = np.exp(-rate[a] * dt[t, a]) * S[a] + dt[t, a] * np.outer(B[t, g], xs[t, a])
            y[t, a] = S[a].T @ C[t, g] + d_skip[a] * xs[t, a]
    return y


def mamba2(m, eps, w, p, h):
    n = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = linear(h, w[p + "in"])
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(time_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    xs = xbc[:, :inner].reshape(n, H, P)
    B = xbc[:, inner:inner + G * N].reshape(n, G, N)
    C = xbc[:, inner + G * N:].reshape(n, G, N)
    dt = softplus(dt + np.asarray(w[p + "dt_bias"], dtype=F64))
    y = mamba2_scan(xs, B, C, dt, w[p + "A_log"], w[p + "D"], H // G).reshape(n, inner)
    y = grouped_rms_norm(y * silu(z), w[p + "norm"], eps, m["norm_groups"])
    return linear(y, w[p + "o"])


# ---- the gated delta rule with a decay per key channel ---------------------------------------
def unit_vectors(v):
    v = np.asarray(v, dtype=F64)
    return v / np.sqrt((v * v).sum(-1, keepdims=True) + UNIT_EPS)


def delta_scan(q, k, v, beta, g):
    """q, k [n, heads, dim] (already spread over the heads), v [n, heads, vdim], beta [n, heads],
    g [n, heads, dim] -> o [n, heads, vdim]."""
    n, H, D = q.shape
    E = v.shape[-1]
    o = np.empty((n, H, E), dtype=F64)
    S = np.zeros((H, D, E), dtype=F64)
    for t in range(n):
        for a in range(H):
            S[a] = g[t, a][:, None] * S[a]
            u = beta[t, a] * (v[t, a] - S[a].T @ k[t, a])
            S[a] = S[a] + np.outer(k[t, a], u)
            o[t, a] = S[a].T @ q[t, a]
    return o


def channel_delta(m, eps, w, p, h):
    n = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(time_conv(linear(h, w[p + "q"]), w[p + "q.conv"])).reshape(n, G, D)
    k = silu(time_conv(linear(h, w[p + "k"]), w[p + "k.conv"])).reshape(n, G, D)
    v = silu(time_conv(linear(h, w[p + "v"]), w[p + "v.conv"])).reshape(n, H, E)
    q = unit_vectors(q) * F64(D) ** -0.5
    k = unit_vectors(k)
    spread = np.arange(H) // (H // G)
    q, k = q[:, spread], k[:, spread]
    beta = sigmoid(linear(h, w[p + "b"]))
    step = softplus(linear(linear(h, w[p + "a1"]), w[p + "a2"]) + np.asarray(w[p + "dt_bias"], dtype=F64)).reshape(n, H, D)
    g = np.exp(-np.exp(np.asarray(w[p + "A_log"], dtype=F64))[None, :, None] * step)
    o = delta_scan(q, k, v, beta, g)
    o = rms_divide(o, eps) * np.asarray(w[p + "norm"], dtype=F64)
    gate = sigmoid(linear(linear(h, w[p + "g1"]), w[p + "g2"])).reshape(n, H, E)
    return linear((o * gate).reshape(n, H * E), w[p + "o"])


# ---- attention -------------------------------------------------------------------------------
def query_temperature(t, coef: float, every: int):
    return 1.0 + F64(coef) * np.log(np.floor((np.asarray(t) + 1) / every) + 1.0)


def distance_bias(r1, r2, n: int):
    """[heads, n, n]: r1_a ln(1 + r2_a (t - j)) where j <= t, 0 elsewhere."""
    t = np.arange(n)
    dist = np.maximum(t[:, None] - t[None, :], 0).astype(F64)
    r1, r2 = np.asarray(r1, dtype=F64), np.asarray(r2, dtype=F64)
    return r1[:, None, None] * np.log1p(r2[:, None, None] * dist[None])


def causal_softmax(s):
    n = s.shape[-1]
    t = np.arange(n)
    s = np.where(t[None, :] <= t[:, None], s, -np.inf)
    e = np.exp(s - s.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


def attention(m, eps, w, p, h):
    n = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w[p + "q"], w[p + "q.b"])
    k = linear(h, w[p + "k"], w[p + "k.b"])
    v = k.reshape(n, G, E)                                  # the values are the keys as projected
    q = rms_norm(q, w[p + "q.norm"], eps).reshape(n, H, D)
    k = rms_norm(k, w[p + "k.norm"], eps).reshape(n, G, D)
    q = q * query_temperature(np.arange(n), m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None]
    bias = distance_bias(w[p + "r1"], w[p + "r2"], n)
    P = np.empty((H, n, n), dtype=F64)
    for a in range(H):
        P[a] = causal_softmax((q[:, a] @ k[:, a // (H // G)].T) * F64(m["scale"]) - bias[a])
    P = np.einsum("ab,bij->aij", np.asarray(w[p + "talk"], dtype=F64), P)
    out = np.empty((n, H, E), dtype=F64)
    for a in range(H):
        out[:, a] = P[a] @ v[:, a // (H // G)]
    return linear(out.reshape(n, H * E), w[p + "o"])


# ---- feed-forward ------------------------------------------------------------------------------
def expert(w, p, f):
    return linear(silu(linear(f, w[p + "gate"])) * linear(f, w[p + "up"]), w[p + "down"])


def route(z, top: int, scale: float):
    """z [n, experts] -> (chosen [n, top] in falling order of the score, weights [n, top])."""
    s = sigmoid(z)
    order = np.argsort(-s, axis=-1, kind="stable")[:, :top]
    return order, np.take_along_axis(s, order, axis=-1) * F64(scale)


def moe_ff(cfg_mlp, w, p, f):
    r = cfg_mlp["router"]
    chosen, weight = route(linear(f, w[p + "router"]), r["top"], r["scale"])
    out = np.zeros((f.shape[0], np.asarray(w[p + "e0.down"]).shape[0]), dtype=F64)
    for e in range(r["experts"]):
        rows, slot = np.nonzero(chosen == e)
        if len(rows):
            out[rows] += weight[rows, slot][:, None] * expert(w, f"{p}e{e}.", f[rows])
    if cfg_mlp.get("shared"):
        out += expert(w, p + "shared.", f)
    return out


def feed_forward(cfg_mlp, w, p, f):
    if cfg_mlp["kind"] == "moe":
        return moe_ff(cfg_mlp, w, p, f)
    raise ValueError(f"no feed-forward of kind {cfg_mlp['kind']!r}")


MIXERS = {"mamba2": mamba2, "channel_delta": channel_delta, "attention": attention}


def layer_forward(cfg, w, i, x):
    layer, p, eps = cfg["layers"][i], f"l{i}.", cfg["norm"]["eps"]
    h = rms_norm(x, w[p + "norm1"], eps)
    h = h + time_conv(h, w[p + "canon1"])
    x = x + MIXERS[layer["type"]](layer["mixer"], eps, w, p + "mix.", h)
    if layer.get("mlp"):
        x = x + feed_forward(layer["mlp"], w, p + "mlp.", rms_norm(x, w[p + "norm2"], eps))
    return x


def forward(cfg, w, tokens, layers_out=None):
    """Logits [n, vocab] of one whole sequence from position 0.  ``layers_out``: a list that
    receives the stream after every layer."""
    x = start(cfg, w, tokens)
    for i in range(len(cfg["layers"])):
        x = layer_forward(cfg, w, i, x)
        if layers_out is not None:
            layers_out.append(x.copy())
    return linear(rms_norm(x, w["final.norm"], cfg["norm"]["eps"]), w["embed"])


def greedy(cfg, w, prompt, n: int):
    """``n`` tokens after ``prompt``, each the first largest logit of the whole sequence so far."""
    tokens, out = list(prompt), []
    for _ in range(n):
        t = int(np.argmax(forward(cfg, w, tokens)[-1]))
        out.append(t)
        tokens.append(t)
    return out
