"""A plain, slow implementation of the Fitatar decoder.

Whole sequences, no cache, one function per mechanism, NumPy in float64 throughout.  It shares no
code with ``sonicboom_amd``: the configuration is the dict of config.json and the weights a dict of
arrays by the file's tensor names.

The design in this file's notation (``n`` tokens, position t = 0 .. n-1, stream x [n, width],
n(v, w) = v / sqrt(mean(v^2) + eps) * w):

* start: x = table[token] * embedding.scale.
* a layer has two branches that read the same stream: x <- x + mixer(n(x, norm1)) + ff(n(x, norm2)).
* mixer ``latent_attention``: cq = n(Wdq h, dq.norm), q = Wuq cq, head a = [dim plain | rot_dim turned];
  Wdkv h = [kv_rank numbers | rot_dim numbers]: c = n(first, dkv.norm), r = turned second, one for all
  heads; head a's key is [Wuk,a c | r], its value Wuv,a c; s = scale * q.k over j <= t, softmax; head a's
  result times sigmoid((Wg h)_a), one number a head; then Wo.  Pairs (2i, 2i+1) turn, with frequencies
  stretched between two wavelengths (YaRN) and cosine and sine times 0.1 ln(factor) + 1.  A layer with
  ``kv_from`` has no Wdkv and takes c and r of the layer it names.
* mixer ``attention``: q, k, v = W h; heads of ``dim`` for q and k, ``vdim`` for v; query head a reads
  key/value head a // (heads / kv_heads); pairs (i, i + dims/2) of the first ``rot.dims`` numbers turn
  by t * base^(-2i/dims) / factor; s = scale * q.k over j <= t; weights exp(s_j) / (exp(sink_a) + sum_j
  exp(s_j)); the heads side by side times sigmoid(Wg h), number by number; then Wo.
* feed-forward ``dense``: Wdown gelu(Wup h + b_up) + b_down, gelu by the error function.
* feed-forward ``moe``: z = Wrouter h, s = softmax(z) over all experts; the experts lie in
  ``groups.count`` equal groups of neighbours, a group's score is its largest s, the best ``groups.keep``
  groups stay; among their experts the ``top`` largest s are chosen and weigh s as it is; an expert is
  Wdown relu(Wup h)^2; a shared expert of the same form is added times sigmoid(Wsg h).
* logits: cap * tanh((head n(x, final.norm)) / cap).
"""
from __future__ import annotations

import math

import numpy as np

F64 = np.float64


def sigmoid(a):
    a = np.asarray(a, dtype=F64)
    return 1.0 / (1.0 + np.exp(-a))


def linear(x, weight, bias=None):
    y = np.asarray(x, dtype=F64) @ np.asarray(weight, dtype=F64).T
    return y if bias is None else y + np.asarray(bias, dtype=F64)


def norm(v, weight, eps: float):
    v = np.asarray(v, dtype=F64)
    return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps) * np.asarray(weight, dtype=F64)


def gelu_erf(z):
    z = np.asarray(z, dtype=F64)
    return 0.5 * z * (1.0 + np.vectorize(math.erf)(z / math.sqrt(2.0)))


# ---- rotation -----------------------------------------------------------------------------------

def frequencies(rot: dict, kind: str):
    """(frequency of every pair, multiplier of cosine and sine) for a ``rot`` object of config.json.
    ``kind``: "linear" (every frequency over the factor) or "yarn"."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor = float(sc["factor"])
    if kind == "linear":
        return f / factor, 1.0

    def where(turns):           # the pair whose wavelength makes `turns` turns over the original length
        return dims * math.log(float(sc["original"]) / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(float(sc["fast"]))), 0)
    hi = min(math.ceil(where(float(sc["slow"]))), dims - 1)
    i = np.arange(dims // 2, dtype=F64)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def turn(v, positions, freq, magnitude: float, interleaved: bool):
    """v [n, ..., m]: the first 2 len(freq) numbers of the last axis turn, the rest pass."""
    v = np.array(v, dtype=F64)
    half = len(freq)
    ang = np.asarray(positions, dtype=F64)[:, None] * freq[None, :]
    shape = (v.shape[0],) + (1,) * (v.ndim - 2) + (half,)
    c, s = (np.cos(ang) * magnitude).reshape(shape), (np.sin(ang) * magnitude).reshape(shape)
    if interleaved:
        a, b = v[..., 0:2 * half:2].copy(), v[..., 1:2 * half:2].copy()
        v[..., 0:2 * half:2], v[..., 1:2 * half:2] = a * c - b * s, b * c + a * s
    else:
        a, b = v[..., :half].copy(), v[..., half:2 * half].copy()
        v[..., :half], v[..., half:2 * half] = a * c - b * s, b * c + a * s
    return v


# ---- softmax ------------------------------------------------------------------------------------

def softmax_visible(s, visible, sink=None):
    """Row by row over the visible keys; ``sink``: one more score per row that holds weight and has no value."""
    s = np.where(visible, s, -np.inf)
    m = s.max(-1, keepdims=True)
    if sink is not None:
        m = np.maximum(m, sink)
    e = np.exp(s - m)
    denom = e.sum(-1, keepdims=True)
    if sink is not None:
        denom = denom + np.exp(sink - m)
    return e / denom


def causal(positions_q, positions_k):
    return np.asarray(positions_k)[None, :] <= np.asarray(positions_q)[:, None]


# ---- mixers ---------------------------------------------------------------------------------------

def latent_rows(mx, eps, w, p, h, positions):
    """What a layer with a latent of its own keeps per token: (c [n, kv_rank], r [n, rot_dim] turned)."""
    rank = mx["kv_rank"]
    both = linear(h, w[p + "dkv"])
    c = norm(both[:, :rank], w[p + "dkv.norm"], eps)
    freq, mag = frequencies(mx["rot"], "yarn")
    return c, turn(both[:, rank:], positions, freq, mag, True)


def latent_attention(mx, eps, w, p, h, kept, positions=None):
    """``kept``: (c, r) of every position of the sequence so far, from this layer or the one it names."""
    n = h.shape[0]
    positions = np.arange(n) if positions is None else np.asarray(positions)
    H, D, R, E, rank = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    cq = norm(linear(h, w[p + "dq"]), w[p + "dq.norm"], eps)
    q = linear(cq, w[p + "uq"]).reshape(n, H, D + R)
    freq, mag = frequencies(mx["rot"], "yarn")
    q_rot = turn(q[:, :, D:], positions, freq, mag, True)
    c, r = kept
    k_plain = linear(c, w[p + "uk"]).reshape(-1, H, D)
    v = linear(c, w[p + "uv"]).reshape(-1, H, E)
    visible = causal(positions, np.arange(c.shape[0]))
    gate = sigmoid(linear(h, w[p + "g"]))                       # [n, H]
    out = np.empty((n, H, E), dtype=F64)
    for a in range(H):
        s = (q[:, a, :D] @ k_plain[:, a].T + q_rot[:, a] @ r.T) * F64(mx["scale"])
        out[:, a] = (softmax_visible(s, visible) @ v[:, a]) * gate[:, a:a + 1]
    return linear(out.reshape(n, H * E), w[p + "o"])


def attention(mx, w, p, h, positions=None, kept=None):
    """``kept``: (k [m, G, D] turned, v [m, G, E]) of earlier positions, put in front of this call's own."""
    n = h.shape[0]
    H, G, D, E = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    first = 0 if kept is None else kept[0].shape[0]
    positions = np.arange(first, first + n) if positions is None else np.asarray(positions)
    freq, mag = frequencies(mx["rot"], "linear")
    q = turn(linear(h, w[p + "q"]).reshape(n, H, D), positions, freq, mag, False)
    k = turn(linear(h, w[p + "k"]).reshape(n, G, D), positions, freq, mag, False)
    v = linear(h, w[p + "v"]).reshape(n, G, E)
    if kept is not None:
        k, v = np.concatenate([kept[0], k]), np.concatenate([kept[1], v])
    visible = causal(positions, np.arange(k.shape[0]))
    sink = np.asarray(w[p + "sink"], dtype=F64)
    out = np.empty((n, H, E), dtype=F64)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * F64(mx["scale"])
        out[:, a] = softmax_visible(s, visible, sink[a]) @ v[:, g]
    gated = out.reshape(n, H * E) * sigmoid(linear(h, w[p + "g"]))
    return linear(gated, w[p + "o"]), (k, v)


# ---- feed-forwards ----------------------------------------------------------------------------------

def dense_ff(w, p, h):
    return linear(gelu_erf(linear(h, w[p + "up"], w[p + "up.b"])), w[p + "down"], w[p + "down.b"])


def expert(w, p, h):
    return linear(np.maximum(linear(h, w[p + "up"]), 0.0) ** 2, w[p + "down"])


def route(z, top: int, groups: int = 1, keep: int = 1):
    """z [n, experts] -> (chosen [n, top] in falling order of score, their scores [n, top])."""
    z = np.asarray(z, dtype=F64)
    e = np.exp(z - z.max(-1, keepdims=True))
    s = e / e.sum(-1, keepdims=True)
    n, E = s.shape
    allowed = np.ones_like(s, dtype=bool)
    if groups > 1:
        best = s.reshape(n, groups, E // groups).max(-1)                      # [n, groups]
        kept = np.argsort(-best, axis=-1, kind="stable")[:, :keep]
        ok = np.zeros((n, groups), dtype=bool)
        np.put_along_axis(ok, kept, True, axis=-1)
        allowed = np.repeat(ok, E // groups, axis=-1)
    order = np.argsort(-np.where(allowed, s, -1.0), axis=-1, kind="stable")[:, :top]
    return order, np.take_along_axis(s, order, axis=-1)


def moe_ff(mlp, w, p, h):
    n = h.shape[0]
    r = mlp["router"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    chosen, weight = route(linear(h, w[p + "router"]), r["top"], g["count"], g["keep"])
    out = np.zeros((n, np.asarray(w[p + "e0.down"]).shape[0]), dtype=F64)
    for e in range(r["experts"]):
        rows, slot = np.nonzero(chosen == e)
        if len(rows):
            out[rows] += weight[rows, slot][:, None] * expert(w, f"{p}e{e}.", h[rows])
    if mlp.get("shared"):
        out += sigmoid(linear(h, w[p + "shared.sg"])) * expert(w, p + "shared.", h)
    return out


def feed_forward(mlp, w, p, h):
    if mlp["kind"] == "dense":
        return dense_ff(w, p, h)
    if mlp["kind"] == "moe":
        return moe_ff(mlp, w, p, h)
    raise ValueError(f"no feed-forward of kind {mlp['kind']!r}")


# ---- the model ----------------------------------------------------------------------------------------

def start(cfg, w, tokens):
    return np.asarray(w["embed"], dtype=F64)[np.asarray(tokens)] * F64(cfg["embedding"]["scale"])


def logits_of(cfg, w, x):
    z = linear(norm(x, w["final.norm"], cfg["norm"]["eps"]), w["head"])
    cap = cfg.get("logit_softcap")
    return F64(cap) * np.tanh(z / F64(cap)) if cap else z


def forward(cfg, w, tokens, layers_out=None):
    """Logits [n, vocab] of one whole sequence from position 0.  ``layers_out``: a list that
    receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = start(cfg, w, tokens)
    positions = np.arange(len(tokens))
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", layer["mixer"]
        h = norm(x, w[p + "norm1"], eps)
        if layer["type"] == "latent_attention":
            src = mx.get("kv_from")
            if src is None:
                kept[i] = latent_rows(mx, eps, w, p + "mix.", h, positions)
                src = i
            y = latent_attention(mx, eps, w, p + "mix.", h, kept[src], positions)
        elif layer["type"] == "attention":
            y, _ = attention(mx, w, p + "mix.", h, positions)
        else:
            raise ValueError(f"layer {i}: no mixer of type {layer['type']!r}")
        if layer.get("mlp"):
            y = y + feed_forward(layer["mlp"], w, p + "mlp.", norm(x, w[p + "norm2"], eps))
        x = x + y
        if layers_out is not None:
            layers_out.append(x.copy())
    return logits_of(cfg, w, x)


def greedy(cfg, w, prompt, n: int):
    """``n`` tokens after ``prompt``, each the first largest logit of the whole sequence so far."""
    tokens, out = list(prompt), []
    for _ in range(n):
        t = int(np.argmax(forward(cfg, w, tokens)[-1]))
        out.append(t)
        tokens.append(t)
    return out
