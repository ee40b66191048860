"""The Nalasun configuration, its model spec and the plain implementation, without a GPU."""
import copy

import numpy as np
import pytest

from plain import nalasun_plain as N


def moe(experts, top, ff, scale=1.0, shared=None):
    return {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale}, "expert": {"ff": ff},
            "shared": None if shared is None else {"ff": shared}}


def ssm(heads, vdim, state, groups, conv, norm_groups, mlp):
    return {"type": "mamba2", "mlp": mlp,
            "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}}


def delta(heads, kv_heads, dim, vdim, conv, mlp, ranks=(6, 5)):
    return {"type": "channel_delta", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                      "decay_rank": ranks[0], "gate_rank": ranks[1]}}


def att(heads, kv_heads, dim, scale, coef, every, mlp):
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
                      "q_temp": {"coef": coef, "every": every}}}


def config(vocab, width, positions, taps, layers, eps=1e-5):
    return {"architecture": "Nalasun", "vocab": vocab, "width": width, "max_positions": positions, "norm": {"eps": eps},
            "canon": {"taps": taps}, "layers": layers}


CFG = config(50, 24, 40, 3, [
    att(4, 2, 6, 0.4, 0.7, 5, moe(3, 1, 8, 1.5)),
    ssm(3, 4, 5, 1, 4, 3, None),
    delta(4, 2, 3, 5, 2, moe(5, 3, 12, 0.8, shared=20)),
    ssm(4, 6, 7, 4, 2, 1, moe(2, 2, 6, 2.0)),
    att(2, 2, 8, 0.3, 0.0, 1, None),
])


def random_weights(cfg, seed=0, spread=0.3):
    """Weights by the file's names for a config.json dict, drawn here (not by the package)."""
    rng = np.random.default_rng(seed)
    d = cfg["width"]
    taps = cfg["canon"]["taps"]
    w = {"embed": rng.normal(0, spread, (cfg["vocab"], d)), "pos": rng.normal(0, spread, (cfg["max_positions"], d)),
         "final.norm": rng.normal(1, 0.1, d)}
    for i, layer in enumerate(cfg["layers"]):
        p, m, f = f"l{i}.", layer["mixer"], layer["mlp"]
        q = p + "mix."
        w[p + "norm1"] = rng.normal(1, 0.1, d)
        w[p + "canon1"] = rng.normal(0, spread, (d, taps))
        if layer["type"] == "mamba2":
            inner, bc = m["heads"] * m["vdim"], 2 * m["groups"] * m["state"]
            w[q + "in"] = rng.normal(0, spread, (2 * inner + bc + m["heads"], d))
            w[q + "conv"] = rng.normal(0, spread, (inner + bc, m["conv"]))
            w[q + "conv.b"] = rng.normal(0, 0.1, inner + bc)
            w[q + "dt_bias"], w[q + "A_log"] = rng.normal(0, 0.5, m["heads"]), rng.normal(0, 0.5, m["heads"])
            w[q + "D"], w[q + "norm"] = rng.normal(1, 0.1, m["heads"]), rng.normal(1, 0.1, inner)
            w[q + "o"] = rng.normal(0, spread, (d, inner))
        elif layer["type"] == "channel_delta":
            qk, vw = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
            for name, rows in (("q", qk), ("k", qk), ("v", vw)):
                w[q + name] = rng.normal(0, spread, (rows, d))
                w[q + name + ".conv"] = rng.normal(0, spread, (rows, m["conv"]))
            w[q + "b"] = rng.normal(0, spread, (m["heads"], d))
            w[q + "A_log"], w[q + "norm"] = rng.normal(-1, 0.5, m["heads"]), rng.normal(1, 0.1, m["vdim"])
            w[q + "a1"], w[q + "a2"] = rng.normal(0, spread, (m["decay_rank"], d)), rng.normal(0, spread, (m["heads"] * m["dim"], m["decay_rank"]))
            w[q + "dt_bias"] = rng.normal(0, 0.5, m["heads"] * m["dim"])
            w[q + "g1"], w[q + "g2"] = rng.normal(0, spread, (m["gate_rank"], d)), rng.normal(0, spread, (vw, m["gate_rank"]))
            w[q + "o"] = rng.normal(0, spread, (d, vw))
        else:
            qw, kw = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
            w[q + "q"], w[q + "k"] = rng.normal(0, spread, (qw, d)), rng.normal(0, spread, (kw, d))
            w[q + "q.b"], w[q + "k.b"] = rng.normal(0, 0.1, qw), rng.normal(0, 0.1, kw)
            w[q + "q.norm"], w[q + "k.norm"] = rng.normal(1, 0.1, qw), rng.normal(1, 0.1, kw)
            w[q + "r1"], w[q + "r2"] = rng.uniform(0.2, 0.8, m["heads"]), rng.uniform(0.2, 0.8, m["heads"])
            w[q + "talk"] = np.eye(m["heads"]) * 0.7 + rng.normal(0.1, 0.1, (m["heads"], m["heads"]))
            w[q + "o"] = rng.normal(0, spread, (d, qw))
        if f is None:
            continue
        w[p + "norm2"] = rng.normal(1, 0.1, d)
        sets = [(f"{p}mlp.e{e}.", f["expert"]["ff"]) for e in range(f["router"]["experts"])]
        w[p + "mlp.router"] = rng.normal(0, 1.0, (f["router"]["experts"], d))
        if f.get("shared"):
            sets.append((p + "mlp.shared.", f["shared"]["ff"]))
        for s, ff in sets:
            w[s + "gate"], w[s + "up"] = rng.normal(0, spread, (ff, d)), rng.normal(0, spread, (ff, d))
            w[s + "down"] = rng.normal(0, spread, (d, ff))
    return w


def test_round_trip_and_registry():
    from sonicboom_amd.config.nalasun import ChannelDeltaConfig, Mamba2Config, NalasunConfig, SharedAttentionConfig
    from sonicboom_amd.config.registry import architecture_of
    arch = architecture_of(CFG)
    assert arch.name == "Nalasun" and arch.config_class is NalasunConfig
    cfg = NalasunConfig.from_dict(CFG)
    assert cfg.to_dict() == CFG
    assert NalasunConfig.from_dict(cfg.to_dict()) == cfg
    assert [type(layer.mixer) for layer in cfg.layers] == [SharedAttentionConfig, Mamba2Config, ChannelDeltaConfig, Mamba2Config,
                                                          SharedAttentionConfig]
    assert cfg.canon_taps == 3 and cfg.layers[0].mixer.temp_every == 5 and cfg.layers[2].mlp.shared_ff == 20
    assert cfg.layers[3].mlp.scale == 2.0 and cfg.layers[1].mlp is None
    # what the file does not say: ranks come from the tensors, a layer's temperature may be absent
    d = copy.deepcopy(CFG)
    del d["layers"][2]["mixer"]["decay_rank"], d["layers"][2]["mixer"]["gate_rank"], d["layers"][4]["mixer"]["q_temp"]
    cfg2 = NalasunConfig.from_dict(d)
    assert cfg2.layers[2].mixer.decay_rank == -1 and cfg2.layers[4].mixer.temp_coef == 0.0
    assert "decay_rank" not in cfg2.to_dict()["layers"][2]["mixer"]


@pytest.mark.parametrize("path, value, message", [
    (("layers", 1, "mixer", "state"), None, "layers[1].mixer.state"),
    (("layers", 0, "mixer", "scale"), "x", "layers[0].mixer.scale"),
    (("layers", 2, "mixer", "conv"), 1, "conv must be at least 2"),
    (("layers", 0, "mixer", "vdim"), 7, "vdim = 7 must equal dim"),
    (("layers", 3, "mixer", "groups"), 3, "not a multiple of 3 groups"),
    (("layers", 1, "mixer", "norm_groups"), 5, "norm_groups"),
    (("layers", 2, "mlp", "router", "top"), 6, "top = 6"),
    (("layers", 0, "type"), "conv", "unknown layer type"),
    (("canon", "taps"), 1, "canon.taps"),
    (("layers", 0, "mixer", "q_temp", "every"), 0, "temp_every must be positive"),
])
def test_errors_name_the_key(path, value, message):
    from sonicboom_amd.config.base import ConfigError
    from sonicboom_amd.config.nalasun import NalasunConfig
    d = copy.deepcopy(CFG)
    at = d
    for key in path[:-1]:
        at = at[key]
    if value is None:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    with pytest.raises(ConfigError, match=message.replace("[", r"\[").replace("]", r"\]")):
        NalasunConfig.from_dict(d)


def test_the_spec_names_the_tensors_of_the_weights():
    from sonicboom_amd.architectures.nalasun import build_spec
    from sonicboom_amd.config.nalasun import NalasunConfig
    spec = build_spec(NalasunConfig.from_dict(CFG))
    w = random_weights(CFG)
    tensors = {t.name: tuple(t.shape) for t in spec.all_tensors()}
    assert set(tensors) == set(w)
    for name, shape in tensors.items():
        assert shape == np.asarray(w[name]).shape, name
    assert [e.cache for e in spec.order] == [0, None, None, None, 4]
    assert spec.blocks[1].parts.get("ffn") is None and "l1.norm2" in spec.ignorable_tensors
    # without the ranks in the file the spec leaves those axes to the tensors
    d = copy.deepcopy(CFG)
    del d["layers"][2]["mixer"]["decay_rank"], d["layers"][2]["mixer"]["gate_rank"]
    loose = {t.name: tuple(t.shape) for t in build_spec(NalasunConfig.from_dict(d)).all_tensors()}
    assert loose["l2.mix.a1"] == (-1, 24) and loose["l2.mix.a2"] == (12, -1) and loose["l2.mix.g2"] == (20, -1)


def test_a_prefix_does_not_change_when_tokens_follow():
    w = random_weights(CFG, seed=3)
    tokens = [int(t) for t in np.random.default_rng(0).integers(0, 50, 30)]
    whole = N.forward(CFG, w, tokens)
    assert np.allclose(N.forward(CFG, w, tokens[:11]), whole[:11], atol=1e-10)


def test_the_plain_mechanisms_do_what_their_names_say():
    rng = np.random.default_rng(1)
    # the convolution sees zeros before the first row, and its last tap is the current row's
    h = rng.normal(size=(6, 3))
    taps = np.array([[0.0, 0.0, 2.0]] * 3)
    assert np.allclose(N.time_conv(h, taps), 2.0 * h)
    taps = np.array([[1.0, 0.0, 0.0]] * 3)
    assert np.allclose(N.time_conv(h, taps)[2:], h[:-2]) and np.allclose(N.time_conv(h, taps)[:2], 0.0)
    # mixing the heads' weights with the identity is plain attention: each head on its own
    m = CFG["layers"][0]["mixer"]
    w = random_weights(CFG, seed=2)
    hh = rng.normal(size=(9, 24))
    a = N.attention(m, 1e-5, w, "l0.mix.", hh)
    w2 = dict(w)
    w2["l0.mix.talk"] = np.eye(4)
    b = N.attention(m, 1e-5, w2, "l0.mix.", hh)
    assert np.abs(a - b).max() > 1e-3, "the mixing matrix of these weights must show"
    # the temperature only starts at position every - 1
    t = N.query_temperature(np.arange(12), 0.7, 5)
    assert np.allclose(t[:4], 1.0) and t[4] > 1.0 and t[9] > t[4]
    # the distance bias is zero on the diagonal and grows with the distance
    bias = N.distance_bias([0.5], [0.4], 5)[0]
    assert np.allclose(np.diag(bias), 0.0) and bias[4, 0] > bias[4, 3] > 0
    # the delta rule with beta = 1 and no decay stores v under k: reading with q = k gives v back
    k = N.unit_vectors(rng.normal(size=(1, 1, 4)))
    v = rng.normal(size=(1, 1, 5))
    o = N.delta_scan(k, k, v, np.ones((1, 1)), np.ones((1, 1, 4)))
    assert np.allclose(o, v * (k * k).sum(), atol=1e-12)
    # the state-space scan with no decay and dt = 1 sums B x^T: y = (sum_s B_s x_s^T)^T C + D x
    xs, B, C = rng.normal(size=(4, 1, 3)), rng.normal(size=(4, 1, 2)), rng.normal(size=(4, 1, 2))
    y = N.mamba2_scan(xs, B, C, np.ones((4, 1)), [-50.0], [0.5], 1)
    S = sum(np.outer(B[s, 0], xs[s, 0]) for s in range(4))
    assert np.allclose(y[3, 0], S.T @ C[3, 0] + 0.5 * xs[3, 0], atol=1e-9)
    # routing: falling scores, weights are the scores times the scale, not renormalized
    z = np.array([[0.1, 2.0, -1.0, 2.0]])
    chosen, weight = N.route(z, 3, 1.5)
    assert chosen.tolist() == [[1, 3, 0]] and np.allclose(weight, 1.5 * N.sigmoid(z[0, [1, 3, 0]]))
