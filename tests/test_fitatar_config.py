"""The Fitatar configuration, its model spec and the plain implementation, without a GPU."""
import copy
import math

import numpy as np
import pytest

from plain import fitatar_plain as P


def lat(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, mlp, base=10000.0, scaling=None, kv_from=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling is not None:
        rot["scaling"] = {"factor": scaling[0], "original": scaling[1], "fast": scaling[2], "slow": scaling[3]}
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
             "scale": scale, "rot": rot}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def att(heads, kv_heads, dim, vdim, scale, mlp, base=10000.0, rot_dims=None, factor=None):
    rot = {"base": base, "dims": dim if rot_dims is None else rot_dims}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}}


def moe(experts, top, ff, groups=None, shared=None):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "router": router, "expert": {"ff": ff}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def config(vocab, width, layers, eps=1e-5, embed_scale=1.0, softcap=0.0):
    return {"architecture": "Fitatar", "vocab": vocab, "width": width, "embedding": {"scale": embed_scale},
            "logit_softcap": softcap, "norm": {"eps": eps}, "layers": layers}


CFG = config(50, 24, [
    att(4, 2, 6, 10, 0.3, moe(6, 2, 8, groups=(3, 2), shared=12), rot_dims=4, factor=4.0),
    lat(2, 6, 4, 10, 12, 7, 0.4, {"kind": "dense", "ff": 40}, scaling=(3.0, 16, 8.0, 1.0)),
    att(3, 3, 8, 4, 0.25, None, base=500.0),
    lat(3, 4, 4, 6, 12, 9, 0.5, moe(4, 3, 10), scaling=(3.0, 16, 8.0, 1.0), kv_from=1),
], eps=2e-5, embed_scale=3.0, softcap=9.0)


def random_weights(cfg, seed=0, spread=0.3):
    """Weights by the file's names for a config.json dict, drawn here (not by the package)."""
    rng = np.random.default_rng(seed)
    d = cfg["width"]
    w = {"embed": rng.normal(0, spread, (cfg["vocab"], d)), "head": rng.normal(0, spread, (cfg["vocab"], d)),
         "final.norm": rng.normal(1, 0.1, d)}
    for i, layer in enumerate(cfg["layers"]):
        p, m, f = f"l{i}.", layer["mixer"], layer["mlp"]
        w[p + "norm1"] = rng.normal(1, 0.1, d)
        H = m["heads"]
        if layer["type"] == "attention":
            w[p + "mix.q"] = rng.normal(0, spread, (H * m["dim"], d))
            w[p + "mix.k"] = rng.normal(0, spread, (m["kv_heads"] * m["dim"], d))
            w[p + "mix.v"] = rng.normal(0, spread, (m["kv_heads"] * m["vdim"], d))
            w[p + "mix.g"] = rng.normal(0, spread, (H * m["vdim"], d))
            w[p + "mix.sink"] = rng.normal(0, 1.0, H)
        else:
            w[p + "mix.dq"] = rng.normal(0, spread, (m["q_rank"], d))
            w[p + "mix.dq.norm"] = rng.normal(1, 0.1, m["q_rank"])
            w[p + "mix.uq"] = rng.normal(0, spread, (H * (m["dim"] + m["rot_dim"]), m["q_rank"]))
            if m.get("kv_from") is None:
                w[p + "mix.dkv"] = rng.normal(0, spread, (m["kv_rank"] + m["rot_dim"], d))
                w[p + "mix.dkv.norm"] = rng.normal(1, 0.1, m["kv_rank"])
            w[p + "mix.uk"] = rng.normal(0, spread, (H * m["dim"], m["kv_rank"]))
            w[p + "mix.uv"] = rng.normal(0, spread, (H * m["vdim"], m["kv_rank"]))
            w[p + "mix.g"] = rng.normal(0, spread, (H, d))
        w[p + "mix.o"] = rng.normal(0, spread, (d, H * m["vdim"]))
        if f is None:
            continue
        w[p + "norm2"] = rng.normal(1, 0.1, d)
        if f["kind"] == "dense":
            w[p + "mlp.up"], w[p + "mlp.down"] = rng.normal(0, spread, (f["ff"], d)), rng.normal(0, spread, (d, f["ff"]))
            w[p + "mlp.up.b"], w[p + "mlp.down.b"] = rng.normal(0, spread, f["ff"]), rng.normal(0, spread, d)
            continue
        sets = [(f"{p}mlp.e{e}.", f["expert"]["ff"]) for e in range(f["router"]["experts"])]
        w[p + "mlp.router"] = rng.normal(0, 1.0, (f["router"]["experts"], d))
        if f.get("shared"):
            sets.append((p + "mlp.shared.", f["shared"]["ff"]))
            w[p + "mlp.shared.sg"] = rng.normal(0, spread, (1, d))
        for q, ff in sets:
            w[q + "up"], w[q + "down"] = rng.normal(0, spread, (ff, d)), rng.normal(0, spread, (d, ff))
    return w


def test_configuration_round_trip_and_spec():
    from sonicboom_amd.config import architecture_of
    arch = architecture_of(CFG)
    cfg = arch.config_class.from_dict(CFG)
    assert cfg.to_dict() == CFG
    assert cfg.layers[0].mlp.groups == 3 and cfg.layers[0].mlp.keep == 2 and cfg.layers[3].mlp.groups == 1
    assert cfg.layers[0].mlp.shared_ff == 12 and cfg.layers[3].mlp.shared_ff == 0 and cfg.layers[2].mlp is None
    spec = arch.build_spec(cfg)
    shapes = {t.name: t.shape for t in spec.all_tensors()}
    want = random_weights(CFG)
    assert set(shapes) == set(want), "the spec names the tensors of the file, no more and no fewer"
    for name, a in want.items():
        assert shapes[name] == a.shape, name
    assert "l3.mix.dkv" not in shapes and "l2.norm2" not in shapes and shapes["l1.mix.g"] == (2, 24)
    # the reading layer names the cache of the layer it reads and does not write it
    assert [(e.cache, e.writes_cache) for e in spec.order] == [(0, True), (1, True), (2, True), (1, False)]
    assert all(b.kind == "parallel" for b in spec.blocks)
    m0 = spec.blocks[0].parts["mixer"].params
    assert (m0["v_dim"], m0["sink"], m0["sink_scores"], m0["out_gate"], m0["scale"], m0["qkv_bias"]) == (10, True, True, True, 0.3, False)
    pos0 = spec.blocks[0].parts["mixer"].parts["position"]
    assert pos0.kind == "rope" and pos0.params["rot_dims"] == 4
    assert np.allclose(pos0.params["frequencies"], [1.0 / 4.0, 10000.0 ** -0.5 / 4.0]) and pos0.params["magnitude"] == 1.0
    pos2 = spec.blocks[2].parts["mixer"].parts["position"]
    assert np.allclose(pos2.params["frequencies"], [500.0 ** (-2.0 * i / 8) for i in range(4)]), "no scaling: plain frequencies"
    m1 = spec.blocks[1].parts["mixer"]
    assert (m1.params["q_rank"], m1.params["gate_per_head"], m1.params["own_latent"]) == (7, True, True)
    assert not spec.blocks[3].parts["mixer"].params["own_latent"]
    pos1 = m1.parts["position"]
    assert pos1.kind == "rope_interleaved" and abs(pos1.params["magnitude"] - (0.1 * math.log(3.0) + 1.0)) < 1e-12
    f0 = spec.blocks[0].parts["ffn"].params
    assert (f0["router_score"], f0["groups"], f0["keep_groups"], f0["activation"]) == ("softmax_all", 3, 2, "relu_sq")
    assert spec.blocks[1].parts["ffn"].params["activation"] == "gelu_erf"
    assert spec.head.params["softcap"] == 9.0 and spec.embedding.params["scale"] == 3.0


def test_absent_keys_mean_absent_mechanisms():
    from sonicboom_amd.config import architecture_of
    bare = copy.deepcopy(CFG)
    bare.pop("logit_softcap")
    bare.pop("embedding")
    cfg = architecture_of(bare).config_class.from_dict(bare)
    assert cfg.logit_softcap == 0.0 and cfg.embedding_scale == 1.0
    spec = architecture_of(bare).build_spec(cfg)
    assert spec.head.params["softcap"] == 0.0


@pytest.mark.parametrize("edit, message", [
    (lambda c: c["layers"][0]["mixer"].pop("heads"), "layers[0].mixer.heads"),
    (lambda c: c["layers"][1]["mixer"].pop("q_rank"), "layers[1].mixer.q_rank"),
    (lambda c: c["layers"][1].update(type="lstm"), "unknown layer type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "not a multiple"),
    (lambda c: c["layers"][3]["mixer"].update(kv_rank=16), "differ from those of layer 1"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=7), "router"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), "groups"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(keep=1, count=6), "hold fewer"),
    (lambda c: c["layers"][0]["mlp"]["expert"].pop("ff"), "layers[0].mlp.expert.ff"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("original"), "layers[1].mixer.rot.scaling.original"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][3]["mlp"].update(kind="sparse"), "unknown feed-forward"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_configuration_errors_name_the_key(edit, message):
    from sonicboom_amd.config import ConfigError, architecture_of
    bad = copy.deepcopy(CFG)
    edit(bad)
    with pytest.raises(ConfigError, match=message.replace("[", r"\[").replace("]", r"\]")):
        architecture_of(bad).config_class.from_dict(bad)


def test_the_package_stretches_frequencies_like_the_plain_implementation():
    from sonicboom_amd.parts.position import stretched_frequencies
    for dims, base, sc in [(32, 5e5, (2.5, 640, 24.0, 1.0)), (8, 100.0, (5.0, 40, 4.0, 0.5)), (64, 1e4, (40.0, 4096, 32.0, 1.0)),
                           (4, 50.0, (1.5, 8, 2.0, 1.0))]:
        rot = {"dims": dims, "base": base, "scaling": {"factor": sc[0], "original": sc[1], "fast": sc[2], "slow": sc[3]}}
        f, m = P.frequencies(rot, "yarn")
        g, n = stretched_frequencies(dims, base, "ramp", *sc)
        assert np.allclose(f, g, rtol=1e-13) and abs(m - n) < 1e-15
        f, m = P.frequencies(rot, "linear")
        g, n = stretched_frequencies(dims, base, "linear", sc[0])
        assert np.allclose(f, g, rtol=1e-13) and m == n == 1.0
    # the ramp leaves the fastest pairs alone and divides the slowest by the factor
    f, _ = P.frequencies({"dims": 64, "base": 1e4, "scaling": {"factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0}}, "yarn")
    plain, _ = P.frequencies({"dims": 64, "base": 1e4}, "yarn")
    assert f[0] == plain[0] and np.isclose(f[-1], plain[-1] / 40.0) and np.all(np.diff(f / plain) <= 1e-15)


def test_the_plain_implementation_is_causal_and_the_reader_sees_the_writers_rows():
    w = random_weights(CFG, seed=3)
    tokens = [int(t) for t in np.random.default_rng(1).integers(0, 50, size=17)]
    whole = P.forward(CFG, w, tokens)
    assert np.allclose(whole[:9], P.forward(CFG, w, tokens[:9]), atol=1e-12), "a prefix's logits do not change"
    assert np.all(np.abs(whole) <= 9.0), "the cap bounds the logits"
    # layer 3 reads what layer 1 keeps: another latent projection in layer 1 moves layer 3's result beyond layer 1's own
    lay_a, lay_b = [], []
    P.forward(CFG, w, tokens, lay_a)
    w2 = dict(w)
    w2["l1.mix.o"] = np.zeros_like(w["l1.mix.o"])          # layer 1's own attention result no longer reaches the stream
    w2["l1.mix.dkv"] = w["l1.mix.dkv"] * 1.5
    w3 = dict(w2)
    w3["l1.mix.dkv"] = w["l1.mix.dkv"]
    P.forward(CFG, w2, tokens, lay_a := [])
    P.forward(CFG, w3, tokens, lay_b := [])
    assert np.allclose(lay_a[2], lay_b[2]) and not np.allclose(lay_a[3], lay_b[3])


def test_the_sink_holds_weight_of_its_own_score():
    s = np.array([[0.0, -np.inf], [2.0, 2.0]])
    vis = np.array([[True, False], [True, True]])
    p = P.softmax_visible(s, vis, sink=np.log(3.0))
    assert np.allclose(p[0], [0.25, 0.0]) and np.allclose(p[1], np.exp(2.0) / (3.0 + 2 * np.exp(2.0)))
    assert np.allclose(P.softmax_visible(s, vis)[0], [1.0, 0.0])


def test_routing_by_groups():
    # 6 experts in 3 groups of 2; the groups' best scores are 0.20, 0.22 and 0.30: with two groups kept, expert 0
    # (the third largest of all) cannot be chosen and expert 5 takes its place
    z = np.log(np.array([[0.20, 0.19, 0.04, 0.22, 0.30, 0.05]]))
    chosen, weight = P.route(z, 3, groups=3, keep=2)
    assert chosen.tolist() == [[4, 3, 5]]
    assert np.allclose(weight, [[0.30, 0.22, 0.05]]), "the scores as they are: not renormalized"
    chosen, weight = P.route(z, 3)
    assert chosen.tolist() == [[4, 3, 0]]
    chosen, _ = P.route(np.array([[1.0, 1.0, 0.0, 1.0]]), 2)
    assert chosen.tolist() == [[0, 1]], "ties go to the lower number"


def test_rotation_pairs_and_the_gelu():
    v = np.arange(1.0, 9.0)[None, None, :]                     # one row, one head, 8 numbers
    f = np.array([0.5, 0.25])
    near = P.turn(v, [2], f, 1.0, True)[0, 0]
    c, s = np.cos(1.0), np.sin(1.0)
    assert np.allclose(near[:2], [1 * c - 2 * s, 2 * c + 1 * s]) and np.allclose(near[4:], [5, 6, 7, 8])
    half = P.turn(v, [2], f, 2.0, False)[0, 0]
    assert np.allclose([half[0], half[2]], [2 * (1 * c - 3 * s), 2 * (3 * c + 1 * s)]) and np.allclose(half[4:], [5, 6, 7, 8])
    assert np.allclose(P.gelu_erf(np.array([0.0, 1.0, -1.0])), [0.0, 0.841344746, -0.158655254])
