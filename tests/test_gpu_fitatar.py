"""The Fitatar design on the GPU against the plain implementation of tests/plain/fitatar_plain.py:
every mechanism alone, whole models of several shapes, prompts cut into portions, token-by-token
decoding, batches of unequal requests on a cache that is used again, one key planted far away and at
both sides of page borders for both mixers (the design's attention sees every key), a sink that must
take its weight, long decoding through the recorded decode step, and greedy generation through the
Python entry point, the command line and the replay program."""
import json
import os

import numpy as np
import pytest
import torch

import helpers
from helpers import run_batch, run_tail_one_by_one, run_whole
from plain import fitatar_plain as P
from test_fitatar_config import att, config, lat, moe

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16
DTYPES = ["float32", "bfloat16"]
TORCH_DT = {"float32": F32, "bfloat16": BF16}
CODES = 8          # channels at the end of the stream that carry a code of the token for the routers

# A: sizes in sixteens (the matrix-core attention kernels and products in bfloat16); a latent layer first, a reader
#    of its rows last, attention with fewer kv heads than heads and values wider than keys, a partly rotated head,
#    routers with and without groups, with and without the expert that every row takes, one layer without a
#    feed-forward, a dense layer in the middle.
# B: sizes that are no multiple of 8 or 16 (plain products, the plain attention kernels), attention first, no
#    stretched frequencies in one layer of each kind, one head, an embedding multiplier of 1, no cap on the logits.
# C: two latents of their own with a reader each, one kv head, every expert chosen (top = experts), groups of one.
CONFIGS = {
    "A": config(160, 96, [
        lat(4, 32, 16, 48, 64, 40, 0.16, {"kind": "dense", "ff": 80}, base=1e4, scaling=(4.0, 64, 16.0, 1.0)),
        att(4, 2, 32, 48, 0.2, moe(6, 2, 32, groups=(3, 1), shared=48), rot_dims=16, factor=8.0),
        att(6, 2, 16, 16, 0.3, None, base=1e5, factor=2.0),
        att(8, 8, 32, 16, 0.2, moe(4, 1, 48)),
        lat(2, 16, 16, 32, 64, 24, 0.2, moe(8, 3, 16, groups=(2, 1), shared=16), base=1e4, scaling=(4.0, 64, 16.0, 1.0), kv_from=0),
    ], eps=3e-4, embed_scale=4.0, softcap=12.0),
    "B": config(131, 60, [
        att(3, 3, 10, 14, 0.35, {"kind": "dense", "ff": 52}, rot_dims=6),
        lat(1, 10, 6, 14, 20, 9, 0.3, moe(3, 2, 20, shared=36), base=300.0),
        att(5, 1, 6, 10, 0.5, moe(6, 4, 12, groups=(2, 2)), base=77.0, factor=3.0),
        lat(3, 6, 6, 5, 20, 13, 0.4, {"kind": "dense", "ff": 30}, base=300.0, kv_from=1),
    ], eps=1e-6),
    "C": config(200, 64, [
        lat(2, 16, 8, 16, 32, 16, 0.25, moe(4, 4, 24, shared=40), base=5e5, scaling=(16.0, 128, 32.0, 1.0)),
        lat(4, 8, 8, 24, 32, 48, 0.3, moe(5, 2, 8, groups=(5, 3)), base=5e5, scaling=(16.0, 128, 32.0, 1.0), kv_from=0),
        lat(3, 24, 16, 8, 48, 16, 0.2, {"kind": "dense", "ff": 136}, base=1e3, scaling=(1.5, 32, 4.0, 2.0)),
        att(4, 1, 64, 32, 0.12, moe(2, 1, 56), factor=1.25),
        lat(1, 16, 16, 64, 48, 8, 0.3, None, base=1e3, scaling=(1.5, 32, 4.0, 2.0), kv_from=2),
    ], eps=1e-5, embed_scale=0.25, softcap=30.0),
}
SEEDS = {"A": 31, "B": 32, "C": 33}
_FOLDERS, _PLAIN, _ENGINES, _WANT = {}, {}, {}, {}


def coded_routers(cfg, w):
    """Routers whose choice does not hang on a close call.  The plain implementation sums in float64 and the
    bfloat16 path rounds what the router reads: two scores a hair apart would be ordered differently by the two.
    So the last CODES channels of the stream carry a code of the token (one of them set, the others 0) that no
    sublayer writes to (the rows of every matrix that writes into the stream are zero there), and the routers read
    those channels alone, with levels that put the scores of every code about a unit apart (the norm in front of
    the router divides the code by the stream's root mean square, which grows from layer to layer: every router's
    levels are set from what a sample prompt's rows look like at its layer).  Every expert is still chosen by
    some code."""
    d = cfg["width"]
    r = slice(d - CODES, d)
    code = np.zeros((cfg["vocab"], CODES))
    code[np.arange(cfg["vocab"]), np.arange(cfg["vocab"]) % CODES] = 1.0
    typical = float(np.sqrt((w["embed"][:, : d - CODES] ** 2).mean())) * cfg["embedding"]["scale"]
    w["embed"][:, r] = code * typical * np.sqrt(d) / cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        p, f = f"l{i}.", layer["mlp"]
        w[p + "mix.o"][r] = 0.0
        if f is None:
            continue
        w[p + "norm2"][r] = 1.0
        for name in [n for n in w if n.startswith(p + "mlp.") and n.endswith("down")]:
            w[name][r] = 0.0
        if f["kind"] == "dense":
            w[p + "mlp.down.b"][r] = 0.0
    sample = [int(t) for t in np.random.default_rng(5).integers(0, cfg["vocab"], size=96)]
    for i, layer in enumerate(cfg["layers"]):
        p, f = f"l{i}.", layer["mlp"]
        if f is None or f["kind"] != "moe":
            continue
        before = []
        P.forward(dict(cfg, layers=cfg["layers"][:i]), w, sample, before)
        x = before[-1] if before else P.start(cfg, w, sample)
        seen = float(np.median(P.norm(x, w[p + "norm2"], cfg["norm"]["eps"])[:, r].max(axis=1)))     # a set code channel after the norm
        e = f["router"]["experts"]
        # [experts, codes]: code c ranks the experts by (number - c + layer) mod experts
        levels = ((np.arange(e)[:, None] - np.arange(CODES)[None, :] + i) % e).astype(np.float64)
        router = np.zeros((e, d))
        router[:, r] = levels * 1.2 / seen
        w[p + "mlp.router"] = np.asarray(torch.from_numpy(router).to(BF16).float().numpy(), dtype=np.float64)
    return w


def sharpen(cfg, w, coded=True, qk_gain=10.0):
    """Random N(0, 0.02) weights give flat scores, gates at one half and activations in their linear part.  Scale
    the projections so that scores spread over several units, gates move and the activations bend."""
    out = {}
    for name, a in w.items():
        a = np.array(a, dtype=np.float64)
        if name.endswith((".mix.q", ".mix.k", ".mix.dq", ".mix.uq", ".mix.dkv", ".mix.uk")):
            a = a * qk_gain
        elif name.endswith((".mix.v", ".mix.uv", ".mix.o", ".mix.g")):
            a = a * 8.0
        elif name.endswith((".up", ".down", ".sg")):
            a = a * 6.0
        elif name.endswith((".up.b", ".down.b")):
            a = a * 20.0
        elif name.endswith(".sink"):
            a = a * 3.0
        elif name.endswith(".router"):
            a = a * 40.0
        elif name in ("embed", "head"):
            a = a * 20.0
        elif name.endswith(("norm", "norm1", "norm2")):
            a = 1.0 + (a - 1.0) * 8.0
        out[name] = a
    return coded_routers(cfg, out) if coded else out


def make_folder(tmp_path_factory, name, cfg, seed, coded=True, qk_gain=10.0):
    from safetensors.torch import load_file, save_file
    from sonicboom_amd.weights import write_random_model
    folder = str(tmp_path_factory.mktemp(f"fitatar_{name}"))
    write_random_model(folder, json.loads(json.dumps(cfg)), seed=seed, dtype="bfloat16", device=None)
    path = os.path.join(folder, "model.safetensors")
    w = sharpen(cfg, {k: v.float().numpy() for k, v in load_file(path).items()}, coded, qk_gain)
    save_file({k: torch.from_numpy(np.asarray(v, dtype=np.float32)).to(BF16).contiguous() for k, v in w.items()}, path,
              metadata={"format": "pt"})
    plain = {k: v.float().numpy().astype(np.float64) for k, v in load_file(path).items()}
    return folder, plain


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """name -> folder with config.json and bfloat16 weights (sharpened, routers coded as above)."""
    for name, cfg in CONFIGS.items():
        if name not in _FOLDERS:
            _FOLDERS[name], _PLAIN[name] = make_folder(tmp_path_factory, name, cfg, SEEDS[name])
    return _FOLDERS


def engine_for(folder, dtype, max_tokens=64 * 24, **kw):
    from sonicboom_amd.engine import DecoderModel, Engine
    key = (folder, dtype, max_tokens, tuple(sorted(kw.items())))
    if key not in _ENGINES:
        _ENGINES[key] = Engine(DecoderModel.from_folder(folder, dtype), max_tokens, **kw)
    return _ENGINES[key]


def want_logits(name, tokens):
    key = (name, tuple(tokens))
    if key not in _WANT:
        _WANT[key] = P.forward(CONFIGS[name], _PLAIN[name], list(tokens))
    return _WANT[key]


def prompts(name, lengths, seed=0):
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, CONFIGS[name]["vocab"], size=n)] for n in lengths]


# Bounds.  float32 differs from the plain implementation (float64) by the rounding of float32 sums.
# bfloat16 is measured in spreads of the logits (their standard deviation): the largest difference
# and the root mean square of all differences of a request.
F32_BOUND = 3e-4
BF16_WORST, BF16_RMS = 0.22, 0.013       # what the whole file measured (0.1585 and 0.0090: the models are sharpened) times 1.4
helpers.BF16_MAX["parallel branches"], helpers.BF16_RMS["parallel branches"] = BF16_WORST, BF16_RMS


def close(got, want, dtype, what):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: not finite"
    spread = max(float(want.std()), 1e-30)
    err = np.abs(got - want) / spread
    if dtype in ("float32", F32):
        assert err.max() <= F32_BOUND, f"{what}: differs by {err.max():.3g} spreads at {np.unravel_index(err.argmax(), err.shape)}"
    else:
        rms = float(np.sqrt((err ** 2).mean()))
        seen = helpers.BF16_SEEN.setdefault("parallel branches", [0.0, 0.0])
        seen[0], seen[1] = max(seen[0], float(err.max())), max(seen[1], rms)
        assert err.max() <= BF16_WORST and rms <= BF16_RMS, \
            f"{what}: differs by {err.max():.3g} spreads at {np.unravel_index(err.argmax(), err.shape)}, rms {rms:.3g}"


def run_cuts(engine, tokens, cuts):
    """One request fed in portions of the given sizes; logits of every position."""
    from sonicboom_amd.engine import StepEntry
    assert sum(cuts) == len(tokens)
    s = engine.alloc_slot()
    try:
        rows, at = [], 0
        for n in cuts:
            rows.append(engine.step([StepEntry(s, tokens[at:at + n], range(n))]).cpu().numpy())
            at += n
        return np.concatenate(rows, axis=0)
    finally:
        engine.free_slot(s)


# ---- whole models -------------------------------------------------------------------------------
def test_the_routers_of_these_models_make_no_close_calls(folders):
    for name, cfg in CONFIGS.items():
        tokens = prompts(name, [120], seed=3)[0]
        lay = []
        P.forward(cfg, _PLAIN[name], tokens, lay)
        x = P.start(cfg, _PLAIN[name], tokens)
        for i, layer in enumerate(cfg["layers"]):
            f = layer["mlp"]
            if f is not None and f["kind"] == "moe":
                r = f["router"]
                z = P.linear(P.norm(x, _PLAIN[name][f"l{i}.norm2"], cfg["norm"]["eps"]), _PLAIN[name][f"l{i}.mlp.router"])
                g = r.get("groups") or {"count": 1, "keep": 1}
                zs = np.sort(z, axis=1)[:, ::-1]
                assert np.abs(np.diff(zs, axis=1)).min() > 0.3, (name, i, "scores a third of a unit apart at least")
                assert zs[:, 0].max() - zs[:, -1].min() < 14.0, "and no softmax that is one expert alone"
                chosen, weight = P.route(z, r["top"], g["count"], g["keep"])
                assert len(np.unique(chosen)) == r["experts"], "every expert is chosen by some token"
                if g["keep"] < g["count"] and r["experts"] > g["count"]:       # (groups of one expert never change a choice)
                    free, _ = P.route(z, r["top"])
                    assert (np.sort(free, axis=1) != np.sort(chosen, axis=1)).any(), "the groups decide some choice"
            x = lay[i]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_requests_and_the_first_tokens(folders, name, dtype):
    eng = engine_for(folders[name], dtype)
    for tokens in prompts(name, [1, 2, 3, 17, 63, 64, 65, 200]):
        close(run_whole(eng, tokens), want_logits(name, tokens), dtype, f"{name} whole n={len(tokens)}")
    assert eng.cache.held_pages() == 0 and not eng.cache.live_slots


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_stream_after_every_layer_in_32_bit(folders, name):
    eng = engine_for(folders[name], "float32")
    tokens = prompts(name, [75], seed=11)[0]
    got = []
    eng.tracer = lambda what, x: got.append(x.detach().cpu().numpy().copy()) if what.endswith(("after_ffn",)) or (
        what.endswith("after_mixer") and CONFIGS[name]["layers"][int(what.split(".")[0][5:])]["mlp"] is None) else None
    try:
        run_whole(eng, tokens)
    finally:
        eng.tracer = None
    want = []
    P.forward(CONFIGS[name], _PLAIN[name], tokens, want)
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        assert np.abs(a - b).max() <= 2e-5 * np.abs(b).max(), f"{name}: the stream after layer {i}"


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_random_routers_in_32_bit(tmp_path_factory, name):
    """The same models with routers of plain random weights (scores as close as chance makes them)."""
    folder, plain = make_folder(tmp_path_factory, name + "_random", CONFIGS[name], SEEDS[name] + 100, coded=False)
    eng = engine_for(folder, "float32")
    for tokens in prompts(name, [90, 5], seed=4):
        close(run_whole(eng, tokens), P.forward(CONFIGS[name], plain, tokens), "float32", f"{name} random routers")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prompt_against_token_by_token(folders, name, dtype):
    eng = engine_for(folders[name], dtype)
    for tokens in prompts(name, [40, 150], seed=1):
        got = run_tail_one_by_one(eng, tokens, tail=len(tokens) - 3)
        close(got, want_logits(name, tokens), dtype, f"{name} one by one n={len(tokens)}")
        if dtype == "float32":
            assert np.array_equal(got, run_whole(eng, tokens)), "in 32-bit the cut must not matter by a bit"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_portions_of_several_sizes(folders, name, dtype):
    eng = engine_for(folders[name], dtype)
    tokens = prompts(name, [331], seed=2)[0]
    whole = run_whole(eng, tokens)
    for cuts in ([2] * 20 + [291], [64, 64, 64, 139], [63, 2, 65, 1, 127, 3, 70], [130, 2, 2, 129, 68], [1, 330]):
        got = run_cuts(eng, tokens, cuts)
        close(got, want_logits(name, tokens), dtype, f"{name} cuts {cuts[:4]}")
        if dtype == "float32":
            assert np.array_equal(got, whole), f"cuts {cuts[:4]} change bits"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_unequal_batches_on_a_cache_that_is_used_again(folders, name, dtype):
    """Nine pages: every batch fills eight of them, the next gets used pages and slots."""
    eng = engine_for(folders[name], dtype, max_tokens=64 * 9, max_slots=5)
    lens = [(1, 9), (70, 4), (5, 30), (130, 12), (33, 1)]
    for round_ in range(3):
        reqs = prompts(name, [p + d for p, d in lens], seed=20 + round_)
        got = run_batch(eng, reqs, [p for p, _ in lens])
        for r, (p, _), g in zip(reqs, lens, got):
            close(g, want_logits(name, r), dtype, f"{name} batch, request of {len(r)}")
        if dtype == "float32":
            alone = run_tail_one_by_one(eng, reqs[3], tail=lens[3][1])
            assert np.array_equal(got[3], alone), "in 32-bit the batch must not matter by a bit"
        assert eng.cache.held_pages() == 0 and not eng.cache.live_slots


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_that_runs_in_portions(folders, dtype):
    """A step of more rows than the engine takes at once is cut inside sequences."""
    eng = engine_for(folders["A"], dtype, max_tokens=64 * 12, max_step_rows=100)
    reqs = prompts("A", [130, 7, 220], seed=5)
    got = run_batch(eng, reqs, [130, 7, 220])
    for r, g in zip(reqs, got):
        close(g, want_logits("A", r), dtype, f"portions, request of {len(r)}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_long_decoding_through_the_decode_loop(folders, name, dtype):
    """150 single-token steps of two sequences past page borders, kernel by kernel and then replayed
    from the recorded step; logits of every step against the plain implementation."""
    eng = engine_for(folders[name], dtype)
    reqs = prompts(name, [60 + 150, 3 + 150], seed=7)
    heads = [60, 3]
    from sonicboom_amd.engine import StepEntry
    slots = [eng.alloc_slot() for _ in reqs]
    try:
        eng.step([StepEntry(s, r[:h], ()) for s, r, h in zip(slots, reqs, heads)])
        loop = eng.decode_loop()
        assert loop.use_graph, "every part of the model says its step can be recorded"
        loop.start(slots, [r[h] for r, h in zip(reqs, heads)])
        rows = [[], []]
        for k in range(150):
            logits = loop.step_logits([r[h + k] for r, h in zip(reqs, heads)]).cpu().numpy()
            for i in range(2):
                rows[i].append(logits[i])
        for r, h, got in zip(reqs, heads, rows):
            close(np.stack(got), want_logits(name, r)[h:], dtype, f"{name} long decoding")
    finally:
        for s in slots:
            eng.free_slot(s)


def test_greedy_generation_through_the_entry_point(folders):
    from sonicboom_amd.api import Model
    for name in ("A", "B"):
        ps = prompts(name, [4, 70, 19], seed=9)
        session = Model.load(folders[name], dtype="float32").session(max_tokens=64 * 8)
        got = session.generate(ps, max_tokens=12, stop_tokens=())
        assert got == [P.greedy(CONFIGS[name], _PLAIN[name], p, 12) for p in ps]
        assert [session.generate([p], max_tokens=12, stop_tokens=())[0] for p in ps] == got
        assert not session.engine.cache.live_slots
        # bfloat16: every chosen token is the plain implementation's best or within rounding of it
        session = Model.load(folders[name], dtype="bfloat16").session(max_tokens=64 * 8)
        for p, out in zip(ps, session.generate(ps, max_tokens=12, stop_tokens=())):
            logits = want_logits(name, p + out)
            for i, t in enumerate(out):
                row = logits[len(p) - 1 + i]
                assert row[t] >= row.max() - 2 * BF16_WORST * row.std(), (name, i)


def test_command_line_and_trace_replay(folders, tmp_path):
    """The command line generates from a folder of this design; the replay program feeds a prompt, then
    its next tokens one by one beside a second request, frees one and goes on, and writes the logits
    the plain implementation gives."""
    import subprocess
    import sys
    from conftest import ROOT
    name = "B"
    ps = prompts(name, [4, 10], seed=9)
    tokens = tmp_path / "prompts.txt"
    tokens.write_text("\n".join(" ".join(map(str, p)) for p in ps) + "\n")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "sb-gen"), "-m", folders[name], "--tokens", str(tokens), "-n", "6",
           "--dtype", "fp32", "--stop", ""]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    got = [[int(t) for t in line.split()] for line in out.stdout.strip().splitlines()]
    assert got == [P.greedy(CONFIGS[name], _PLAIN[name], p, 6) for p in ps]
    a, b = prompts(name, [75, 12], seed=10)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:70], "want": [0, 69]}, {"id": "b", "tokens": b[:9], "want": [8]}], "end": []}]
    for k in range(3):
        steps.append({"step": k + 1, "entries": [{"id": "a", "tokens": [a[70 + k]], "want": [0]},
                                                 {"id": "b", "tokens": [b[9 + k]], "want": [] if k == 1 else [0]}],
                      "end": ["b"] if k == 2 else []})
    steps.append({"step": 4, "entries": [{"id": "a", "tokens": a[73:75], "want": [1]}], "end": ["a"]})
    for dtype in DTYPES:
        outdir = tmp_path / f"out_{dtype}"
        run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", dtype,
                              "--out", str(outdir), "--max-tokens", "256"], input="\n".join(json.dumps(x) for x in steps) + "\n",
                             capture_output=True, text=True, timeout=300)
        assert run.returncode == 0, run.stderr
        assert [ln for ln in run.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(5)]
        wa, wb = want_logits(name, a), want_logits(name, b)
        vocab = CONFIGS[name]["vocab"]
        read = lambda i: np.fromfile(outdir / f"{i}.f32", dtype="<f4").reshape(-1, vocab)
        close(read(0), np.stack([wa[0], wa[69], wb[8]]), dtype, "replay, prompts")
        close(read(1), np.stack([wa[70], wb[9]]), dtype, "replay, first single tokens")
        close(read(2), wa[71:72], dtype, "replay, a step where one request wants nothing")
        close(read(3), np.stack([wa[72], wb[11]]), dtype, "replay, last step of the short request")
        close(read(4), wa[74:75], dtype, "replay, two more tokens alone")


def drawn_configuration(seed):
    """A configuration from a seed: two to five layers in any order of kinds (a latent layer may read an earlier
    one's rows), head counts with one, several and as many kv heads as heads, sizes with and without factors of 8
    and 16, partly rotated heads, rotations with and without stretched frequencies, every kind of feed-forward and
    none, routers with and without groups and with and without the expert that every row takes."""
    rng = np.random.default_rng(1000 + seed)
    pick = lambda *v: v[int(rng.integers(len(v)))]
    width = pick(48, 64, 72, 100, 128, 192)
    layers, latents = [], {}
    for i in range(int(rng.integers(2, 6))):
        kind = pick("dense", "moe", "moe", None)
        if kind == "dense":
            mlp = {"kind": "dense", "ff": pick(40, 64, 100, 136)}
        elif kind == "moe":
            experts = pick(2, 3, 4, 6, 8, 12)
            count = pick(*[g for g in (1, 2, 3, 4, 6) if experts % g == 0])
            keep = int(rng.integers(1, count + 1))
            top = int(rng.integers(1, keep * (experts // count) + 1))
            mlp = moe(experts, top, pick(8, 20, 32, 48), groups=None if count == 1 and rng.random() < 0.5 else (count, keep),
                      shared=pick(None, 24, 64))
        else:
            mlp = None
        if rng.random() < 0.5:
            heads = pick(1, 2, 3, 4, 6, 8)
            kv_heads = pick(*[g for g in (1, 2, 3, 4, 6, 8) if heads % g == 0])
            dim = pick(8, 16, 24, 32, 40, 64, 128)
            layers.append(att(heads, kv_heads, dim, pick(8, 16, 24, 32, 48, 64), float(rng.uniform(0.5, 1.5)) / np.sqrt(dim), mlp,
                              base=pick(100.0, 1e4, 1e6), rot_dims=pick(dim, dim // 2, 2, 0), factor=pick(None, 2.0, 7.5)))
            continue
        src = pick(None, *latents) if latents else None
        if src is None:
            rot_dim, rank = pick(2, 4, 8, 16, 32), pick(16, 24, 32, 64, 128)
            base, scaling = pick(300.0, 1e4, 1e6), pick(None, (2.5, 384, 24.0, 1.0), (6.0, 40, 8.0, 0.5))
            latents[i] = (rot_dim, rank, base, scaling)
        else:
            rot_dim, rank, base, scaling = latents[src]
        dim = pick(8, 16, 24, 32, 64)
        layers.append(lat(pick(1, 2, 3, 4, 5, 16), dim, rot_dim, pick(8, 16, 24, 32, 64), rank, pick(8, 12, 48, 80),
                          float(rng.uniform(0.5, 1.5)) / np.sqrt(dim + rot_dim), mlp, base=base, scaling=scaling, kv_from=src))
    return config(pick(97, 128, 300, 512), width, layers, eps=pick(1e-6, 1e-5, 1e-3), embed_scale=pick(0.5, 1.0, 6.0),
                  softcap=pick(0.0, 10.0, 25.0))


@pytest.mark.parametrize("seed", range(24))
def test_configurations_drawn_from_seeds(tmp_path_factory, seed):
    cfg = drawn_configuration(seed)
    # (scores less spread than in the three models above: a drawn shape may have one head of few numbers, where a
    # spread of ten units makes near ties between keys that bfloat16 rounding decides)
    folder, plain = make_folder(tmp_path_factory, f"drawn{seed}", cfg, 500 + seed, qk_gain=5.0)
    rng = np.random.default_rng(seed)
    reqs = [[int(t) for t in rng.integers(0, cfg["vocab"], size=n)] for n in (150, 9, 71)]
    want = [P.forward(cfg, plain, r) for r in reqs]
    for dtype in DTYPES:
        eng = engine_for(folder, dtype, max_tokens=64 * 8)
        close(run_whole(eng, reqs[0]), want[0], dtype, f"seed {seed} whole")
        close(run_tail_one_by_one(eng, reqs[0], tail=40), want[0], dtype, f"seed {seed} tail one by one")
        for r, w, g in zip(reqs, want, run_batch(eng, reqs, [100, 3, 70])):
            close(g, w, dtype, f"seed {seed} batch, request of {len(r)}")
        assert eng.cache.held_pages() == 0 and not eng.cache.live_slots
        _ENGINES.clear()


# ---- mechanisms alone ---------------------------------------------------------------------------
def runtime(dtype, fast=True):
    from sonicboom_amd.parts import Runtime
    return Runtime(torch.device(DEV), TORCH_DT[dtype], fast)


def rand(*shape, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(1000 * seed + sum(shape) + len(shape))
    return torch.randn(tuple(shape), generator=g) * scale


def part_tensors(spec, dtype, seed=0, scale=0.3):
    dev, ref = {}, {}
    for i, t in enumerate(spec.all_tensors()):
        a = (rand(*t.shape, scale=scale, seed=seed + i) + t.init[0]).to(TORCH_DT[dtype])
        dev[t.name], ref[t.name] = a.to(DEV), a.float().numpy().astype(np.float64)
    return dev, ref


def part_close(got, want, dtype, what, bf16=2.5e-2):
    got, want = got.detach().float().cpu().numpy().astype(np.float64), np.asarray(want, dtype=np.float64)
    scale = max(float(np.abs(want).max()), 1e-30)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    err = np.abs(got - want).max() / scale
    assert err <= (2e-5 if dtype == "float32" else bf16), f"{what}: off by {err:.3g} of the largest value"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [96, 60, 35, 520, 4096, 5000])
@pytest.mark.parametrize("rows", [7, 300])
def test_two_norms_of_the_same_rows_in_one_pass(dtype, width, rows):
    from sonicboom_amd import ops
    x = rand(rows, width, scale=3.0)
    w1, w2 = (1.0 + rand(width, seed=1)).to(TORCH_DT[dtype]), (1.0 + rand(width, seed=2)).to(TORCH_DT[dtype])
    y1, y2 = ops.rmsnorm_pair(x.to(DEV), w1.to(DEV), w2.to(DEV), 2e-3, TORCH_DT[dtype])
    part_close(y1, P.norm(x.numpy(), w1.float().numpy(), 2e-3), dtype, "first norm", bf16=5e-3)
    part_close(y2, P.norm(x.numpy(), w2.float().numpy(), 2e-3), dtype, "second norm", bf16=5e-3)
    assert torch.equal(y1, ops.rmsnorm(x.to(DEV), w1.to(DEV), 2e-3, TORCH_DT[dtype])), "the bits of the norm alone"
    # a part of wider rows, normed where it lies
    wide = rand(rows, width + 24, scale=2.0, seed=3).to(DEV)
    part, none = ops.rmsnorm_pair(wide[:, 8:8 + width], w1.to(DEV), None, 1e-5, TORCH_DT[dtype], second=False)
    assert none is None
    part_close(part, P.norm(wide[:, 8:8 + width].cpu().numpy(), w1.float().numpy(), 1e-5), dtype, "a part of wider rows", bf16=5e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_sigmoid_gate_and_the_cap_on_logits(dtype):
    from sonicboom_amd import ops
    a, g = rand(37, 50, scale=2.0).to(TORCH_DT[dtype]), rand(37, 70, scale=3.0, seed=1)
    got = ops.sigmoid_mul_(a.to(DEV).clone(), g.to(DEV)[:, 11:61])
    part_close(got, a.float().numpy() * P.sigmoid(g.numpy()[:, 11:61]), dtype, "gate", bf16=5e-3)
    z = rand(9, 333, scale=20.0, seed=2)
    part_close(ops.softcap_(z.to(DEV).clone(), 7.5), 7.5 * np.tanh(z.numpy().astype(np.float64) / 7.5), "float32", "cap")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [3, 70, 300])
@pytest.mark.parametrize("width, inner", [(72, 200), (60, 52)])
def test_dense_feed_forward_with_biases(dtype, rows, width, inner):
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.ffn import dense_ffn_spec
    spec = dense_ffn_spec("m.up", "m.down", width, inner, "gelu_erf", up_bias_name="m.up.b", down_bias_name="m.down.b")
    dev, ref = part_tensors(spec, dtype)
    ffn = build_part(spec, dev, runtime(dtype))
    h = rand(rows, width, scale=2.0).to(TORCH_DT[dtype])
    x = torch.zeros(rows, width, dtype=F32, device=DEV)
    ffn.forward(h.to(DEV), x, None)
    want = P.dense_ff(ref, "m.", h.float().numpy())
    part_close(x, want, dtype, "feed-forward")
    tanh_form = 0.5 * (z := P.linear(h.float().numpy(), ref["m.up"], ref["m.up.b"])) * (1 + np.tanh(np.sqrt(2 / np.pi) * (z + 0.044715 * z ** 3)))
    assert np.abs(P.linear(tanh_form, ref["m.down"], ref["m.down.b"]) - want).max() > 3e-5 * np.abs(want).max(), \
        "the two forms of the gelu differ by more than the 32-bit bound"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 3, 70, 300])
@pytest.mark.parametrize("experts, top, inner, shared, groups", [
    (4, 1, 48, 0, None), (6, 3, 32, 64, (3, 2)), (3, 3, 20, 36, None), (9, 2, 136, 16, (3, 1)), (8, 3, 56, 80, (4, 2))])
def test_routed_experts_alone(dtype, rows, experts, top, inner, shared, groups):
    """The router's scores over all experts, the choice within the best groups, the experts' products (grouped by
    expert on the matrix cores in bfloat16 when the sizes allow, else a thread an output), the shared expert and
    its gate, and the pass that adds them up."""
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.moe import moe_ffn_spec
    width = 72 if inner % 8 else 64
    g = groups or (1, 1)
    spec = moe_ffn_spec("m.", width, experts, top, inner, 0.0, shared_inner=shared, activation="relu_sq",
                        router_score="softmax_all", groups=g[0], keep_groups=g[1])
    dev, ref = part_tensors(spec, dtype, scale=0.4)
    assert "m.e0.gate" not in dev and ("m.shared.gate" not in dev)
    # routers apart by construction: the first `experts` input numbers decide, in levels
    gen = torch.Generator().manual_seed(rows + experts)
    h = rand(rows, width, scale=1.0, seed=rows)
    h[:, :experts] = torch.stack([torch.randperm(experts, generator=gen).float() for _ in range(rows)])
    router = torch.zeros(experts, width)
    router[:, :experts] = torch.eye(experts) * 0.75
    dev["m.router"], ref["m.router"] = router.to(TORCH_DT[dtype]).to(DEV), router.numpy().astype(np.float64)
    ffn = build_part(spec, dev, runtime(dtype))
    h = h.to(TORCH_DT[dtype])
    cfg = moe(experts, top, inner, groups=groups, shared=shared or None)
    want = P.moe_ff(cfg, ref, "m.", h.float().numpy())
    x = torch.zeros(rows, width, dtype=F32, device=DEV)
    ffn.forward(h.to(DEV), x, None)
    part_close(x, want, dtype, "routed experts")
    if groups and rows >= 70:
        free = P.moe_ff(moe(experts, top, inner, shared=shared or None), ref, "m.", h.float().numpy())
        assert np.abs(free - want).max() > 0.05 * np.abs(want).max(), "the groups do not show: the test shows nothing"


def test_the_router_kernel_orders_like_the_plain_one():
    from sonicboom_amd import ops
    z = rand(500, 12, seed=3)
    z[5, 2] = z[5, 7]                       # a tie goes to the lower number
    z[6] = 0.0
    gate = rand(500, 1, seed=4)
    zd = torch.cat([z, gate], dim=1).contiguous().to(DEV)
    for top, groups, keep in [(1, 1, 1), (2, 3, 2), (5, 2, 1), (12, 1, 1), (4, 4, 2), (3, 12, 3), (6, 6, 6)]:
        ids, w = ops.moe_route(zd, 12, top, True, score="softmax_all", groups=groups, keep_groups=keep)
        chosen, weight = P.route(z.numpy().astype(np.float64), top, groups, keep)
        assert np.array_equal(ids.cpu().numpy(), chosen), (top, groups, keep)
        assert np.allclose(w[:, :top].cpu().numpy(), weight, atol=1e-6)
        assert np.allclose(w[:, top].cpu().numpy(), P.sigmoid(gate.numpy()[:, 0]), atol=1e-6)


def mixer_harness(mixer, rt, width, n_tokens_cap=64 * 20, reader=None):
    """A cache for one mixer alone, and a function that feeds rows of one sequence in cuts and returns what the
    mixer adds into an empty stream.  ``reader``: a second mixer that reads the rows the first one stores; the
    function then returns its result."""
    from sonicboom_amd.cache import PagedCache, group_entries
    from sonicboom_amd.engine.model import LayerBinding
    from sonicboom_amd.engine.step import StepContext, StepEntry
    cs = mixer.cache_spec()
    cache = PagedCache(group_entries({0: cs.key()}), n_tokens_cap, rt.cache_dtype, rt.device, None, max_slots=4)
    tiles = set()
    for m in (mixer, reader):
        t = getattr(m, "row_tile", None) or ()
        tiles.update((t,) if isinstance(t, int) else tuple(t))

    def feed(h_rows, cuts, reader_rows=None):
        k, v, g = cache.entry_views(0)
        slot = cache.alloc_slot()
        outs, at = [], 0
        try:
            for n in cuts:
                cache.reserve([slot], [n])
                ctx = StepContext(cache, [StepEntry(slot, [0] * n, ())], rt.device, tuple(sorted(tiles)))
                ctx.shared = {}
                x = torch.zeros(n, width, dtype=F32, device=DEV)
                mixer.forward(h_rows[at:at + n].to(DEV).contiguous(), x, ctx, LayerBinding(0, g, k, v, True, None))
                if reader is not None:
                    x = torch.zeros(n, width, dtype=F32, device=DEV)
                    reader.forward(reader_rows[at:at + n].to(DEV).contiguous(), x, ctx, LayerBinding(1, g, k, v, False, None))
                outs.append(x)
                cache.advance([slot], [n])
                at += n
        finally:
            cache.free_slot(slot)
        return torch.cat(outs)
    return feed


def attention_mixer(dtype, heads, kv_heads, dim, vdim, scale, rot_dims=None, base=1e4, factor=None, width=64, seed=0, fast=True):
    from sonicboom_amd.architectures.fitatar import ATTENTION_NAMES
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.attention import attention_spec
    from sonicboom_amd.parts.position import rope_spec, stretched_frequencies
    layer = att(heads, kv_heads, dim, vdim, scale, None, base=base, rot_dims=rot_dims, factor=factor)
    mx = layer["mixer"]
    freq, mag = stretched_frequencies(mx["rot"]["dims"], base, "linear" if factor else None, factor or 1.0)
    spec = attention_spec("a.", width, heads, kv_heads, dim, rope_spec(dim, base, rot_dims=mx["rot"]["dims"], frequencies=freq, magnitude=mag),
                          scale=scale, qkv_bias=False, v_dim=vdim, sink=True, sink_scores=True, out_gate=True, names=ATTENTION_NAMES)
    dev, ref = part_tensors(spec, dtype, seed=seed, scale=0.5)
    rt = runtime(dtype, fast)
    return build_part(spec, dev, rt), rt, ref, mx, spec


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, rot_dims, factor", [
    (4, 2, 32, 16, 16, 8.0), (3, 3, 10, 14, 6, None), (5, 1, 16, 64, None, 3.0), (2, 1, 24, 6, 2, 2.0), (8, 1, 64, 48, 32, 40.0),
    (1, 1, 128, 128, None, None)])
def test_attention_alone(dtype, heads, kv_heads, dim, vdim, rot_dims, factor):
    """Rotation of a part of the head, the sink's own scores, values of their own size, the gate: whole, in
    portions and token by token."""
    # (queries and keys of these weights have numbers of about 4: scores of about 3)
    mixer, rt, ref, mx, _ = attention_mixer(dtype, heads, kv_heads, dim, vdim, 3.0 / (16.0 * np.sqrt(dim)), rot_dims, factor=factor)
    feed = mixer_harness(mixer, rt, 64)
    n = 200
    h = rand(n, 64).to(TORCH_DT[dtype])
    want, _ = P.attention(mx, ref, "a.", h.float().numpy())
    for cuts in ([n], [70, 2, 60] + [1] * 68):
        part_close(feed(h, cuts), want, dtype, f"attention cuts {cuts[:3]}")
    # positions count: the same rows without the rotation give another result
    still, _ = P.attention(dict(mx, rot=dict(mx["rot"], dims=0)), ref, "a.", h.float().numpy())
    assert np.abs(still - want).max() > 0.02 * np.abs(want).max()


def latent_mixer(dtype, heads, dim, rot_dim, vdim, rank, q_rank, scale, scaling, base=1e4, width=64, seed=0, fast=True, own=True):
    from sonicboom_amd.parts import PartSpec, build_part
    from sonicboom_amd.parts.latent_attention import latent_attention_spec
    from sonicboom_amd.parts.position import rope_interleaved_spec, stretched_frequencies
    mx = lat(heads, dim, rot_dim, vdim, rank, q_rank, scale, None, base=base, scaling=scaling)["mixer"]
    position = PartSpec("position", "none")
    if rot_dim:
        freq, mag = stretched_frequencies(rot_dim, base, "ramp" if scaling else None, *(scaling or ()))
        position = rope_interleaved_spec(rot_dim, base, frequencies=freq, magnitude=mag)
    spec = latent_attention_spec("a.", width, heads, dim, rot_dim, vdim, rank, scale, position, eps=1e-5, own_latent=own,
                                 q_rank=q_rank, gate_per_head=True)
    dev, ref = part_tensors(spec, dtype, seed=seed, scale=0.5)
    rt = runtime(dtype, fast)
    return build_part(spec, dev, rt), rt, ref, mx


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, rot_dim, vdim, rank, q_rank, scaling", [
    (4, 32, 16, 48, 64, 40, (4.0, 64, 16.0, 1.0)), (1, 10, 6, 14, 20, 9, None), (3, 24, 16, 8, 48, 16, (1.5, 32, 4.0, 2.0)),
    (16, 16, 8, 16, 32, 24, (16.0, 128, 32.0, 1.0)), (2, 48, 32, 80, 96, 56, (3.0, 256, 16.0, 1.0))])
def test_latent_attention_alone(dtype, heads, dim, rot_dim, vdim, rank, q_rank, scaling):
    """Queries through their own normed latent, the cached latent row with the shared rotated part, stretched
    frequencies with their magnitude, a gate a head: whole, in portions and token by token; and a second mixer
    that reads the rows of the first."""
    scale = 3.0 / (0.3 * np.sqrt(q_rank * rank * (dim + rot_dim)))       # scores of about 3 with these weights
    mixer, rt, ref, mx = latent_mixer(dtype, heads, dim, rot_dim, vdim, rank, q_rank, scale, scaling)
    feed = mixer_harness(mixer, rt, 64)
    n = 200
    h = rand(n, 64).to(TORCH_DT[dtype])
    hn = h.float().numpy()
    kept = P.latent_rows(mx, 1e-5, ref, "a.", hn, np.arange(n))
    want = P.latent_attention(mx, 1e-5, ref, "a.", hn, kept)
    for cuts in ([n], [70, 2, 60] + [1] * 68):
        part_close(feed(h, cuts), want, dtype, f"latent attention cuts {cuts[:3]}")
    if scaling:
        flat = P.latent_attention(dict(mx, rot={"base": mx["rot"]["base"], "dims": rot_dim}), 1e-5, ref, "a.", hn,
                                  P.latent_rows(dict(mx, rot={"base": mx["rot"]["base"], "dims": rot_dim}), 1e-5, ref, "a.", hn, np.arange(n)))
        assert np.abs(flat - want).max() > 1e-3 * np.abs(want).max(), "the stretched frequencies do not show"
    # a reader with other heads and sizes of its own
    reader, _, ref2, mx2 = latent_mixer(dtype, heads + 1, dim // 2, rot_dim, vdim + 8, rank, q_rank + 3, scale, scaling, seed=50, own=False)
    h2 = rand(n, 64, seed=9).to(TORCH_DT[dtype])
    both = mixer_harness(mixer, rt, 64, reader=reader)
    want2 = P.latent_attention(mx2, 1e-5, ref2, "a.", h2.float().numpy(), kept)
    for cuts in ([n], [130, 3] + [1] * 67):
        part_close(both(h, cuts, reader_rows=h2), want2, dtype, f"a reader of the rows, cuts {cuts[:2]}")


@pytest.mark.parametrize("heads, kv_heads, dim, vdim", [(4, 1, 32, 16), (6, 2, 64, 64), (16, 2, 128, 64), (5, 5, 16, 48)])
def test_matrix_core_attention_equals_the_plain_kernel(heads, kv_heads, dim, vdim):
    """bfloat16: a prompt, portions and single rows over several pages (the pages of a step of few rows are shared
    out over blocks and merged, the sink counted once) against the kernel of one wave per (row, head)."""
    n = 700
    h = rand(n, 64).to(BF16)
    outs = {}
    for fast in (True, False):
        mixer, rt, ref, mx, _ = attention_mixer("bfloat16", heads, kv_heads, dim, vdim, 3.0 / (16.0 * np.sqrt(dim)), dim // 2, factor=4.0, fast=fast)
        feed = mixer_harness(mixer, rt, 64)
        outs[fast] = [feed(h, cuts) for cuts in ([n], [560, 17, 3] + [1] * 120)]
    want, _ = P.attention(mx, ref, "a.", h.float().numpy())
    for a, b in zip(outs[True], outs[False]):
        part_close(a, b.float().cpu().numpy(), "bfloat16", "matrix cores against the plain kernel", bf16=1.5e-2)
        part_close(a, want, "bfloat16", "matrix cores against the plain implementation")


def planted_attention(dtype, dim=16, vdim=16, width=48, gain=14.0, fast=True):
    """An attention mixer whose weights are set by hand: keys read the input's numbers 0..dim-1, queries the numbers
    behind them (both heads alike); nothing rotates in the numbers that carry the signal (the head rotates its
    last numbers only: the first rot.dims are left empty).  A row whose input has number dim+8 set asks for keys
    whose input has number 8 set: the score of that pair is large, every other score is nothing.  The sinks score
    a little above nothing, so a query that nobody answers leaves most of its weight there."""
    mixer, rt, ref, mx, spec = attention_mixer(dtype, 2, 1, dim, vdim, gain / 9.0, rot_dims=8, factor=2.0, width=width, fast=fast)
    t = {k: torch.zeros(v.shape) for k, v in ref.items()}
    for d in range(8, dim):
        t["a.k"][d, d] = 1.0
        for a in range(2):
            t["a.q"][a * dim + d, dim + d] = 1.0
    t["a.v"], t["a.o"] = rand(vdim, width, seed=1), rand(width, 2 * vdim, scale=0.3, seed=3)
    t["a.g"] = rand(2 * vdim, width, scale=0.05, seed=5)
    t["a.sink"] = torch.tensor([4.0, 6.5])
    from sonicboom_amd.parts import build_part
    dev = {k: v.to(TORCH_DT[dtype]).to(DEV) for k, v in t.items()}
    ref = {k: v.to(TORCH_DT[dtype]).float().numpy().astype(np.float64) for k, v in t.items()}
    return build_part(spec, dev, rt), rt, ref, mx, width


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("fast", [True, False])
def test_one_key_stands_out_and_the_sink_takes_its_weight(dtype, fast):
    """A prompt of 700 rows in which the last row asks and one row answers: the query's weight falls on that key
    however far back it lies: the row before, at both sides of page borders, hundreds of rows away, the very
    first row.  The query runs as the last row of a prompt, as a single decoded row, and behind a portion of two
    rows.  With no key that answers, most of the weight goes to the sink and the result is small: leaving the sink
    out, or taking its score for 0, would show."""
    if fast and dtype == "float32":
        pytest.skip("the 32-bit path has one attention kernel")
    dim = 16
    mixer, rt, ref, mx, width = planted_attention(dtype, dim=dim, fast=fast)
    feed = mixer_harness(mixer, rt, width)
    n = 700
    t = n - 1
    shows = 0
    for b in [1, 2, 63, 64, 65, 127, 128, 129, 500, 636, 699]:
        j = t - b
        h = rand(n, width, seed=b) * 0.05
        h[:, :2 * dim] = 0.0                # no key answers and no row asks,
        h[j, 8], h[t, dim + 8] = 3.0, 3.0   # but for these two
        h = h.to(TORCH_DT[dtype])
        hn = h.float().numpy()
        want, _ = P.attention(mx, ref, "a.", hn)
        for cuts in ([n], [n - 1, 1], [300, 336, 61, 2, 1]):
            part_close(feed(h, cuts)[t:], want[t:], dtype, f"key {b} back, cuts {cuts}")
        hidden = hn.copy()
        hidden[j, 8] = 0.0
        other, _ = P.attention(mx, ref, "a.", hidden)
        if np.abs(other[t] - want[t]).max() > 0.3 * np.abs(want[t]).max():
            shows += 1
    assert shows >= 10, "the planted key does not decide the result: the test shows nothing"
    # nobody answers: the sinks hold most of the weight (e^4 and e^6.5 against 700 keys of weight 1)
    h = rand(n, width, seed=99) * 0.05
    h[:, :2 * dim] = 0.0
    h = h.to(TORCH_DT[dtype])
    hn = h.float().numpy()
    want, _ = P.attention(mx, ref, "a.", hn)
    for cuts in ([n], [n - 1, 1]):
        part_close(feed(h, cuts)[t:], want[t:], dtype, "no key answers")
    for sinks in ([-50.0, -50.0], [0.0, 0.0], [6.5, 4.0]):
        other, _ = P.attention(mx, dict(ref, **{"a.sink": np.array(sinks)}), "a.", hn)
        assert np.abs(other[t] - want[t]).max() > 0.2 * np.abs(want[t]).max(), f"sinks of {sinks} would not show"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("fast", [True, False])
@pytest.mark.parametrize("through", ["latent", "rotated"])
def test_one_latent_row_stands_out(dtype, fast, through):
    """The same for latent attention, through the part of the key that comes out of the latent, or through the
    rotated part that the heads share (in its slowest pair, whose stretched frequency turns it by a sixth of a
    radian over 699 positions): the asking row's query latent points at one direction, one cached row holds it."""
    if fast and dtype == "float32":
        pytest.skip("the 32-bit path has one attention kernel")
    heads, dim, rot_dim, vdim, rank, q_rank, width = 2, 16, 8, 16, 32, 16, 64
    mixer, rt, ref, mx = latent_mixer(dtype, heads, dim, rot_dim, vdim, rank, q_rank, 1.0, (4.0, 64, 16.0, 1.0), width=width, fast=fast)
    t = {k: torch.zeros(v.shape) for k, v in ref.items()}
    # the latent c reads input numbers 0..rank-1 (its norm makes a row with one number set a unit row times
    # sqrt(rank)); the plain key of both heads is the latent's first dim numbers; queries' latent reads the input
    # numbers behind, and the plain query is the query latent's first dim numbers.  The rotated parts are empty.
    for i in range(rank):
        t["a.dkv"][i, i] = 1.0
    for i in range(q_rank):
        t["a.dq"][i, rank + i] = 1.0
    for a in range(heads):
        for d in range(dim):
            t["a.uk"][a * dim + d, d] = 1.0
            t["a.uq"][a * (dim + rot_dim) + d, d] = 1.0
    if through == "rotated":
        # number 3 of the input goes into the rotated key part's last pair instead of the latent, and number 3 of the
        # query latent into the rotated query part's
        t["a.dkv"][3, 3] = 0.0
        t["a.dkv"][rank + 6, 3] = 1.0
        for a in range(heads):
            t["a.uq"][a * (dim + rot_dim) + 3, 3] = 0.0
            t["a.uq"][a * (dim + rot_dim) + dim + 6, 3] = 1.0
    t["a.dkv.norm"][:], t["a.dq.norm"][:] = 1.0, 1.0
    t["a.uv"], t["a.o"] = rand(heads * vdim, rank, seed=1), rand(width, heads * vdim, scale=0.3, seed=3)
    t["a.g"] = rand(heads, width, scale=0.05, seed=5)
    from sonicboom_amd.parts import build_part
    dev = {k: v.to(TORCH_DT[dtype]).to(DEV) for k, v in t.items()}
    ref = {k: v.to(TORCH_DT[dtype]).float().numpy().astype(np.float64) for k, v in t.items()}
    mixer = build_part(mixer.spec, dev, rt)
    feed = mixer_harness(mixer, rt, width)
    n = 700
    last = n - 1
    shows = 0
    for b in [1, 2, 63, 64, 65, 127, 128, 129, 500, 636, 699]:
        j = last - b
        h = torch.zeros(n, width)
        h[:, 20:rank] = rand(n, rank - 20, seed=b).abs() + 0.5      # every row's latent lies in numbers that no query reads
        h[:, rank + 10] = 1.0                                        # every query's latent points at number 10, where no key has anything
        h[j, 3] = 6.0                                                # one row's latent has number 3 set
        h[last, rank + 3], h[last, rank + 10] = 1.0, 0.0             # and the last row asks for it
        h = h.to(TORCH_DT[dtype])
        hn = h.float().numpy()
        want = P.latent_attention(mx, 1e-5, ref, "a.", hn, P.latent_rows(mx, 1e-5, ref, "a.", hn, np.arange(n)))
        for cuts in ([n], [n - 1, 1], [300, 336, 61, 2, 1]):
            part_close(feed(h, cuts)[last:], want[last:], dtype, f"latent row {b} back, cuts {cuts}")
        hidden = hn.copy()
        hidden[j, 3] = 0.0
        other = P.latent_attention(mx, 1e-5, ref, "a.", hidden, P.latent_rows(mx, 1e-5, ref, "a.", hidden, np.arange(n)))
        if np.abs(other[last] - want[last]).max() > 0.3 * np.abs(want[last]).max():
            shows += 1
    assert shows >= 10, "the planted row does not decide the result: the test shows nothing"
