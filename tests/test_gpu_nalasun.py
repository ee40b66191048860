"""The Nalasun design on the GPU against the plain implementation of tests/plain/nalasun_plain.py:
every mechanism alone, whole models of several shapes, prompts cut into portions down to two tokens,
token-by-token decoding, batches of unequal requests on a cache and slots that are used again, a key
planted far away and at both sides of page borders, states that must survive hundreds of steps, long
decoding through the recorded decode step, and greedy generation through the Python entry point, the
command line and the replay program."""
import json
import os

import numpy as np
import pytest
import torch

import helpers
from helpers import run_batch, run_tail_one_by_one, run_whole
from plain import nalasun_plain as N
from test_nalasun_config import att, config, delta, moe, ssm

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16
DTYPES = ["float32", "bfloat16"]
TORCH_DT = {"float32": F32, "bfloat16": BF16}
CODES = 8          # channels at the end of the stream that carry a code of the token for the routers

# P: sizes in sixteens (the matrix-core products and attention in bfloat16); attention first, a layer without a
#    feed-forward, groups of the state space equal to 2 and to its heads, the delta rule with fewer query/key heads
#    than value heads, one expert a row and three a row, with and without the shared expert.
# Q: sizes that are no multiple of 8 or 16 (plain products), a recurrence first, one group, one norm group, two taps,
#    as many chosen experts as there are, ranks that 8 does not divide, no temperature in one layer.
# R: the delta rule first and alone with one head, five taps, a temperature whose period is 1.
CONFIGS = {
    "P": config(160, 96, 400, 4, [
        att(6, 2, 32, 0.35, 0.6, 50, moe(4, 1, 48, 1.25)),
        ssm(4, 32, 16, 2, 4, 2, moe(6, 3, 32, 0.8, shared=64)),
        delta(4, 2, 16, 32, 3, None, ranks=(8, 16)),
        att(4, 4, 16, 0.5, 0.3, 7, moe(5, 2, 16, 2.0, shared=16)),
        ssm(2, 48, 32, 2, 2, 4, None),
    ], eps=3e-4),
    "Q": config(131, 60, 350, 2, [
        ssm(3, 20, 24, 1, 3, 1, moe(3, 3, 20, 1.0, shared=36)),
        att(3, 3, 10, 0.6, 0.0, 1, moe(7, 4, 12, 0.5)),
        delta(3, 1, 12, 20, 2, moe(2, 1, 28, 1.7), ranks=(5, 7)),
        att(5, 1, 6, 0.9, 1.1, 13, None),
    ], eps=1e-6),
    "R": config(200, 64, 600, 5, [
        delta(1, 1, 64, 48, 5, moe(8, 2, 24, 1.5, shared=40), ranks=(24, 8)),
        att(2, 1, 48, 0.3, 0.5, 1, moe(2, 2, 56, 0.6)),
        ssm(8, 8, 40, 8, 4, 1, moe(4, 2, 32, 1.0)),
    ], eps=1e-5),
}
SEEDS = {"P": 31, "Q": 32, "R": 33}
_FOLDERS, _PLAIN, _ENGINES, _WANT = {}, {}, {}, {}


def coded_routers(cfg, w):
    """Routers whose choice does not hang on a close call.  The plain implementation sums in float64 and the
    bfloat16 path rounds what the router reads: two scores a hair apart would be ordered differently by the two.
    So the last CODES channels of the stream carry a code of the token (one of them 2, the others 0) that no
    sublayer writes to (the rows of every output matrix are zero there), and the routers read those channels
    alone, with levels half a unit apart around zero, so that every score stays inside the sigmoid's bend."""
    d = cfg["width"]
    r = slice(d - CODES, d)
    code = np.zeros((cfg["vocab"], CODES))
    code[np.arange(cfg["vocab"]), np.arange(cfg["vocab"]) % CODES] = 2.0
    w["embed"][:, r] = code
    w["pos"][:, r] = 0.0
    for name in w:
        if name.endswith((".mix.o", ".down")):
            w[name][r, :] = 0.0
    for i, layer in enumerate(cfg["layers"]):
        f = layer["mlp"]
        if f is None:
            continue
        w[f"l{i}.norm2"][r] = 1.0
        e = f["router"]["experts"]
        levels = ((np.arange(e)[:, None] - np.arange(CODES)[None, :] + i) % e).astype(np.float64) - (e - 1) / 2.0
        router = np.zeros((e, d))
        router[:, r] = levels * 0.5
        w[f"l{i}.mlp.router"] = router
    return w


def sharpen(cfg, w, coded=True):
    """Random N(0, 0.02) weights give almost uniform attention, gates near one half and states that hardly move.
    Scale the projections so that scores spread over several units, the recurrences' decays and step sizes differ
    between tokens and the experts' gates bend."""
    out = {}
    for name, a in w.items():
        a = np.array(a, dtype=np.float64)
        if name.endswith((".mix.q", ".mix.k", ".mix.v", ".mix.b")):
            a = a * 10.0
        elif name.endswith(".mix.in"):
            a = a * 4.0           # (x, B and C multiply each other: a larger factor makes the layer amplify rounding)
        elif name.endswith((".a1", ".a2", ".g1", ".g2")):
            a = a * 5.0
        elif name.endswith(".mix.o"):
            a = a * 3.0
        elif name.endswith((".q.b", ".k.b")):
            a = a * 10.0
        elif name.endswith((".gate", ".up", ".down")):
            a = a * 4.0
        elif name.endswith((".r1", ".r2")):
            a = np.abs(a)
        elif name in ("embed", "pos"):
            a = a * 30.0
        elif name.endswith(".router"):
            a = a * 3.0           # (sigmoid scores: larger and float32 no longer tells the largest apart)
        out[name] = a
    return coded_routers(cfg, out) if coded else out


def make_folder(tmp_path_factory, name, cfg, seed, coded=True):
    from safetensors.torch import load_file, save_file
    from sonicboom_amd.weights import write_random_model
    folder = str(tmp_path_factory.mktemp(f"nalasun_{name}"))
    write_random_model(folder, json.loads(json.dumps(cfg)), seed=seed, dtype="bfloat16", device=None)
    path = os.path.join(folder, "model.safetensors")
    w = sharpen(cfg, {k: v.float().numpy() for k, v in load_file(path).items()}, coded)
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
        _WANT[key] = N.forward(CONFIGS[name], _PLAIN[name], list(tokens))
    return _WANT[key]


def prompts(name, lengths, seed=0):
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, CONFIGS[name]["vocab"], size=n)] for n in lengths]


# Bounds.  float32 differs from the plain implementation (float64) by the rounding of float32 sums.
# bfloat16 is measured in spreads of the logits (their standard deviation): the largest difference
# and the root mean square of all differences of a request.
F32_BOUND = 3e-4
BF16_WORST, BF16_RMS = 0.072, 0.011      # what the whole file measured (0.0512 and 0.0078) times 1.4
helpers.BF16_MAX["recurrences and shared attention"], helpers.BF16_RMS["recurrences and shared attention"] = BF16_WORST, BF16_RMS


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
        seen = helpers.BF16_SEEN.setdefault("recurrences and shared attention", [0.0, 0.0])
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
        x = N.start(cfg, _PLAIN[name], tokens)
        for i, layer in enumerate(cfg["layers"]):
            f = layer["mlp"]
            p = f"l{i}."
            h = N.rms_norm(x, _PLAIN[name][p + "norm1"], cfg["norm"]["eps"])
            h = h + N.time_conv(h, _PLAIN[name][p + "canon1"])
            x = x + N.MIXERS[layer["type"]](layer["mixer"], cfg["norm"]["eps"], _PLAIN[name], p + "mix.", h)
            if f is None:
                continue
            fx = N.rms_norm(x, _PLAIN[name][p + "norm2"], cfg["norm"]["eps"])
            s = np.sort(N.sigmoid(N.linear(fx, _PLAIN[name][p + "mlp.router"])), axis=1)[:, ::-1]
            top = f["router"]["top"]
            if top < s.shape[1]:
                assert (s[:, top - 1] - s[:, top]).min() > 0.01, (name, i)
            assert (s[:, :-1] - s[:, 1:]).min() > 1e-4, "scores that float32 tells apart"
            chosen, _ = N.route(N.linear(fx, _PLAIN[name][p + "mlp.router"]), top, 1.0)
            assert len(np.unique(chosen)) == f["router"]["experts"], "every expert is chosen by some token"
            x = x + N.feed_forward(f, _PLAIN[name], p + "mlp.", fx)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_requests_and_the_first_tokens(folders, name, dtype):
    eng = engine_for(folders[name], dtype)
    for tokens in prompts(name, [1, 2, 3, 4, 17, 63, 64, 65, 200]):
        close(run_whole(eng, tokens), want_logits(name, tokens), dtype, f"{name} whole n={len(tokens)}")
    assert eng.cache.held_pages() == 0 and not eng.cache.live_slots


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_random_routers_in_32_bit(tmp_path_factory, name):
    """The same models with routers of plain random weights (scores as close as chance makes them)."""
    folder, plain = make_folder(tmp_path_factory, name + "_random", CONFIGS[name], SEEDS[name] + 100, coded=False)
    eng = engine_for(folder, "float32")
    for tokens in prompts(name, [90, 5], seed=4):
        close(run_whole(eng, tokens), N.forward(CONFIGS[name], plain, tokens), "float32", f"{name} random routers")


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
    """Portions of two tokens are shorter than every convolution's reach: their inputs come from the state
    that two steps before them left."""
    eng = engine_for(folders[name], dtype)
    tokens = prompts(name, [331], seed=2)[0]
    whole = run_whole(eng, tokens)
    for cuts in ([2] * 20 + [291], [64, 64, 64, 139], [63, 2, 65, 1, 127, 3, 70], [130, 2, 2, 129, 68], [1, 330],
                 [1, 1, 2, 1, 3, 323]):
        got = run_cuts(eng, tokens, cuts)
        close(got, want_logits(name, tokens), dtype, f"{name} cuts {cuts[:4]}")
        if dtype == "float32":
            assert np.array_equal(got, whole), f"cuts {cuts[:4]} change bits"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_unequal_batches_on_a_cache_that_is_used_again(folders, name, dtype):
    """Nine pages and five slots: every batch fills eight pages, the next gets used pages and slots, whose
    states must start from zero again."""
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
    eng = engine_for(folders["P"], dtype, max_tokens=64 * 12, max_step_rows=100)
    reqs = prompts("P", [130, 7, 220], seed=5)
    got = run_batch(eng, reqs, [130, 7, 220])
    for r, g in zip(reqs, got):
        close(g, want_logits("P", r), dtype, f"portions, request of {len(r)}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q"])
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
    for name in ("P", "Q"):
        ps = prompts(name, [4, 70, 19], seed=9)
        session = Model.load(folders[name], dtype="float32").session(max_tokens=64 * 8)
        got = session.generate(ps, max_tokens=12, stop_tokens=())
        assert got == [N.greedy(CONFIGS[name], _PLAIN[name], p, 12) for p in ps]
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
    name = "Q"
    ps = prompts(name, [4, 10], seed=9)
    tokens = tmp_path / "prompts.txt"
    tokens.write_text("\n".join(" ".join(map(str, p)) for p in ps) + "\n")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "sb-gen"), "-m", folders[name], "--tokens", str(tokens), "-n", "6",
           "--dtype", "fp32", "--stop", ""]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    got = [[int(t) for t in line.split()] for line in out.stdout.strip().splitlines()]
    assert got == [N.greedy(CONFIGS[name], _PLAIN[name], p, 6) for p in ps]
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


def part_close(got, want, dtype, what, bf16=2.5e-2, f32=2e-5):
    got, want = got.detach().float().cpu().numpy().astype(np.float64), np.asarray(want, dtype=np.float64)
    scale = max(float(np.abs(want).max()), 1e-30)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: not finite"
    err = np.abs(got - want).max() / scale
    assert err <= (f32 if dtype == "float32" else bf16), f"{what}: off by {err:.3g} of the largest value"


class Harness:
    """A cache and per-sequence states for one part alone, and ``feed``: rows of sequences in cuts through
    ``fn(h, x, ctx, binding)``, which adds into the float32 rows ``x`` that come back."""

    def __init__(self, rt, cache_spec=None, states=None, width=64, pages=24, max_slots=4, tiles=()):
        from sonicboom_amd.cache import PagedCache, group_entries
        self.rt, self.width = rt, width
        groups = group_entries({0: cache_spec.key()}) if cache_spec is not None else []
        shapes = {(0, name): (tuple(s.shape), s.dtype) for name, s in (states or {}).items()}
        self.cache = PagedCache(groups, 64 * pages, rt.cache_dtype, rt.device, shapes, max_slots=max_slots)
        self.has_cache = cache_spec is not None
        self.tiles = (tiles,) if isinstance(tiles, int) else tuple(tiles or ())

    def binding(self):
        from sonicboom_amd.engine.model import LayerBinding
        k = v = g = None
        if self.has_cache:
            k, v, g = self.cache.entry_views(0)
        named = {key[1]: t for key, t in self.cache.state.items()}
        return LayerBinding(0, g, k, v, self.has_cache, None, named)

    def feed(self, fn, h_rows, cuts, slot=None):
        """``h_rows`` [n, *]: one sequence's rows, fed in portions of ``cuts``."""
        from sonicboom_amd.engine.step import StepContext, StepEntry
        own = slot is None
        slot = self.cache.alloc_slot() if own else slot
        outs, at = [], 0
        try:
            for n in cuts:
                self.cache.reserve([slot], [n])
                ctx = StepContext(self.cache, [StepEntry(slot, [0] * n, ())], self.rt.device, self.tiles)
                ctx.shared = {}
                x = torch.zeros((n, self.width), dtype=F32, device=DEV)
                fn(h_rows[at:at + n].to(DEV).contiguous(), x, ctx, self.binding())
                outs.append(x)
                self.cache.advance([slot], [n])
                at += n
        finally:
            if own:
                self.cache.free_slot(slot)
        return torch.cat(outs)

    def feed_batch(self, fn, seqs):
        """Several sequences' rows in one step each; returns the rows sequence by sequence."""
        from sonicboom_amd.engine.step import StepContext, StepEntry
        slots = [self.cache.alloc_slot() for _ in seqs]
        try:
            lens = [s.shape[0] for s in seqs]
            self.cache.reserve(slots, lens)
            ctx = StepContext(self.cache, [StepEntry(s, [0] * n, ()) for s, n in zip(slots, lens)], self.rt.device, self.tiles)
            ctx.shared = {}
            x = torch.zeros((sum(lens), self.width), dtype=F32, device=DEV)
            fn(torch.cat(seqs).to(DEV).contiguous(), x, ctx, self.binding())
            self.cache.advance(slots, lens)
            return list(torch.split(x, lens))
        finally:
            for s in slots:
                self.cache.free_slot(s)


CUTS = ([150], [64, 3] + [1] * 83, [2] * 30 + [90], [1, 1, 1, 147], [63, 65, 22])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channels, taps, act, bias, residual", [(48, 4, "silu", True, False), (60, 2, None, False, True),
                                                                  (520, 7, None, True, False), (35, 3, "silu", False, True)])
def test_convolution_over_time_with_its_state(dtype, channels, taps, act, bias, residual):
    """Whole, in portions shorter than the taps reach, and two sequences side by side; a column range of
    wider rows as the mixers use it."""
    from sonicboom_amd import ops
    from sonicboom_amd.parts import StateSpec
    rt = runtime(dtype)
    h = Harness(rt, states={"s": StateSpec((taps - 1, channels))}, width=channels)
    w, b = rand(channels, taps, seed=1).to(TORCH_DT[dtype]), rand(channels, seed=2).to(TORCH_DT[dtype]) if bias else None
    rows = rand(150, channels + 9, seed=3).to(TORCH_DT[dtype])
    x = rows[:, 5:5 + channels].float().numpy().astype(np.float64)
    want = N.time_conv(x, w.float().numpy(), None if b is None else b.float().numpy())
    want = N.silu(want) if act else want
    want = want + x if residual else want

    def fn(hh, xx, ctx, binding):
        y = ops.time_conv(hh, w.to(DEV), None if b is None else b.to(DEV), binding.states["s"], ctx, F32, activation=act,
                          residual=residual, columns=(5, channels))
        xx.copy_(y)
    for cuts in CUTS:
        part_close(h.feed(fn, rows, cuts), want, "float32" if dtype == "float32" else "bfloat16", f"cuts {cuts[:3]}", bf16=1e-5, f32=1e-5)
    a, b2 = h.feed_batch(fn, [rows[:40], rows[:150]])
    part_close(a, want[:40], dtype, "batch, short", bf16=1e-5, f32=1e-5)
    part_close(b2, want, dtype, "batch, long", bf16=1e-5, f32=1e-5)


def mixer_of(spec, dtype, seed=0, scale=0.5, fast=True, edit=None):
    from sonicboom_amd.parts import build_part
    dev, ref = part_tensors(spec, dtype, seed=seed, scale=scale)
    if edit is not None:
        edit(dev, ref)
    rt = runtime(dtype, fast)
    return build_part(spec, dev, rt), rt, ref


def mixer_harness(mixer, rt, width=64):
    ss = mixer.state_spec()
    return Harness(rt, cache_spec=mixer.cache_spec(), states=ss if isinstance(ss, dict) else None, width=width,
                   tiles=getattr(mixer, "row_tile", None))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, vdim, state, groups, taps, norm_groups", [(4, 32, 16, 2, 4, 2), (3, 20, 24, 1, 3, 1), (8, 8, 40, 8, 2, 4),
                                                                          (2, 64, 128, 2, 4, 1), (1, 48, 7, 1, 5, 3)])
def test_state_space_mixer_alone(dtype, heads, vdim, state, groups, taps, norm_groups):
    from sonicboom_amd.parts.state_space import ssd_spec
    spec = ssd_spec("a.", 64, heads, vdim, state, groups, taps, norm_groups, 1e-5)
    mixer, rt, ref = mixer_of(spec, dtype)
    m = {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": taps, "norm_groups": norm_groups}
    h = rand(150, 64, seed=5).to(TORCH_DT[dtype])
    want = N.mamba2(m, 1e-5, ref, "a.", h.float().numpy())
    hs = mixer_harness(mixer, rt)
    outs = [hs.feed(mixer.forward, h, cuts) for cuts in CUTS]
    for cuts, got in zip(CUTS, outs):
        part_close(got, want, dtype, f"state space, cuts {cuts[:3]}", bf16=3e-2, f32=5e-5)
        if dtype == "float32":
            assert torch.equal(got, outs[0]), "in 32-bit the cut must not matter by a bit"
    a, b = hs.feed_batch(mixer.forward, [h[:40], h])
    part_close(b, want, dtype, "state space, batch", bf16=3e-2, f32=5e-5)
    if dtype == "float32":
        assert torch.equal(b, outs[0]) and torch.equal(a, outs[0][:40])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, taps, ranks", [(4, 2, 16, 32, 3, (8, 16)), (3, 1, 12, 20, 2, (5, 7)), (1, 1, 64, 48, 5, (24, 8)),
                                                                    (2, 2, 32, 64, 4, (24, 24)), (6, 3, 8, 128, 4, (16, 8))])
def test_delta_rule_mixer_alone(dtype, heads, kv_heads, dim, vdim, taps, ranks):
    from sonicboom_amd.parts.state_space import channel_delta_spec
    spec = channel_delta_spec("a.", 64, heads, kv_heads, dim, vdim, taps, 1e-5, decay_rank=ranks[0], gate_rank=ranks[1])
    mixer, rt, ref = mixer_of(spec, dtype)
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps}
    h = rand(150, 64, seed=6).to(TORCH_DT[dtype])
    want = N.channel_delta(m, 1e-5, ref, "a.", h.float().numpy())
    hs = mixer_harness(mixer, rt)
    outs = [hs.feed(mixer.forward, h, cuts) for cuts in CUTS]
    for cuts, got in zip(CUTS, outs):
        part_close(got, want, dtype, f"delta rule, cuts {cuts[:3]}", bf16=4e-2, f32=5e-5)
        if dtype == "float32":
            assert torch.equal(got, outs[0]), "in 32-bit the cut must not matter by a bit"
    a, b = hs.feed_batch(mixer.forward, [h[:40], h])
    part_close(b, want, dtype, "delta rule, batch", bf16=4e-2, f32=5e-5)


def test_a_state_written_once_is_read_hundreds_of_steps_later():
    """The delta rule with no decay: what the first token writes under its key is what a query for that key
    reads 700 single-token steps later, and a slot that is used again starts empty."""
    from sonicboom_amd.parts.state_space import channel_delta_spec
    spec = channel_delta_spec("a.", 64, 1, 1, 16, 16, 2, 1e-5, decay_rank=8, gate_rank=8)

    def edit(dev, ref):
        for name in dev:
            dev[name].zero_()
        dev["a.A_log"].fill_(-30.0)                     # a decay of exp(-exp(-30) ...) = 1
        for d in range(16):
            dev["a.q"][d, d] = dev["a.k"][d, d] = dev["a.v"][d, 16 + d] = 1.0
            dev["a.o"][d, d] = 1.0
        for name in ("a.q.conv", "a.k.conv", "a.v.conv"):
            dev[name][:, -1] = 4.0                      # the current token alone, and a silu that is almost the identity
        dev["a.b"][0, 40] = 1.0                         # beta = sigmoid(20 * flag): the first row writes, the others hardly
        dev["a.norm"].fill_(1.0)
        for name in dev:
            ref[name] = dev[name].float().cpu().numpy().astype(np.float64)
    mixer, rt, ref = mixer_of(spec, "float32", edit=edit)
    m = {"heads": 1, "kv_heads": 1, "dim": 16, "vdim": 16, "conv": 2}
    n = 700
    h = torch.zeros(n, 64)
    h[:, 40] = -20.0
    h[0, 40] = 20.0
    h[0, 3], h[0, 16 + 5] = 5.0, 5.0                   # key 3 holds value 5
    h[1:, 7] = 5.0                                      # the rows between ask for another key
    h[n - 1, 7], h[n - 1, 3] = 0.0, 5.0                # the last row asks for key 3
    want = N.channel_delta(m, 1e-5, ref, "a.", h.numpy())
    assert np.abs(want[n - 1]).argmax() == 5 and np.abs(want[n - 1, 5]) > 10 * np.abs(want[n - 2]).max()
    hs = mixer_harness(mixer, rt)
    for cuts in ([n], [1] * n, [699, 1]):
        part_close(hs.feed(mixer.forward, h, cuts), want, "float32", f"a far write, cuts {cuts[:2]}", f32=1e-4)
    slot = hs.cache.alloc_slot()
    hs.feed(mixer.forward, h[:5], [5], slot=slot)
    hs.cache.free_slot(slot)
    again = hs.cache.alloc_slot()
    assert again == slot
    got = hs.feed(mixer.forward, h[n - 1:], [1], slot=again)
    hs.cache.free_slot(again)
    assert float(got.abs().max()) < 1e-3 * float(np.abs(want[n - 1]).max()), "a slot that is used again starts from an empty state"


def shared_attention_mixer(dtype, heads, kv_heads, dim, scale, coef, every, width=64, seed=0, fast=True, edit=None):
    from sonicboom_amd.parts.shared_attention import shared_attention_spec
    spec = shared_attention_spec("a.", width, heads, kv_heads, dim, 1e-5, scale=scale, temp_coef=coef, temp_every=every)

    def fix(dev, ref):
        for name in ("a.r1", "a.r2"):
            dev[name].abs_()
            ref[name] = np.abs(ref[name])
        if edit is not None:
            edit(dev, ref)
    mixer, rt, ref = mixer_of(spec, dtype, seed=seed, fast=fast, edit=fix)
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "q_temp": {"coef": coef, "every": every}}
    return mixer, rt, ref, m


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, scale, coef, every", [
    (6, 2, 32, 0.5, 0.6, 50), (3, 3, 10, 1.0, 0.0, 1), (5, 1, 16, 0.8, 1.1, 13), (2, 1, 48, 0.4, 0.5, 1), (8, 4, 64, 0.3, 0.2, 64),
    (1, 1, 128, 0.2, 0.3, 100)])
def test_shared_attention_alone(dtype, heads, kv_heads, dim, scale, coef, every):
    mixer, rt, ref, m = shared_attention_mixer(dtype, heads, kv_heads, dim, scale, coef, every)
    h = rand(150, 64, seed=7).to(TORCH_DT[dtype])
    want = N.attention(m, 1e-5, ref, "a.", h.float().numpy())
    hs = mixer_harness(mixer, rt)
    for cuts in CUTS:
        part_close(hs.feed(mixer.forward, h, cuts), want, dtype, f"attention, cuts {cuts[:3]}", bf16=3e-2, f32=5e-5)
    a, b = hs.feed_batch(mixer.forward, [h[:40], h])
    part_close(b, want, dtype, "attention, batch", bf16=3e-2, f32=5e-5)
    part_close(a, want[:40], dtype, "attention, batch", bf16=3e-2, f32=5e-5)


@pytest.mark.parametrize("heads, kv_heads, dim", [(4, 1, 32), (6, 2, 64), (16, 2, 128), (5, 5, 16), (9, 3, 48)])
def test_matrix_core_attention_equals_the_plain_kernel(heads, kv_heads, dim):
    """bfloat16: a prompt, portions and single rows over several pages against the kernel of one wave per
    (row, head, value head)."""
    n = 700
    h = rand(n, 64, seed=8).to(BF16)
    outs = {}
    for fast in (True, False):
        mixer, rt, ref, m = shared_attention_mixer("bfloat16", heads, kv_heads, dim, 2.0 / np.sqrt(dim), 0.4, 100, fast=fast)
        hs = mixer_harness(mixer, rt)
        outs[fast] = [hs.feed(mixer.forward, h, cuts) for cuts in ([n], [560, 17, 3] + [1] * 120)]
    want = N.attention(m, 1e-5, ref, "a.", h.float().numpy())
    for a, b in zip(outs[True], outs[False]):
        part_close(a, b.float().cpu().numpy(), "bfloat16", "matrix cores against the plain kernel", bf16=1.5e-2)
        part_close(a, want, "bfloat16", "matrix cores against the plain implementation", bf16=3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("fast", [True, False])
def test_one_key_stands_out(dtype, fast):
    """A prompt of 700 rows in which the last row asks and one row answers: the query's weight falls on that
    key however far back it lies: the row before, at both sides of page borders, hundreds of rows away, the
    very first row; the distance bias takes some of the score but not the lead.  The values are the keys as
    projected, so the answer carries the planted number.  The query runs as the last row of a prompt, as a
    single decoded row, and behind a portion of two rows."""
    if fast and dtype == "float32":
        pytest.skip("the 32-bit path has one attention kernel")
    dim, width = 16, 48

    def edit(dev, ref):
        for name in dev:
            dev[name].zero_()
        for d in range(dim):
            dev["a.k"][d, d] = 1.0
            for a in range(2):
                dev["a.q"][a * dim + d, dim + d] = 1.0
        dev["a.q.norm"].fill_(1.0)
        dev["a.k.norm"].fill_(1.0)
        dev["a.q.b"][0], dev["a.q.b"][dim], dev["a.k.b"][0] = 1.0, 1.0, 1.0       # a constant that keeps a silent row's norm calm
        dev["a.r1"][:] = torch.tensor([0.3, 0.6])
        dev["a.r2"][:] = torch.tensor([1.0, 0.25])
        dev["a.talk"][:] = torch.tensor([[0.8, 0.3], [-0.2, 1.1]])
        dev["a.o"] = rand(width, 2 * dim, scale=0.3, seed=3).to(dev["a.o"].dtype).to(DEV)
        for name in dev:
            ref[name] = dev[name].float().cpu().numpy().astype(np.float64)
    mixer, rt, ref, m = shared_attention_mixer(dtype, 2, 1, dim, 7.0, 0.5, 256, width=width, fast=fast, edit=edit)
    hs = mixer_harness(mixer, rt, width=width)
    n = 700
    t = n - 1
    for back in [1, 2, 63, 64, 65, 127, 128, 129, 500, 636, 699]:
        j = t - back
        h = torch.zeros(n, width)
        h[j, 1] = 4.0                       # the key that answers
        h[t, dim + 1] = 4.0                 # the query that asks
        want = N.attention(m, 1e-5, ref, "a.", h.numpy())
        silent = h.clone()
        silent[j, 1] = 0.0
        hidden = N.attention(m, 1e-5, ref, "a.", silent.numpy())
        assert np.abs(want[t] - hidden[t]).max() > 0.3 * np.abs(want[t]).max(), "hiding the key would not show: the test shows nothing"
        hd = h.to(TORCH_DT[dtype])
        for cuts in ([n], [n - 1, 1], [n - 3, 2, 1]):
            got = hs.feed(mixer.forward, hd, cuts)
            part_close(got[t:], want[t:], dtype, f"a key {back} back, cuts {cuts}", bf16=4e-2, f32=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows, experts, top, inner, shared, scale", [(40, 4, 1, 48, 0, 1.25), (300, 6, 3, 32, 64, 0.8), (7, 7, 7, 12, 36, 1.0),
                                                                      (1, 16, 3, 64, 96, 1.5), (130, 2, 1, 28, 0, 2.0)])
def test_routed_experts_alone(dtype, rows, experts, top, inner, shared, scale):
    """Sigmoid scores, weights that are not renormalized, an ungated shared expert."""
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.moe import moe_ffn_spec
    width = 64
    spec = moe_ffn_spec("f.", width, experts, top, inner, 0.0, 1.0, shared, 0.0, activation="silu", router_score="sigmoid",
                        router_scale=scale, shared_gate=False)
    dev, ref = part_tensors(spec, dtype, scale=0.4)
    # scores well apart: every row's router input is one of eight codes
    router = torch.zeros(experts, width)
    levels = ((torch.arange(experts)[:, None] - torch.arange(8)[None, :]) % experts).float() - (experts - 1) / 2
    router[:, :8] = levels * 0.7
    dev["f.router"], ref["f.router"] = router.to(TORCH_DT[dtype]).to(DEV), router.numpy().astype(np.float64)
    ffn = build_part(spec, dev, runtime(dtype))
    h = rand(rows, width, seed=9)
    h[:, :8] = 0.0
    h[torch.arange(rows), torch.arange(rows) % 8] = 1.0
    h = h.to(TORCH_DT[dtype])
    cfg_mlp = {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale}, "expert": {"ff": inner},
               "shared": {"ff": shared} if shared else None}
    want = N.moe_ff(cfg_mlp, ref, "f.", h.float().numpy().astype(np.float64))

    class Ctx:
        shared = {}
    x = torch.zeros(rows, width, dtype=F32, device=DEV)
    ffn.forward(h.to(DEV), x, Ctx)
    part_close(x, want, dtype, "routed experts", bf16=3e-2, f32=5e-5)


def test_the_router_kernel_scores_like_the_plain_one():
    from sonicboom_amd import ops
    z = rand(500, 11, scale=2.0, seed=3)
    z[7, 3] = z[7, 5]                        # a tie goes to the lower number
    for top in (1, 4, 11):
        ids, w = ops.moe_route(z.contiguous().to(DEV), 11, top, False, score="sigmoid", score_scale=1.5)
        chosen, weight = N.route(z.numpy().astype(np.float64), top, 1.5)
        assert np.array_equal(ids.cpu().numpy(), chosen)
        assert np.allclose(w[:, :top].cpu().numpy(), weight, atol=1e-6)


# ---- the scans' chunked form against the walk ------------------------------------------------------------------


def scan_context(lens, slots, chunk):
    """What the scans read of a step: rows of sequences of ``lens`` rows in state rows ``slots``, and its chunks."""
    from types import SimpleNamespace
    from sonicboom_amd.engine.step import row_runs
    cu = np.zeros(len(lens) + 1, dtype=np.int32)
    cu[1:] = np.cumsum(lens)
    i32 = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)
    return SimpleNamespace(n_rows=int(cu[-1]), n_seqs=len(lens), cu_rows=i32(cu), slots=i32(slots)), i32(row_runs(lens, cu, chunk))


SCAN_LENS = ([200], [64], [65, 1, 128, 7], [3, 129, 300])


@pytest.mark.parametrize("lens", SCAN_LENS)
@pytest.mark.parametrize("heads, groups, state, vdim", [(4, 2, 16, 32), (3, 1, 24, 20), (2, 2, 128, 64), (1, 1, 7, 130), (2, 1, 160, 24),
                                                        (1, 1, 40, 7), (1, 1, 136, 140), (2, 2, 130, 100)])
def test_state_space_scan_in_chunks_equals_the_walk(lens, heads, groups, state, vdim):
    from sonicboom_amd import ops
    chunk = ops.state_scan_chunk_rows()
    slots = [5, 0, 3, 2][:len(lens)]
    ctx, chunks = scan_context(lens, slots, chunk)
    n, inner, bc = ctx.n_rows, heads * vdim, groups * state
    rows = rand(n, 2 * inner + 2 * bc + heads, seed=31).to(DEV)
    z, x, b, c, dt = rows[:, :inner], rows[:, inner:2 * inner], rows[:, 2 * inner:2 * inner + bc], \
        rows[:, 2 * inner + bc:2 * inner + 2 * bc], rows[:, 2 * inner + 2 * bc:]
    vecs = [rand(heads, scale=0.5, seed=32 + i).to(DEV) for i in range(3)]
    start = rand(6, heads, state, vdim, seed=35).to(DEV)
    walked, chunked = start.clone(), start.clone()
    want = ops.ssd_scan(z, x, b, c, dt, *vecs, walked, ctx, heads, groups, state, vdim)
    got = ops.ssd_scan(z, x, b, c, dt, *vecs, chunked, ctx, heads, groups, state, vdim, chunks)
    part_close(got, want.cpu().numpy(), "float32", "the state space's outputs in chunks", f32=2e-5)
    part_close(chunked, walked.cpu().numpy(), "float32", "the state space's states after chunks", f32=2e-5)
    assert torch.equal(chunked[1], start[1]) and torch.equal(chunked[4], start[4]), "a state row of no sequence was written"


@pytest.mark.parametrize("lens", SCAN_LENS)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim", [(4, 2, 16, 32), (3, 1, 12, 20), (2, 2, 128, 128), (1, 1, 70, 9), (2, 1, 8, 200),
                                                          (2, 1, 144, 40), (1, 1, 33, 255), (1, 1, 136, 140),
                                                          (2, 2, 130, 100)])
def test_delta_rule_scan_in_chunks_equals_the_walk(lens, heads, kv_heads, dim, vdim):
    from sonicboom_amd import ops
    chunk = ops.state_scan_chunk_rows()
    slots = [5, 0, 3, 2][:len(lens)]
    ctx, chunks = scan_context(lens, slots, chunk)
    n = ctx.n_rows
    qkv = rand(n, 2 * kv_heads * dim + heads * vdim, seed=41).to(DEV)
    beta, decay, gate = rand(n, heads, seed=42).to(DEV), rand(n, heads * dim, seed=43).to(DEV), rand(n, heads * vdim, seed=44).to(DEV)
    dt_bias, a_log, w = rand(heads * dim, scale=0.5, seed=45).to(DEV), (rand(heads, scale=0.5, seed=46) - 1.0).to(DEV), \
        (1.0 + rand(vdim, scale=0.1, seed=47)).to(DEV)
    start = rand(6, heads, dim, vdim, seed=48).to(DEV)
    walked, chunked = start.clone(), start.clone()
    args = (heads, kv_heads, dim, vdim, 1e-5, 1e-6, F32)
    want = ops.delta_scan(qkv, beta, decay, gate, dt_bias, a_log, w, walked, ctx, *args)
    got = ops.delta_scan(qkv, beta, decay, gate, dt_bias, a_log, w, chunked, ctx, *args, chunks)
    part_close(got, want.cpu().numpy(), "float32", "the delta rule's outputs in chunks", f32=5e-5)
    part_close(chunked, walked.cpu().numpy(), "float32", "the delta rule's states after chunks", f32=5e-5)
    assert torch.equal(chunked[1], start[1]) and torch.equal(chunked[4], start[4]), "a state row of no sequence was written"
