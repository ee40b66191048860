"""Decode and prefill throughput of the Qwen2.5 layer sizes with random bf16 weights on one
MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]
                    [--sizes 0.5b|1.5b|3b|7b|14b|32b|72b] [--prompt T] [--context C] [--workload steady|mixed|forms]

A "step" is one decode step: every sequence of the batch goes on by one token (step function,
greedy choice on the device, the token fed back).

``--workload steady`` (the default) has the sizes of the benchmark configuration (28 layers,
width 3584, 28 heads, 4 kv heads, head size 128, inner width 18944, vocabulary 152064), a batch
of 8 and a cache for 4096 tokens per sequence, each holding a 2,048-token prompt of seeded random
ids.  One JSON line is printed: decoded tokens a second (from the median step), the prefill of one
2,048-token prompt, the decode step against the HBM roofline with the rates of its kernels, and
decode at batch 1 and 64.

The same line carries the context-length curve as further ``points`` (and with bytes, flops and
fractions under ``curve``): for cached depths of 512, 4,096, 8,192, 16,384 and 32,768 tokens the
decode rate at batch 1 and batch 8 (``decode_b1_d8192`` ...) and the prefill rate of one prompt of
that length (``prefill_8192`` ...); ``--no-curve`` leaves it out, ``--curve 512,4096`` picks depths.
``--runs R`` (R > 1) starts R fresh processes of the same command one after the other, before
anything touches the GPU here, and prints the run whose ``value`` is the median, with all values.
Beside the JSON line on standard output, every metric goes to standard error as a
``RESULT key=value ...`` line; the engine clock sampled during the timed decode steps is in both.

``--workload mixed`` runs what the baseline names for the larger sizes through the generation
loop itself: ``--sizes 14b``: 16 prompts of seeded lengths uniform in [256, 4096] in a cache of
8192 tokens a sequence, prompts in one step, then 256 greedy steps; ``--sizes 72b``: 8 prompts of
512 to 2048 tokens, 128 steps, 4096 tokens a sequence.  Prefill and decode are timed apart.

``--workload designs`` runs the Rasizen design (gated recurrences and latent attention) at a few
layer sizes that resemble a real model's (``--design-sizes``: widths) beside the Qwen2.5 design at
the same width, head count and feed-forward weight count: prefill of one ``--prompt``-token prompt
and decode of ``--batch`` sequences at that depth, tokens a second, and the time of every kernel of
one prompt step and one decode step with what it reaches of its roofline (bytes it must move over
8 TB/s, or flops over the dense bf16 peak, whichever is the larger time).  A table goes to standard
error, one JSON line to standard output.  ``--design tatelorn`` puts the Tatelorn design (blocks that
norm what their sublayers give back, attention with head norms, capped scores and a sink, routed
experts) in the Rasizen design's place (``--design fitatar``: the Fitatar design, layers of two parallel branches with
latent attention through a query latent, gated attention with a sink score a head and experts chosen within groups;
``--design nalasun``: the Nalasun design, state-space and delta-rule
recurrences, attention with shared head weights and routed experts behind short convolutions): eight layers, the first with a dense gated feed-forward, the
others with eight experts of which a row takes two plus a shared one, so that a row passes as many
feed-forward weights as in the Qwen2.5 design beside it, and the same heads.

``--workload forms`` prints a table instead of the line: the decode step (``--batches 1,8``) with
the qkv, output and down product forced, one at a time, to every form (waves a block x K slices)
of the kernel that streams the weights, against the launchers' own choices.
"""
import argparse
import json
import statistics
import sys
import time

PEAK_HBM_GBS = 8000.0            # MI355X, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

CONFIG_7B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 28, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
    "intermediate_size": 18944, "vocab_size": 152064, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 131072, "tie_word_embeddings": False, "use_sliding_window": False,
    "hidden_act": "silu",
}
# the other sizes the baseline names, for runs beyond the default one (--sizes)
CONFIG_14B = dict(CONFIG_7B, num_hidden_layers=48, hidden_size=5120, num_attention_heads=40,
                  num_key_value_heads=8, intermediate_size=13824)
CONFIG_72B = dict(CONFIG_7B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64,
                  num_key_value_heads=8, intermediate_size=29568)
CONFIG_32B = dict(CONFIG_14B, num_hidden_layers=64, intermediate_size=27648)
# the family's small members: tied head, a vocabulary of 151,936
CONFIG_05B = dict(CONFIG_7B, num_hidden_layers=24, hidden_size=896, num_attention_heads=14, num_key_value_heads=2,
                  intermediate_size=4864, vocab_size=151936, tie_word_embeddings=True)
CONFIG_15B = dict(CONFIG_05B, num_hidden_layers=28, hidden_size=1536, num_attention_heads=12, intermediate_size=8960)
CONFIG_3B = dict(CONFIG_05B, num_hidden_layers=36, hidden_size=2048, num_attention_heads=16, intermediate_size=11008)
SIZES = {"7b": ("Qwen2.5-7B", CONFIG_7B), "14b": ("Qwen2.5-14B", CONFIG_14B), "72b": ("Qwen2.5-72B", CONFIG_72B),
         "32b": ("Qwen2.5-32B", CONFIG_32B), "0.5b": ("Qwen2.5-0.5B", CONFIG_05B), "1.5b": ("Qwen2.5-1.5B", CONFIG_15B),
         "3b": ("Qwen2.5-3B", CONFIG_3B)}
# the mixed workloads: prompts, shortest, longest, greedy steps, cache tokens a sequence
MIXED = {"72b": (8, 512, 2048, 128, 4096), "32b": (8, 512, 2048, 128, 4096)}
MIXED_DEFAULT = (16, 256, 4096, 256, 8192)
CONTEXT = 4096
PROMPT = 2048
CURVE_DEPTHS = (512, 4096, 8192, 16384, 32768)
CURVE_BATCHES = (1, 8)


def model_numbers(cfg, n_layers):
    d, ff, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    hq, hkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = d // hq
    qw, kvw = hq * hd, hkv * hd
    layer_params = d * (qw + 2 * kvw) + (qw + 2 * kvw) + qw * d + 3 * d * ff + 2 * d
    return dict(d=d, ff=ff, v=v, hq=hq, hkv=hkv, hd=hd, qw=qw, kvw=kvw, layer_params=layer_params,
                layers=n_layers)


def prefill_flops(m, lengths):
    """Flops of a prompt step of sequences of these lengths whose last rows go through the head."""
    t = sum(lengths)
    per_layer = 2 * t * (m["d"] * (m["qw"] + 2 * m["kvw"]) + m["qw"] * m["d"] + 3 * m["d"] * m["ff"])
    attn = sum(4 * (n * (n + 1) // 2) * m["hq"] * m["hd"] for n in lengths)   # scores and mix, causal pairs
    return m["layers"] * (per_layer + attn) + len(lengths) * 2 * m["v"] * m["d"]


def decode_bytes(m, batch, lengths):
    """Bytes a decode step has to read: every weight it uses once (bf16), the embedding rows of
    the batch, and the cached keys and values of the live requests."""
    weights = m["layers"] * m["layer_params"] * 2 + (m["v"] * m["d"] + m["d"]) * 2 + batch * m["d"] * 2
    kv = sum(lengths) * 2 * m["kvw"] * 2 * m["layers"]
    return weights + kv


class ClockSampler:
    """Samples the GPU's engine clock in a thread while work runs (the driver's ``pp_dpm_sclk``
    file, else ``rocm-smi --showclocks``): what the matrix pipes' peak has to be scaled by under
    load, and what a run's figures have to be read against."""

    def __init__(self, period=0.4):
        import threading
        self.period, self.mhz, self._stop = period, [], threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True)

    @staticmethod
    def read():
        import glob
        import re
        import subprocess
        # the driver's own file first (microseconds to read): the level marked with a star
        for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
            try:
                with open(path) as f:
                    m = re.search(r"(\d+)\s*Mhz\s*\*", f.read(), re.IGNORECASE)
            except OSError:
                continue
            if m:
                return int(m.group(1))
        try:
            out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20).stdout
        except (OSError, subprocess.SubprocessError):
            return None
        m = re.search(r"sclk clock level: \S+ \((\d+)Mhz\)", out)
        return int(m.group(1)) if m else None

    def _run(self):
        while not self._stop.is_set():
            v = self.read()
            if v is not None:
                self.mhz.append(v)
            self._stop.wait(self.period)

    def __enter__(self):
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._thread.join()

    def summary(self):
        if not self.mhz:
            return None
        return {"samples": len(self.mhz), "min_mhz": min(self.mhz), "max_mhz": max(self.mhz),
                "median_mhz": int(statistics.median(self.mhz))}


class OpTimer:
    """Times the kernel calls of one step that runs kernel by kernel: every function of
    ``sonicboom_amd.ops`` that launches is wrapped between two events on the stream, and the
    times are summed by (function, what it worked on)."""

    NAMES = ("embed", "rmsnorm", "gemm_bf16", "gemm_bf16_partial", "reduce_resid_norm", "rope_kv_store",
             "attention", "attention_decode_rope", "argmax", "gemm_plain", "silu_mul", "add_into", "cast")

    def __init__(self, m):
        self.m, self.records, self._saved = m, [], {}

    def _label(self, name, args, kw):
        m = self.m
        if name in ("gemm_bf16", "gemm_bf16_partial"):
            n, k = kw.get("packed_shape") or (args[1].shape[0], args[1].shape[-1])
            if kw.get("gated"):
                return "gate_up"
            return {(m["qw"] + 2 * m["kvw"], m["d"]): "qkv", (m["d"], m["qw"]): "out", (m["d"], m["ff"]): "down",
                    (m["v"], m["d"]): "head"}.get((n, k), f"product_{n}x{k}")
        # (a decode step's attention rotates and stores the new key and value itself)
        return {"reduce_resid_norm": "add_slices_norm", "rope_kv_store": "rotate_store",
                "attention_decode_rope": "attention"}.get(name, name)

    def __enter__(self):
        import torch
        from sonicboom_amd import ops
        for name in self.NAMES:
            fn = getattr(ops, name)
            self._saved[name] = fn

            def timed(*args, _fn=fn, _name=name, **kw):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                out = _fn(*args, **kw)
                e1.record()
                if out is not None or _name not in ("gemm_bf16", "gemm_bf16_partial"):   # None: not taken
                    self.records.append((self._label(_name, args, kw), e0, e1))
                return out
            setattr(ops, name, timed)
        return self

    def __exit__(self, *exc):
        from sonicboom_amd import ops
        for name, fn in self._saved.items():
            setattr(ops, name, fn)

    def totals(self):
        """label -> (microseconds, calls)"""
        import torch
        torch.cuda.synchronize()
        out = {}
        for label, e0, e1 in self.records:
            us, n = out.get(label, (0.0, 0))
            out[label] = (us + e0.elapsed_time(e1) * 1e3, n + 1)
        return out


def kernel_rates(m, totals, rows, kv_tokens, prefill_lengths=None):
    """Achieved rates of the step's kernels from an OpTimer's totals: GB/s of the bytes each must
    read for a decode step, TFLOP/s for a prompt step."""
    L = m["layers"]
    weights = {"qkv": m["d"] * (m["qw"] + 2 * m["kvw"]), "out": m["qw"] * m["d"], "gate_up": 2 * m["d"] * m["ff"],
               "down": m["d"] * m["ff"]}
    out = {}
    for label, (us, calls) in sorted(totals.items()):
        item = {"us": round(us, 1), "calls": calls}
        if prefill_lengths is None:
            if label in weights:
                item["GB/s"] = round(weights[label] * 2 * calls / us / 1e3, 1)
            elif label == "head":
                item["GB/s"] = round(m["v"] * m["d"] * 2 * calls / us / 1e3, 1)
            elif label == "attention":
                item["GB/s"] = round(kv_tokens * 2 * m["kvw"] * 2 * calls / us / 1e3, 1)
            if "GB/s" in item:
                item["frac"] = round(item["GB/s"] / PEAK_HBM_GBS, 3)
        else:
            if label in weights:
                # per layer, not per call: a long prompt runs in portions, several calls a layer
                item["TFLOP/s"] = round(2 * rows * weights[label] * L / us / 1e6, 1)
            elif label == "attention":
                flops = sum(4 * (n * (n + 1) // 2) * m["hq"] * m["hd"] for n in prefill_lengths)
                item["TFLOP/s"] = round(flops * L / us / 1e6, 1)
            if "TFLOP/s" in item:
                item["frac"] = round(item["TFLOP/s"] * 1e12 / PEAK_FLOPS["bf16"], 3)
        out[label] = item
    return out


def main() -> int:
    global PROMPT, CONTEXT
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="run fewer layers than the configuration has")
    ap.add_argument("--sizes", choices=sorted(SIZES), default="7b", help="layer sizes (default: the benchmark's)")
    ap.add_argument("--prompt", type=int, default=PROMPT, help="cached prompt tokens per sequence")
    ap.add_argument("--context", type=int, default=CONTEXT, help="cache size per sequence")
    ap.add_argument("--workload", choices=("steady", "mixed", "forms", "designs"), default="steady")
    ap.add_argument("--design", choices=("rasizen", "tatelorn", "nalasun", "fitatar"), default="rasizen",
                    help="--workload designs: the design that runs beside the Qwen2.5 design")
    ap.add_argument("--beside", choices=("qwen2", "rasizen", "tatelorn", "nalasun", "fitatar"), default="qwen2",
                    help="--workload designs: the design at the same sizes that the first one runs beside")
    ap.add_argument("--design-sizes", default="2048,4096",
                    help="--workload designs: the widths of the layer sizes to run, comma separated")
    ap.add_argument("--batches", default="1,8", help="--workload forms: the batch sizes, comma separated")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    ap.add_argument("--no-graph", action="store_true", help="launch decode steps kernel by kernel")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel rates")
    ap.add_argument("--clocks", action="store_true",
                    help="also run prompt steps back to back for a few seconds and sample the engine clock meanwhile")
    ap.add_argument("--curve", default=",".join(str(d) for d in CURVE_DEPTHS),
                    help="cached depths of the context-length curve (decode at batch 1 and 8, prefill of one prompt)")
    ap.add_argument("--no-curve", action="store_true", help="skip the context-length curve")
    ap.add_argument("--runs", type=int, default=1,
                    help="fresh processes to run one after the other; the median run is printed")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported")
        return 2
    if a.runs > 1:
        argv, skip = [], False
        for arg in sys.argv[1:]:
            if skip:
                skip = False
            elif arg == "--runs":
                skip = True
            elif not arg.startswith("--runs="):
                argv.append(arg)
        return median_of_runs(argv, a.runs)

    if a.workload == "designs":
        return design_comparison(a)

    import numpy as np
    import torch

    from sonicboom_amd import ops
    from sonicboom_amd.engine import DecoderModel, Engine, StepEntry, generate
    from sonicboom_amd.engine.decode import DecodeLoop
    from sonicboom_amd.sampling import SamplingParams

    PROMPT, CONTEXT = a.prompt, max(a.context, a.prompt + a.steps + a.warmup + 64)
    if a.prompt != 2048 and "--curve" not in " ".join(sys.argv[1:]):
        a.no_curve = True           # a run at a depth of its own is one point, not the curve
    model_name, base_cfg = SIZES[a.sizes]
    cfg = dict(base_cfg)
    full_layers = cfg["num_hidden_layers"]
    if a.layers:
        cfg["num_hidden_layers"] = a.layers
    cfg["max_position_embeddings"] = max(cfg["max_position_embeddings"], CONTEXT)
    m = model_numbers(cfg, cfg["num_hidden_layers"])
    t0 = time.time()
    model = DecoderModel.from_random(cfg, seed=0, dtype="bfloat16", device="cuda:0")
    torch.cuda.synchronize()
    print(f"[bench] model of {cfg['num_hidden_layers']} layers ready in {time.time() - t0:.1f} s, "
          f"{torch.cuda.max_memory_allocated() / 2**30:.1f} GiB at most on the device",
          file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)
    peak_measured = None if a.no_kernels else round(ops.read_bandwidth() / 1e9, 1)

    def config(**more):
        c = {
            "model": f"{model_name} sizes, random bf16 weights", "layers": cfg["num_hidden_layers"],
            "layers_of_configuration": full_layers, "hidden_size": m["d"], "num_attention_heads": m["hq"],
            "num_key_value_heads": m["hkv"], "head_dim": m["hd"], "intermediate_size": m["ff"],
            "vocab_size": m["v"], "rope_theta": cfg["rope_theta"], "rms_norm_eps": cfg["rms_norm_eps"],
            "tie_word_embeddings": bool(cfg["tie_word_embeddings"]), "parallelism": "single GPU", "decode_graph": not a.no_graph,
        }
        c.update(more)
        return c

    def random_prompts(lengths):
        return [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)] for n in lengths]

    def sync_time(fn):
        torch.cuda.synchronize()
        t = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        return time.perf_counter() - t

    # ------------------------------------------------------------------------------------------
    if a.workload == "forms":
        # The decode step with one product at a time forced to every form of the weight-streaming
        # kernel (waves a block x K slices), everything else as the launchers choose: a table on
        # standard output, no JSON line.  The products are told apart by their packed shapes.
        d, ff = m["d"], m["ff"]
        targets = {"qkv": ((m["hq"] + 2 * m["hkv"]) * m["hd"], d), "out": (d, m["hq"] * m["hd"]), "down": (d, ff)}
        forced = {"shape": None, "form": (0, 0)}
        launcher_partial = ops.gemm_bf16_partial

        def partial(x, w, packed_shape=None):
            if packed_shape is not None and tuple(packed_shape) == forced["shape"]:
                with ops.gemm_few_rows_kernel(None, *forced["form"]):
                    return launcher_partial(x, w, packed_shape=packed_shape)
            return launcher_partial(x, w, packed_shape=packed_shape)
        ops.gemm_bf16_partial = partial
        layers = cfg["num_hidden_layers"]
        slice_counts = (1, 2, 3, 4, 5, 6, 8)
        for batch in (int(b) for b in a.batches.split(",")):
            eng = Engine(model, ((PROMPT + 511) // 64) * 64 * batch, max_slots=batch)
            slots = [eng.alloc_slot() for _ in range(batch)]
            eng.step([StepEntry(s, p, (PROMPT - 1,)) for s, p in zip(slots, random_prompts([PROMPT] * batch))])

            def step_ms(shape, form):
                forced["shape"], forced["form"] = shape, form
                loop = DecodeLoop(eng, use_graph=not a.no_graph)
                loop.start(slots, [1] * batch)
                for _ in range(4):
                    loop.step()
                times = [sync_time(loop.step) for _ in range(24)]
                loop.close()
                for s in slots:
                    eng.cache.truncate(s, PROMPT)
                return statistics.median(times) * 1e3
            own = statistics.median(step_ms(None, (0, 0)) for _ in range(3))
            print(f"{model_name} sizes, batch {batch}, {PROMPT} cached tokens: the launchers' own choices {own:.4f} ms a step")
            for name, shape in targets.items():
                print(f"  {name} {shape[0]} x {shape[1]} ({shape[0] * shape[1] * 2 / 1e6:.1f} MB); step in ms (difference a layer "
                      f"in us) by waves; columns: {', '.join(str(c) for c in slice_counts)} slices", flush=True)
                for waves in (4, 5, 6, 7, 8):
                    cells = []
                    for slices in slice_counts:
                        t = step_ms(shape, (waves, slices))
                        cells.append(f"{t:.3f} ({(t - own) * 1e3 / layers:+.2f})")
                    print(f"    {waves} waves: " + "  ".join(cells), flush=True)
            for s in slots:
                eng.free_slot(s)
            del eng
        ops.gemm_bf16_partial = launcher_partial
        return 0

    if a.workload == "mixed":
        n_prompts, shortest, longest, n_steps, per_seq = MIXED.get(a.sizes, MIXED_DEFAULT)
        lengths = [int(n) for n in rng.integers(shortest, longest + 1, size=n_prompts)]
        prompts = random_prompts(lengths)
        engine = Engine(model, max_tokens=per_seq * n_prompts)
        engine.use_graphs = not a.no_graph
        params = SamplingParams(max_tokens=n_steps)
        marks = []

        def run():
            marks.clear()
            t_start = time.perf_counter()

            def first_token(i, t):
                if not marks:
                    marks.append(time.perf_counter())      # the prompt step and the first choice are done
                return False
            outs = generate(engine, prompts, params, stop_tokens=(), max_batch=n_prompts, callback=first_token)
            torch.cuda.synchronize()
            t_end = time.perf_counter()
            assert all(len(o) == n_steps for o in outs)
            return marks[0] - t_start, t_end - marks[0]

        warm = generate(engine, [p[:64] for p in prompts], SamplingParams(max_tokens=4), stop_tokens=(),
                        max_batch=n_prompts)          # compiles nothing, but pages in the kernels
        del warm
        runs = [run() for _ in range(3)]
        prefill_s = statistics.median(r[0] for r in runs)
        decode_s = statistics.median(r[1] for r in runs)
        decoded = n_prompts * (n_steps - 1)           # the first token of each comes from the prompt step
        step_s = decode_s / (n_steps - 1)
        mean_lengths = [n + n_steps / 2 for n in lengths]
        nbytes = decode_bytes(m, n_prompts, mean_lengths)
        pf = prefill_flops(m, lengths)
        line = {
            "metric": f"decode tokens/s, {model_name} sizes, {n_prompts} prompts of {shortest}-{longest} tokens "
                      f"in one batch, {n_steps} greedy steps through the generation loop",
            "value": round(decoded / decode_s, 1), "unit": "tokens/s", "n_gpus": 1, "steps": n_steps - 1,
            "warmup": 1, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": config(global_batch=n_prompts, seq_len=per_seq, prompt_tokens=sum(lengths),
                             shortest_prompt=min(lengths), longest_prompt=max(lengths)),
            "prefill": {"value": round(sum(lengths) / prefill_s, 1), "tokens": sum(lengths),
                        "ms": round(prefill_s * 1e3, 3), "frac": round(pf / prefill_s / PEAK_FLOPS["bf16"], 4)},
            "roofline": {"bound": "hbm", "achieved": round(nbytes / step_s / 1e9, 1), "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": round(nbytes / step_s / 1e9 / PEAK_HBM_GBS, 4),
                         "peak_measured": peak_measured, "bytes_per_step": int(nbytes)},
            "runs": [{"prefill_ms": round(p * 1e3, 2), "decode_ms": round(d * 1e3, 2)} for p, d in runs],
        }
        print(json.dumps(line), flush=True)
        return 0

    # ---- prefill of one prompt (2,048 tokens unless --prompt says otherwise) ----------------
    def prefill_run(engine, n_tokens, timed, kernels):
        """Median seconds of ``timed`` prompt steps of one prompt of ``n_tokens`` in an empty slot
        (after one untimed step), as the bench line's ``prefill`` entry."""
        times = []
        for i in range(timed + 1):
            p = random_prompts([n_tokens])[0]
            slot = engine.alloc_slot()
            times.append(sync_time(lambda: engine.step([StepEntry(slot, p, (n_tokens - 1,))])))
            engine.free_slot(slot)
        secs = statistics.median(times[1:])
        pf = prefill_flops(m, [n_tokens])
        out = {"value": round(n_tokens / secs, 1), "tokens": n_tokens, "ms": round(secs * 1e3, 3),
               "frac": round(pf / secs / PEAK_FLOPS["bf16"], 4), "flops": int(pf)}
        if kernels:
            slot = engine.alloc_slot()
            with OpTimer(m) as timer:
                engine.step([StepEntry(slot, random_prompts([n_tokens])[0], (n_tokens - 1,))])
            engine.free_slot(slot)
            out["kernels"] = kernel_rates(m, timer.totals(), n_tokens, 0, prefill_lengths=[n_tokens])
        return out, pf

    engine = Engine(model, max_tokens=CONTEXT)
    prefill, pf = prefill_run(engine, PROMPT, 4, not a.no_kernels)
    if a.clocks:
        idle = ClockSampler.read()
        p = random_prompts([PROMPT])[0]
        with ClockSampler() as sampler:
            t_end = time.time() + 6.0
            n_runs, t_run = 0, 0.0
            while time.time() < t_end:
                slot = engine.alloc_slot()
                t_run += sync_time(lambda: engine.step([StepEntry(slot, p, (PROMPT - 1,))]))
                engine.free_slot(slot)
                n_runs += 1
        clocks = sampler.summary()
        if clocks is not None:
            clocks.update(idle_mhz=idle, prompt_steps=n_runs, ms_per_prompt_step=round(t_run / n_runs * 1e3, 3),
                          frac_at_median_clock=round(pf / (t_run / n_runs) / (PEAK_FLOPS["bf16"] * clocks["median_mhz"] / 2400.0), 4))
        prefill["clocks"] = clocks
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)
    del engine

    # ---- decode -----------------------------------------------------------------------------
    def decode_steps(eng, slots, first, steps, warmup, kernels=False, clock=None):
        """Time ``steps`` decode steps of the sequences in ``slots`` (fed ``first``) after
        ``warmup`` untimed ones: median and mean seconds a step, the lengths after the run, the
        kernels' rates, and the tokens the next step would feed."""
        loop = DecodeLoop(eng, use_graph=not a.no_graph)
        batch = len(slots)
        loop.start(slots, first)
        for _ in range(warmup):
            loop.step()
        torch.cuda.synchronize()
        per_step = []
        if clock is not None:
            clock.__enter__()
        t_all = time.perf_counter()
        for _ in range(steps):
            t = time.perf_counter()
            loop.step()                         # ends with the chosen tokens on the host
            per_step.append(time.perf_counter() - t)
        torch.cuda.synchronize()
        mean = (time.perf_counter() - t_all) / steps
        if clock is not None:
            clock.__exit__()
        lengths = [eng.length(s) for s in slots]
        rates = None
        if kernels:
            plain = DecodeLoop(eng, use_graph=False)
            plain.start(slots, loop.pending)
            plain.step()
            with OpTimer(m) as timer:
                plain.step()
            rates = kernel_rates(m, timer.totals(), batch, sum(lengths) + batch, None)
            loop.pending = plain.pending
        pending = list(loop.pending)
        loop.close()
        return statistics.median(per_step), mean, lengths, rates, pending

    def fill(eng, batch, prompt):
        """``batch`` slots, each with a cached prompt of ``prompt`` random tokens, and the first
        token of each; the prompts run in one step (in portions of the engine's row limit)."""
        slots = [eng.alloc_slot() for _ in range(batch)]
        ps = random_prompts([prompt] * batch)
        logits = eng.step([StepEntry(s, p, (prompt - 1,)) for s, p in zip(slots, ps)])
        return slots, torch.argmax(logits, dim=-1).tolist()

    def per_sequence(prompt, steps, warmup):
        """Cache tokens a sequence needs for these runs (whole pages, with room to spare)."""
        return ((prompt + 2 * (steps + warmup) + 8 + 127) // 64) * 64

    def decode_run(batch, steps, warmup, kernels=False, clock=None):
        eng = Engine(model, max_tokens=max(CONTEXT, per_sequence(PROMPT, steps, warmup)) * batch)
        slots, first = fill(eng, batch, PROMPT)
        out = decode_steps(eng, slots, first, steps, warmup, kernels, clock)
        for s in slots:
            eng.free_slot(s)
        del eng
        return out[:4]

    def hbm(nbytes, secs):
        return {"bound": "hbm", "achieved": round(nbytes / secs / 1e9, 1), "peak": PEAK_HBM_GBS,
                "unit": "GB/s", "frac": round(nbytes / secs / 1e9 / PEAK_HBM_GBS, 4),
                "peak_measured": peak_measured, "bytes_per_step": int(nbytes)}

    sampler = ClockSampler(period=0.2)
    idle_mhz = ClockSampler.read()
    step_s, mean_s, lengths, rates = decode_run(a.batch, a.steps, a.warmup, kernels=not a.no_kernels, clock=sampler)
    clock = sampler.summary()
    if clock is not None:
        clock["idle_mhz"] = idle_mhz
    value = a.batch / step_s
    roofline = hbm(decode_bytes(m, a.batch, lengths), step_s)
    if rates is not None:
        roofline["kernels"] = rates
    print(f"[bench] decode b{a.batch}: {value:.1f} tok/s, median {step_s * 1e3:.3f} ms/step "
          f"(mean {mean_s * 1e3:.3f}), {roofline}, engine clock {clock}", file=sys.stderr, flush=True)
    points = {}
    if not a.no_points:
        for b in (1, 64):
            dt, _, _, _ = decode_run(b, max(16, a.steps // 2), max(4, a.warmup // 2))
            points[f"decode_b{b}"] = round(b / dt, 1)
            print(f"[bench] decode b{b}: {points[f'decode_b{b}']} tok/s", file=sys.stderr, flush=True)

    # ---- the context-length curve --------------------------------------------------------------
    curve = {}
    depths = [] if (a.no_curve or a.no_points) else [int(d) for d in a.curve.split(",") if d.strip()]
    steps_c, warm_c = max(8, min(a.steps, 32)), max(3, min(a.warmup, 8))
    for depth in depths:
        per_seq = per_sequence(depth, steps_c, warm_c)
        eng = Engine(model, max_tokens=per_seq * max(CURVE_BATCHES))
        item, _ = prefill_run(eng, depth, 2, not a.no_kernels)
        if "kernels" in item:          # the curve keeps the rate of the kernel that grows with the depth
            item["attention_TFLOPs"] = item["kernels"].get("attention", {}).get("TFLOP/s")
            item["attention_frac"] = item["kernels"].get("attention", {}).get("frac")
            del item["kernels"]
        entry = {"prefill": item}
        points[f"prefill_{depth}"] = item["value"]
        slots, first = fill(eng, max(CURVE_BATCHES), depth)
        for b in sorted(CURVE_BATCHES, reverse=True):        # the larger batch first, then its first sequences
            for s in slots[b:]:
                eng.free_slot(s)
            slots, first = slots[:b], first[:b]
            dt, _, lens, rates_c, first = decode_steps(eng, slots, first, steps_c, warm_c, kernels=not a.no_kernels)
            d_item = {"value": round(b / dt, 1), "ms": round(dt * 1e3, 4)}
            d_item.update({k: v for k, v in hbm(decode_bytes(m, b, lens), dt).items()
                           if k in ("achieved", "frac", "bytes_per_step")})
            if rates_c is not None and "attention" in rates_c:
                d_item["attention_us"] = rates_c["attention"]["us"]
                d_item["attention_GBs"] = rates_c["attention"].get("GB/s")
            entry[f"decode_b{b}"] = d_item
            points[f"decode_b{b}_d{depth}"] = d_item["value"]
        for s in slots:
            eng.free_slot(s)
        del eng
        curve[f"d{depth}"] = entry
        print(f"[bench] depth {depth}: {entry}", file=sys.stderr, flush=True)

    # ---- prefix reuse: a 512-token prefix is in the cache, 64 new tokens come, time to the first token ----
    prefix_reuse = None
    if depths:
        from sonicboom_amd.api import Model
        session = Model(model).session(max_tokens=64 * 32)
        base = random_prompts([512])[0]
        session.generate([base], max_tokens=1, stop_tokens=[], keep=True)
        with_reuse, whole = [], []
        for i in range(6):
            new = base + random_prompts([64])[0]
            with_reuse.append(sync_time(lambda: session.generate([new], max_tokens=1, stop_tokens=[], keep=True)))
            assert session.reused == [512]
        session.forget()
        for i in range(4):
            new = base + random_prompts([64])[0]
            whole.append(sync_time(lambda: session.generate([new], max_tokens=1, stop_tokens=[])))
        prefix_reuse = {"prefix": 512, "new": 64, "ttft_ms": round(statistics.median(with_reuse[1:]) * 1e3, 3),
                        "ttft_ms_without_reuse": round(statistics.median(whole[1:]) * 1e3, 3)}
        print(f"[bench] prefix reuse {prefix_reuse}", file=sys.stderr, flush=True)
        del session

    line = {
        "metric": f"decode tokens/s, {model_name} sizes, batch {a.batch}, {PROMPT}-token cached prompts",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "ms_per_step_mean": round(mean_s * 1e3, 4),
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": config(global_batch=a.batch, seq_len=CONTEXT, cached_prompt_tokens=PROMPT),
        "prefill": prefill, "roofline": roofline, "points": points, "clock": clock,
    }
    if curve:
        line["curve"] = curve
    if prefix_reuse:
        line["prefix_reuse"] = prefix_reuse
    result_lines(line)
    print(json.dumps(line), flush=True)
    return 0


# ---- the designs side by side --------------------------------------------------------------------
def rasizen_sizes(width, n_blocks=2, window=4096, vocab=32768):
    """Layer sizes in the manner of a real model of this width: heads of 128 plain + 64 rotated
    numbers and 128 values, a latent of 512, an ungated feed-forward of 4 widths, recurrences of 2
    widths; a block of four layers = recurrence, attention with its own latent, attention that
    reads it, recurrence; the attention layers carry the feed-forwards."""
    heads = width // 128
    att = {"heads": heads, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "scale": 192 ** -0.5,
           "mask": {"size": window}, "rot": {"base": 1e6, "dims": 64}}
    layers = []
    for b in range(n_blocks):
        own = len(layers) + 1
        layers += [{"type": "mingru", "mixer": {"width": 2 * width}, "mlp": None},
                   {"type": "latent_attention", "mixer": dict(att), "mlp": {"kind": "dense", "ff": 4 * width}},
                   {"type": "latent_attention", "mixer": dict(att, kv_from=own), "mlp": {"kind": "dense", "ff": 4 * width}},
                   {"type": "mingru", "mixer": {"width": 2 * width}, "mlp": None}]
    return {"architecture": "Rasizen", "vocab": vocab, "width": width, "residual_mult": 0.5,
            "norm": {"eps": 1e-5, "groups": 2}, "layers": layers}


def qwen_sizes(width, n_layers=8, vocab=32768):
    """The Qwen2.5 design at the same width, head count and number of layers, a gated feed-forward of the same weight
    count as the ungated one of 4 widths (inner 8/3 widths, in 256s), a quarter of the heads as kv heads."""
    heads = width // 128
    return dict(CONFIG_7B, num_hidden_layers=n_layers, hidden_size=width, num_attention_heads=heads,
                num_key_value_heads=max(1, heads // 4), intermediate_size=(8 * width // 3 + 255) // 256 * 256,
                vocab_size=vocab, tie_word_embeddings=True)


def tatelorn_sizes(width, n_layers=8, vocab=32768, experts=8, top=2):
    """Layer sizes in the manner of a real model of this width: heads of 128 for keys and for values, a quarter
    of them kv heads, every layer mixing values; the first layer with a dense feed-forward of 8/3 widths, the
    others with `experts` experts of one width of which a row takes `top`, and a shared expert that brings a
    row's feed-forward weights to those of the dense layer."""
    heads = width // 128
    inner = (8 * width // 3 + 255) // 256 * 256
    mixer = {"heads": heads, "kv_heads": max(1, heads // 4), "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
             "softcap": 30.0, "v_mix": True}
    routed = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": width, "limit": 7.0},
              "shared": {"ff": max(256, inner - top * width), "limit": 7.0}}
    layers = [{"type": "attention", "mixer": dict(mixer), "mlp": {"kind": "dense", "ff": inner} if i == 0 else routed}
              for i in range(n_layers)]
    return {"architecture": "Tatelorn", "vocab": vocab, "width": width, "max_positions": 1 << 16, "logit_scale": 0.5,
            "embedding": {"scale": width ** 0.5}, "norm": {"eps": 1e-6}, "layers": layers}


def nalasun_sizes(width, vocab=32768, experts=8, top=2):
    """Layer sizes in the manner of a real model of this width, eight layers: state-space layers of 2 widths in
    heads of 64 channels with a state of 128 rows and eight groups, attention with heads of 128 (a quarter of them
    key/value heads), delta-rule layers with heads of 128 x 128, every layer's mixer behind a convolution of four taps;
    `experts` experts of one width of which a row takes `top`, and a shared expert that brings a row's feed-forward
    weights to those of the dense layer of the Qwen2.5 design beside it."""
    heads = width // 128
    inner = (8 * width // 3 + 255) // 256 * 256
    routed = {"kind": "moe", "router": {"experts": experts, "top": top, "scale": 1.5}, "expert": {"ff": width},
              "shared": {"ff": max(256, inner - top * width)}}
    ssm = {"type": "mamba2", "mixer": {"heads": 2 * width // 64, "vdim": 64, "state": 128, "groups": 8, "conv": 4, "norm_groups": 8}}
    att = {"type": "attention", "mixer": {"heads": heads, "kv_heads": max(1, heads // 4), "dim": 128, "vdim": 128,
                                          "scale": 128 ** -0.5, "q_temp": {"coef": 0.5, "every": 256}}}
    delta = {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": max(1, heads // 2), "dim": 128, "vdim": 128, "conv": 4,
                                                "decay_rank": 64, "gate_rank": 64}}
    layers = [dict(layer, mlp=routed) for layer in (ssm, att, att, delta, ssm, att, delta, ssm)]
    return {"architecture": "Nalasun", "vocab": vocab, "width": width, "max_positions": 1 << 16, "norm": {"eps": 1e-6},
            "canon": {"taps": 3}, "layers": layers}


def fitatar_sizes(width, vocab=32768, experts=8, top=2):
    """Layer sizes in the manner of a real model of this width, eight layers: latent attention with heads of 128
    plain + 64 rotated numbers and 128 values, a latent of 512 and a query latent of half a width (the first keeps
    its latent, the fifth reads it), attention with heads of 128 for keys and values, a quarter of them kv heads;
    the first layer with a dense feed-forward of 4 widths, the others with `experts` experts of one width in four
    groups of which a row takes `top` from the best three, and a shared expert of 2 widths: a row passes as many
    feed-forward weights as in the Qwen2.5 layer beside it."""
    heads = width // 128
    rot = {"base": 1e6, "dims": 64, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}
    lat = {"heads": heads, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "q_rank": max(256, width // 2),
           "scale": 192 ** -0.5, "rot": rot}
    att = {"heads": heads, "kv_heads": max(1, heads // 4), "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
           "rot": {"base": 1e6, "dims": 128, "scaling": {"factor": 8.0}}}
    routed = {"kind": "moe", "router": {"experts": experts, "top": top, "groups": {"count": 4, "keep": 3}},
              "expert": {"ff": width}, "shared": {"ff": 2 * width}}
    layers = []
    for i in range(8):
        if i == 0:
            layers.append({"type": "latent_attention", "mixer": dict(lat), "mlp": {"kind": "dense", "ff": 4 * width}})
        elif i == 4:
            layers.append({"type": "latent_attention", "mixer": dict(lat, kv_from=0), "mlp": routed})
        else:
            layers.append({"type": "attention", "mixer": dict(att), "mlp": routed})
    return {"architecture": "Fitatar", "vocab": vocab, "width": width, "embedding": {"scale": 2.0}, "logit_softcap": 30.0,
            "norm": {"eps": 1e-6}, "layers": layers}


VECTOR_F32_FLOPS = 157.3e12      # the vector units' float32 peak, against which the recurrences' scans are priced


class AllOpsTimer:
    """Times every launching function of ``sonicboom_amd.ops`` between two events, summed by
    (function, what tells its calls apart: a product's matrix, the rows)."""

    SKIP = ("pack_weight", "read_bandwidth", "random_normal", "attention_row_tile", "attention_row_tiles",
            "attention_tall_ok", "attention_mfma_ok", "attention_decode_rope_ok", "gate_code", "reduce_resid_norm_ok",
            "attention_decode_pages_per_wave", "gemm_tile_shape", "gemm_few_rows_kernel", "mingru_chunk_rows",
            "loaded_paths", "check", "latent_attention_mfma_ok", "capped_attention_mfma_ok", "moe_max_top", "moe_plan",
            "time_conv_max_taps", "state_scan_limits", "state_scan_chunk_rows", "shared_attention_mfma_ok")
    INNER = ("attention_plain", "attention_decode_mfma", "attention_prefill_mfma", "latent_attention_plain",
             "latent_attention_mfma", "attention_capped_plain", "attention_capped_mfma",
             "moe_product_plain", "attention_shared_plain", "attention_shared_mfma",
             "head_mix")               # called by the dispatchers that are timed themselves

    def __init__(self):
        self.records, self._saved = [], {}

    def __enter__(self):
        import inspect

        import torch
        from sonicboom_amd import ops
        from sonicboom_amd.ops import kernels
        for name, fn in vars(kernels).items():
            if name.startswith("_") or name in self.SKIP or name in self.INNER or not inspect.isfunction(fn) \
                    or fn.__module__ != kernels.__name__:
                continue
            self._saved[name] = fn

            def timed(*args, _fn=fn, _name=name, **kw):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                out = _fn(*args, **kw)
                e1.record()
                if out is not None or not _name.startswith("gemm_bf16"):
                    label = _name
                    if _name.startswith("gemm"):
                        n, k = kw.get("packed_shape") or (args[1].shape[0], args[1].shape[-1])
                        label = f"{_name} {n}x{k}"
                    elif _name == "head_product":
                        label = f"{_name} {tuple(args[1].shape)}"
                    elif _name == "time_conv":
                        label = f"{_name} {args[1].shape[0]}"
                    elif _name in ("activate", "sigmoid_mul_", "rmsnorm_pair"):
                        label = f"{_name} {args[0].shape[-1]}"
                    elif _name == "moe_product":
                        label = f"{_name} {args[1].experts}x{args[1].n_out}x{args[1].n_in}{' gated' if args[1].gated else ''}"
                    self.records.append((label, e0, e1))
                return out
            setattr(ops, name, timed)
            setattr(kernels, name, timed)
        return self

    def __exit__(self, *exc):
        from sonicboom_amd import ops
        from sonicboom_amd.ops import kernels
        for name, fn in self._saved.items():
            setattr(ops, name, fn)
            setattr(kernels, name, fn)

    def totals(self):
        import torch
        torch.cuda.synchronize()
        out = {}
        for label, e0, e1 in self.records:
            us, n = out.get(label, (0.0, 0))
            out[label] = (us + e0.elapsed_time(e1) * 1e3, n + 1)
        return out


def design_roofline(label, us, calls, rows, depth, batch, width, cfgs):
    """(share of the roofline reached, what bounds it) for the kernels whose work is easy to count:
    per call, the bytes it must move over 8 TB/s against the flops over the dense bf16 peak."""
    per = us / calls * 1e-6
    peak_b, peak_f = PEAK_HBM_GBS * 1e9, PEAK_FLOPS["bf16"]
    decode = rows == batch
    keys = min(depth, cfgs["window"])
    H, rank, rot = cfgs["heads"], cfgs["rank"], cfgs["rot"]
    nbytes = flops = None
    if label.startswith("gemm"):
        n, k = (int(v) for v in label.split()[-1].split("x"))
        if n == cfgs["vocab"] and not decode:
            rows = 1                     # the head runs on the wanted rows only: the prompt's last
        nbytes, flops = 2 * n * k + 2 * rows * k + 4 * rows * (n // (2 if "gated" in label else 1)), 2 * rows * n * k
    elif label.startswith("rmsnorm") or label == "reduce_resid_norm":
        nbytes = rows * width * (4 + 2 + (8 if label == "reduce_resid_norm" else 0))
    elif label == "mingru_scan":
        nbytes = rows * cfgs["gru"] * (12 + 2)
    elif label == "activate":
        nbytes = rows * cfgs["ff"] * (4 + 2)
    elif label.startswith("activate "):
        nbytes = rows * int(label.split()[1]) * (4 + 2)
    elif label.startswith("sigmoid_mul_ "):
        nbytes = rows * int(label.split()[1]) * (2 + 2 + 4)
    elif label.startswith("rmsnorm_pair "):
        nbytes = rows * int(label.split()[1]) * (4 + 2 + (2 if int(label.split()[1]) == width else 0))
    elif label == "softcap_":
        nbytes = (rows if decode else 1) * cfgs["vocab"] * 8
    elif label == "latent_prepare":
        nbytes = rows * (4 * (H * 192 + rank + rot) + 2 * (H * (192 + rank) + rank + rot))
    elif label.startswith("head_product"):
        a, i, o = (int(v) for v in label.split("(")[1].rstrip(")").split(","))
        nbytes, flops = 2 * a * i * o + 2 * rows * a * (i + o), 2 * rows * a * i * o
    elif label == "latent_attention":
        pairs = batch * keys if decode else sum(min(t + 1, cfgs["window"]) for t in range(rows))
        flops = 2 * pairs * H * (2 * rank + rot)
        nbytes = (batch * keys if decode else rows) * 2 * (rank + rot) + 2 * rows * H * (2 * rank + rot)
    elif label in ("attention", "attention_decode_rope"):
        pairs = batch * depth if decode else rows * (rows + 1) // 2
        flops = 4 * pairs * H * 128
        nbytes = (batch * depth if decode else rows) * 2 * 2 * cfgs["kvw"] + 4 * rows * H * 128
    elif label == "rope_kv_store":
        nbytes = rows * (H * 128 + 2 * cfgs["kvw"]) * (4 + 2)
    elif label == "attention_capped":
        pairs = batch * depth if decode else rows * (rows + 1) // 2
        flops = 4 * pairs * H * 128
        nbytes = (batch * depth if decode else rows) * 2 * 2 * cfgs["kvw"] + 4 * rows * H * 128
    elif label == "headnorm_kv_store":
        nbytes = rows * (H * 128 + 2 * cfgs["kvw"]) * (4 + 2)
    elif label == "norm_add":
        nbytes = rows * width * (4 + 8 + 2)          # one slice of the sublayer's result at least
    elif label in ("cast", "embed_pos_norm"):
        nbytes = rows * width * (4 + 2)
    elif label.startswith("moe_product"):
        e, n, k = (int(v) for v in label.split()[1].split("x"))
        m = 2 if "gated" in label else 1
        pairs = rows * (cfgs["top"] if e > 1 else 1)
        nbytes = 2 * min(e, pairs) * m * n * k + 2 * pairs * (k + n)
        flops = 2 * pairs * m * n * k
    elif label.startswith("time_conv"):
        nbytes = rows * int(label.split()[1]) * (4 + 4)
    elif label == "ssd_scan":
        h, n, p = cfgs["ssd"]
        nbytes = rows * (4 * 3 * h * p + 4 * h) + (2 * batch * 4 * h * n * p if decode else 0)
        flops, peak_f = rows * h * n * p * 4, VECTOR_F32_FLOPS
    elif label == "delta_scan":
        h, d, e = cfgs["delta"]
        nbytes = rows * (4 * (2 * h * d + 3 * h * e) + 2 * h * e) + (2 * batch * 4 * h * d * e if decode else 0)
        flops, peak_f = rows * h * d * e * 7, VECTOR_F32_FLOPS
    elif label == "qk_rownorm_store":
        nbytes = rows * (H * 128 + cfgs["kvw"]) * (4 + 2) + rows * cfgs["kvw"] * 2
    elif label == "attention_shared":
        pairs = batch * depth if decode else rows * (rows + 1) // 2
        g = cfgs["kvw"] // 128
        flops = 2 * pairs * H * 128 * (1 + g)
        nbytes = (batch * depth if decode else rows) * 2 * 2 * cfgs["kvw"] + 2 * rows * H * 128 * 2
    if nbytes is None and flops is None:
        return None, ""
    tb, tf = (nbytes or 0) / peak_b, (flops or 0) / peak_f
    return max(tb, tf) / per, "bytes" if tb >= tf else "flops"


def design_comparison(a) -> int:
    import numpy as np
    import torch

    from sonicboom_amd.engine import DecoderModel, Engine, StepEntry

    rng = np.random.default_rng(0)
    out, table = {}, []
    for width in (int(v) for v in a.design_sizes.split(",")):
        sizes = {"rasizen": rasizen_sizes, "tatelorn": tatelorn_sizes, "nalasun": nalasun_sizes, "fitatar": fitatar_sizes,
                 "qwen2": qwen_sizes}
        for design, cfg in ((a.design, sizes[a.design](width)), (a.beside, sizes[a.beside](width))):
            model = DecoderModel.from_random(cfg, seed=0, dtype="bfloat16", device="cuda:0")
            heads = width // 128
            cfgs = {"heads": heads, "rank": 512, "rot": 64, "window": 4096 if design == "rasizen" else 1 << 30,
                    "gru": 2 * width, "ff": 4 * width, "kvw": max(1, heads // 4) * 128,
                    "vocab": cfg.get("vocab", cfg.get("vocab_size")), "top": 2,
                    "ssd": (2 * width // 64, 128, 64), "delta": (heads, 128, 128)}
            eng = Engine(model, (a.prompt + a.steps + a.warmup + 128) * (a.batch + 1), max_positions=0)
            prompt = [int(t) for t in rng.integers(0, cfg.get("vocab", cfg.get("vocab_size")), size=a.prompt)]

            def prefill_once(timer=None):
                slot = eng.alloc_slot()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                eng.step([StepEntry(slot, prompt, [a.prompt - 1])])
                torch.cuda.synchronize()
                dt = time.perf_counter() - t0
                eng.free_slot(slot)
                return dt
            for _ in range(2):
                prefill_once()
            prefill_s = statistics.median(prefill_once() for _ in range(5))
            with AllOpsTimer() as tm:
                prefill_once()
                pre_kernels = tm.totals()
            # decode: a batch at the prompt's depth, through the recorded step
            slots = [eng.alloc_slot() for _ in range(a.batch)]
            eng.step([StepEntry(s, prompt, ()) for s in slots])
            loop = eng.decode_loop()
            loop.start(slots, [1] * a.batch)
            for _ in range(a.warmup):
                loop.step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(a.steps):
                loop.step()
            torch.cuda.synchronize()
            step_s = (time.perf_counter() - t0) / a.steps
            with AllOpsTimer() as tm:
                eng.step([StepEntry(s, [1], [0]) for s in slots])
                dec_kernels = tm.totals()
            for s in slots:
                eng.free_slot(s)
            key = f"{design}_{width}"
            out[key] = {"prefill_tokens_per_s": round(a.prompt / prefill_s, 1), "decode_tokens_per_s": round(a.batch / step_s, 1),
                        "prefill_ms": round(prefill_s * 1e3, 3), "decode_step_ms": round(step_s * 1e3, 3),
                        "layers": len(model.order), "kernels": {}}
            for phase, totals, rows in (("prefill", pre_kernels, a.prompt), ("decode", dec_kernels, a.batch)):
                for label, (us, calls) in sorted(totals.items(), key=lambda kv: -kv[1][0]):
                    share, bound = design_roofline(label.replace("gemm_bf16_partial", "gemm").replace("gemm_bf16", "gemm"),
                                                   us, calls, rows, a.prompt, a.batch, width, cfgs)
                    out[key]["kernels"][f"{phase}: {label}"] = {"us": round(us, 1), "calls": calls,
                                                                "of_roofline": None if share is None else round(share, 3)}
                    table.append(f"| {key} | {phase} | {label} | {calls} | {us / calls:.1f} | "
                                 f"{'' if share is None else f'{share:.3f} ({bound})'} |")
            del eng, model, loop
            torch.cuda.empty_cache()
    print("| model | step | kernel | calls | us a call | of its roofline |\n|---|---|---|---|---|---|", file=sys.stderr)
    print("\n".join(table), file=sys.stderr)
    for key, v in out.items():
        print(f"RESULT {key} prefill_tokens_per_s={v['prefill_tokens_per_s']} decode_tokens_per_s={v['decode_tokens_per_s']} "
              f"prefill_ms={v['prefill_ms']} decode_step_ms={v['decode_step_ms']}", file=sys.stderr)
    print(json.dumps({"workload": "designs", "design": a.design, "beside": a.beside, "prompt": a.prompt, "batch": a.batch, "steps": a.steps, "dtype": "bf16",
                      "data": "synthetic", "models": out}))
    return 0


def result_lines(line, out=sys.stderr):
    """The run's metrics as ``RESULT key=value ...`` lines, one a metric, for tools that parse
    such lines rather than JSON; the engine clock the timed steps ran at is on every line."""
    clock = line.get("clock") or {}
    mhz = clock.get("median_mhz")
    tail = f" sclk_mhz={mhz if mhz is not None else 'unknown'}"
    print(f"RESULT metric=decode_tok_s batch={line['config']['global_batch']} value={line['value']} "
          f"ms_per_step={line['ms_per_step']} hbm_frac={line['roofline']['frac']}{tail}", file=out)
    pre = line.get("prefill")
    if pre:
        print(f"RESULT metric=prefill_tok_s tokens={pre['tokens']} value={pre['value']} ms={pre['ms']} "
              f"flops_frac={pre['frac']}{tail}", file=out)
    for name, v in (line.get("points") or {}).items():
        print(f"RESULT metric={name} value={v}{tail}", file=out)
    reuse = line.get("prefix_reuse")
    if reuse:
        print(f"RESULT metric=prefix_reuse_ttft_ms prefix={reuse['prefix']} new={reuse['new']} value={reuse['ttft_ms']} "
              f"without_reuse={reuse['ttft_ms_without_reuse']}{tail}", file=out)
    out.flush()


def median_of_runs(argv, runs):
    """``runs`` fresh processes of this program, one after the other (nothing here has touched
    the GPU); the line of the run whose value is the median, with every run's value."""
    import os
    import subprocess
    lines = []
    for i in range(runs):
        cmd = [sys.executable, os.path.abspath(__file__)] + argv + ["--runs", "1"]
        p = subprocess.run(cmd, stdout=subprocess.PIPE, text=True)
        if p.returncode != 0:
            print(f"bench.py: run {i + 1} of {runs} ended with {p.returncode}", file=sys.stderr)
            return p.returncode or 1
        found = [ln for ln in p.stdout.splitlines() if ln.startswith("{")]
        lines.append(json.loads(found[-1]))
        print(f"[bench] run {i + 1} of {runs}: {lines[-1]['value']} {lines[-1]['unit']}", file=sys.stderr, flush=True)
    order = sorted(range(runs), key=lambda i: lines[i]["value"])
    line = lines[order[(runs - 1) // 2]]
    line["process_runs"] = runs
    line["values_of_runs"] = [ln["value"] for ln in lines]
    if all("points" in ln for ln in lines):
        line["points"] = {k: statistics.median(ln["points"][k] for ln in lines) for k in line["points"]
                          if all(k in ln["points"] for ln in lines)}
    result_lines(line)
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
