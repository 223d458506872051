#!/usr/bin/env python3
"""Benchmark of the serving step on one MI355X: decode tokens/s at batch 8 (value), batch 1 and 64 (points),
and a 2,048-token prefill, for the Qwen2.5-0.5B layer sizes with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole batch, run by the scheduler (`Scheduler.step`): the engine's step function on
one token per request, greedy sampling on the device, the sampled tokens brought to the host (a server needs them
there to detect the end of a request) and the scheduler's bookkeeping.  The scheduler launches a step one step ahead
of the host, the token ids going from the sampler to the next step on the device (--no-lookahead waits for every
step's tokens first).  Prints one JSON line.  The default run adds to `points`: the same quantities at further
context lengths and batch sizes, in float32, at a head size of 96, at the 1.5B, 3B, 7B and 14B layer sizes, and the
mixed serving workload (see FURTHER_* below; --no-further-points skips them).
"""
import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_GBPS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "fp32": 157.3}

# Qwen2.5-0.5B layer sizes: the shape that the headline numbers are quoted on
QWEN25_05B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 24, "hidden_size": 896,
    "num_attention_heads": 14, "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 151936,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 32768,
    "use_sliding_window": False, "hidden_act": "silu", "torch_dtype": "bfloat16",
}
FULL_LAYERS = 24
PREFIX = 2048
NEW_TOKENS = 128
CONTEXT = 4096
PREFILL_TOKENS = 2048

# The larger Qwen2.5 layer sizes, for --shape and for the further points (the default run and its record stay the
# 0.5B ones): (config changes, layers of the model, prefix length of the decode runs)
OTHER_SHAPES = {
    "1.5b": (dict(hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960,
                  vocab_size=151936, tie_word_embeddings=True), 28, 2048),
    "3b": (dict(hidden_size=2048, num_attention_heads=16, num_key_value_heads=2, intermediate_size=11008,
                vocab_size=151936, tie_word_embeddings=True), 36, 4096),
    "7b": (dict(hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944,
                vocab_size=152064, tie_word_embeddings=False), 28, 4096),
    "14b": (dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, intermediate_size=13824,
                 vocab_size=152064, tie_word_embeddings=False), 48, 4096),
    # the 1.5B sizes with 16 heads of 96 instead of 12 of 128: the same products and attention FLOPs, another head size
    "1.5b-hd96": (dict(hidden_size=1536, num_attention_heads=16, num_key_value_heads=2, head_dim=96,
                       intermediate_size=8960, vocab_size=151936, tie_word_embeddings=True), 28, 2048),
}


SERVE_REQUESTS, SERVE_NEW_TOKENS, SERVE_CHUNK = 64, 256, 512


def serve_workload(engine, args, vocab: int, name: str = "Qwen2.5-0.5B") -> dict:
    """64 requests, submitted together, prompt lengths uniform in [128, 2048], 256 new tokens each (greedy, end token
    ignored), through the scheduler with prompts in portions of 512 tokens: total tokens a second, as a record."""
    import random

    import torch

    from easy_gpt.cpp_amd.engine.scheduler import Request, Scheduler, SchedulerConfig
    from easy_gpt.cpp_amd.sampling import SamplingParams

    rnd = random.Random(0)
    lo, hi = (int(v) for v in args.serve_prompts.split(","))
    lens = [rnd.randint(lo, hi) for _ in range(args.serve_requests)]
    g = torch.Generator().manual_seed(0)
    results = []
    for rep in range(2):                                       # the first pass warms up (graphs, library choices)
        sched = Scheduler(engine, SchedulerConfig(max_active=args.serve_requests, max_admit_per_step=8,
                                                  max_tokens_per_step=args.serve_budget,
                                                  prefill_chunk=min(SERVE_CHUNK, args.serve_budget)), eos_token_id=-1)
        if args.no_lookahead:
            sched.lookahead = False
        for i, n in enumerate(lens):
            sched.add(Request(f"s{rep}_{i}", torch.randint(0, vocab, (n,), generator=g).tolist(), SamplingParams(greedy=True),
                              max_new_tokens=SERVE_NEW_TOKENS, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while sched.has_work():
            sched.step()
        torch.cuda.synchronize()
        results.append((time.perf_counter() - t0, sched.stats))
        print(f"[bench] serve pass {rep}: {results[-1][0]:.2f} s, {sched.stats.steps} steps", file=sys.stderr, flush=True)
    sec, st = results[-1]
    total = sum(lens) + args.serve_requests * SERVE_NEW_TOKENS
    return {
        "metric": f"tokens/s through the scheduler, prompts and generated ({name})", "value": round(total / sec, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": st.steps, "ms_per_step": round(sec / st.steps * 1e3, 3),
        "higher_is_better": True, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "generated_per_s": round(args.serve_requests * SERVE_NEW_TOKENS / sec, 1), "seconds": round(sec, 3),
        "data": "synthetic: uniform-random token ids, random weights N(0, 0.02) from seed 0",
        "config": {"model": f"{name} layer sizes", "requests": args.serve_requests, "prompt_tokens": sum(lens),
                   "new_tokens_each": SERVE_NEW_TOKENS, "prefill_chunk": min(SERVE_CHUNK, args.serve_budget),
                   "max_tokens_per_step": args.serve_budget,
                   "preemptions": st.preemptions, "steps_launched_ahead": st.steps_ahead, "sampling": "greedy"},
    }


# What the default run measures beside its record (all layers of each model, random weights drawn on the GPU):
# at the 0.5B sizes (the record's model) prefixes of 8k and 32k tokens with a prefill of that length, and batches of
# 128 and 256 behind 2k and 8k;
FURTHER_CONTEXTS = (("ctx8k", 8192, (256, 128, 64, 8, 1)), ("ctx32k", 32640, (64, 8, 1)))
FURTHER_BATCHES = (128, 256)
# at other layer sizes a 2,048-token prefill and decode runs (label, shape, dtype, ((prefix, batches), ...)); the
# first prefix is the shape's own and its points are named without it
FURTHER_SHAPES = (
    ("fp32", "0.5b", "float32", ((2048, (8,)),)),
    ("hd96", "1.5b-hd96", "bfloat16", ()),
    ("q1p5b", "1.5b", "bfloat16", ((2048, (1, 8, 64)),)),
    ("q3b", "3b", "bfloat16", ((4096, (1, 8, 64)),)),
    ("q7b", "7b", "bfloat16", ((4096, (1, 8, 64)), (2048, (128, 256)), (8192, (128,)))),
    ("q14b", "14b", "bfloat16", ((4096, (1, 8, 64)),)),
)
FURTHER_WARMUP, FURTHER_STEPS = 4, 32
FILL_TOKENS = 65536         # prompts are put into the cache several to a step, up to this many tokens


def remove_folder(path: str) -> None:
    for f in os.listdir(path):
        os.remove(os.path.join(path, f))
    os.rmdir(path)


def shape_config(shape: str) -> tuple[dict, int]:
    if shape == "0.5b":
        return dict(QWEN25_05B), PREFIX
    changes, n_layers, prefix = OTHER_SHAPES[shape]
    return dict(QWEN25_05B, **changes, num_hidden_layers=n_layers), prefix


def further_points(args, model_dir: str, cfg: dict, g, points: dict) -> None:
    """The points beside the record, tokens a second each, into the flat dict `points` (what was measured before a
    failure stays there)."""
    import torch

    from easy_gpt.cpp_amd.engine import Engine
    from easy_gpt.cpp_amd.engine.engine import load_random_model
    from easy_gpt.cpp_amd.sampling import Sampler

    page = args.page_size
    warm, steps = FURTHER_WARMUP, FURTHER_STEPS

    def rate(name, tokens, sec, per_step=True):
        points[name] = round(tokens / sec, 1)
        print(f"[bench] {name}: {tokens / sec:.1f} tok/s, {sec / (steps if per_step else 1) * 1e3:.3f} ms",
              file=sys.stderr, flush=True)

    def decode_runs(engine, sampler, vocab, label, prefix, batches):
        """Prefixes of `prefix` tokens for the largest batch, filled once and decoded as each of `batches`
        (largest first: every run's first requests have decoded in the runs before it)."""
        batches = sorted(batches, reverse=True)
        rids, last = fill_requests(engine, sampler, vocab, prefix, batches[0], g)
        for b in batches:
            sub = last[:b]
            sec = decode_seconds(engine, sampler, rids[:b], sub, warm, steps, args.no_lookahead)[0]
            rate(f"{label}_decode_b{b}" if label else f"decode_b{b}", b * steps, sec)
            last[:b] = sub
        for rid in rids:
            engine.finish(rid)

    def room(prefix, batches):        # tokens the runs of one prefix hold: every run decodes the first requests further
        return max(batches) * (-(-(prefix + len(batches) * (warm + steps) + 1) // page) * page)

    # ---- the record's model: further contexts and batches
    tokens = max([room(p, b) for _, p, b in FURTHER_CONTEXTS] + [room(PREFIX, FURTHER_BATCHES)])
    engine = Engine.from_dir(model_dir, dtype=args.dtype, device="cuda:0", page_size=page,
                             max_tokens=tokens + FILL_TOKENS, max_requests=max(FURTHER_BATCHES) + 2,
                             tune_products=not args.no_tune)
    sampler = Sampler(engine.device)
    decode_runs(engine, sampler, cfg["vocab_size"], "", PREFIX, FURTHER_BATCHES)
    for label, prefix, batches in FURTHER_CONTEXTS:
        rate(f"{label}_prefill", prefix, prefill_seconds(engine, cfg["vocab_size"], prefix, g, reps=3), per_step=False)
        if label == "ctx32k":
            # the same prompt as the scheduler feeds it under a budget of 512 tokens a step
            rate(f"{label}_prefill_in_512s", prefix,
                 prefill_in_portions_seconds(engine, cfg["vocab_size"], prefix, SERVE_CHUNK, g), per_step=False)
        decode_runs(engine, sampler, cfg["vocab_size"], label, prefix, batches)
    # ---- the mixed serving workload through the scheduler (what `--serve` prints)
    serve = serve_workload(engine, args, cfg["vocab_size"])
    points["serve_tokens_per_s"] = serve["value"]
    print(f"[bench] serve: {serve['value']} tok/s (prompts and generated), {serve['steps']} steps", file=sys.stderr, flush=True)
    del engine, sampler
    torch.cuda.empty_cache()

    # ---- other layer sizes, head sizes and float32
    for label, shape, dtype, runs in FURTHER_SHAPES:
        other, _ = shape_config(shape)
        t0 = time.time()
        model = load_random_model(other, seed=0, dtype=dtype, device="cuda:0")
        tokens = max([room(p, b) for p, b in runs] + [0]) + max(FILL_TOKENS, PREFILL_TOKENS)
        engine = Engine(model, page_size=page, max_tokens=tokens, max_requests=max([max(b) for _, b in runs] + [1]) + 2,
                        tune_products=not args.no_tune)
        sampler = Sampler(engine.device)
        print(f"[bench] {label} model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
        rate(f"{label}_prefill", PREFILL_TOKENS, prefill_seconds(engine, other["vocab_size"], PREFILL_TOKENS, g, reps=5),
             per_step=False)
        for i, (prefix, batches) in enumerate(runs):
            decode_runs(engine, sampler, other["vocab_size"], label if i == 0 else f"{label}_ctx{prefix // 1024}k",
                        prefix, batches)
        del engine, sampler, model
        torch.cuda.empty_cache()


def prefill_seconds(engine, vocab: int, tokens: int, g, reps: int = 10) -> float:
    """One prompt of `tokens` tokens in one step, logits at its last place: the median of `reps` after one warm-up."""
    import torch

    from easy_gpt.cpp_amd.engine import StepEntry

    ids = torch.randint(0, vocab, (tokens,), generator=g).tolist()
    times = []
    for rep in range(reps + 1):
        engine.add_request("prefill")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([StepEntry("prefill", ids, [tokens - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.finish("prefill")
    return sorted(times[1:])[len(times[1:]) // 2]


def prefill_in_portions_seconds(engine, vocab: int, tokens: int, portion: int, g, reps: int = 2) -> float:
    """One prompt of `tokens` tokens in steps of `portion` tokens each, as the scheduler feeds a long prompt under a token
    budget; logits at its last place: the fastest of `reps` passes after one warm-up."""
    import torch

    from easy_gpt.cpp_amd.engine import StepEntry

    ids = torch.randint(0, vocab, (tokens,), generator=g).tolist()
    times = []
    for rep in range(reps + 1):
        engine.add_request("prefill")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for pos in range(0, tokens, portion):
            n = min(portion, tokens - pos)
            engine.step([StepEntry("prefill", ids[pos : pos + n], [n - 1] if pos + n == tokens else [])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.finish("prefill")
    return min(times[1:])


def fill_requests(engine, sampler, vocab: int, prefix: int, batch: int, g):
    """`batch` requests with prefixes of `prefix` random tokens in the cache (untimed, several prompts to a step); their
    ids and next tokens."""
    import torch

    from easy_gpt.cpp_amd.engine import StepEntry
    from easy_gpt.cpp_amd.sampling import SamplingParams

    greedy = SamplingParams(greedy=True)
    rids, last = [f"d{i}" for i in range(batch)], []
    per_step = max(1, FILL_TOKENS // prefix)
    from easy_gpt.cpp_amd import kernels

    tuned = kernels.library_tuning
    if tuned and per_step > 1:
        kernels.tune_library_products(False)       # (no measurements for the shapes of these untimed steps)
    for first in range(0, batch, per_step):
        group = rids[first : first + per_step]
        entries = []
        for rid in group:
            engine.add_request(rid)
            entries.append(StepEntry(rid, torch.randint(0, vocab, (prefix,), generator=g).tolist(), [prefix - 1]))
        out = engine.step(entries)
        last.extend(sampler.sample(out, [greedy] * len(group), [0] * len(group), [0] * len(group)))
    if tuned and per_step > 1:
        kernels.tune_library_products(True)
    return rids, last


def scheduler_decode_seconds(engine, vocab: int, prefix: int, batch: int, warmup: int, steps: int, g,
                             no_lookahead: bool = False) -> tuple[float, float]:
    """Seconds of `steps` decode steps of `batch` requests through `Scheduler.step` after `warmup` untimed ones, and the
    median time between two steps' returns.  The requests are admitted together and their prompts (the prefixes) run
    in one step, so that all of them decode from the same context length on."""
    import torch

    from easy_gpt.cpp_amd.engine.scheduler import Request, Scheduler, SchedulerConfig
    from easy_gpt.cpp_amd.sampling import SamplingParams

    sched = Scheduler(engine, SchedulerConfig(max_active=batch, max_admit_per_step=batch,
                                              max_tokens_per_step=batch * prefix, prefill_chunk=prefix), eos_token_id=-1)
    if no_lookahead:
        sched.lookahead = False
    for i in range(batch):
        sched.add(Request(f"d{i}", torch.randint(0, vocab, (prefix,), generator=g).tolist(), SamplingParams(greedy=True),
                          max_new_tokens=warmup + steps + 8, ignore_eos=True))
    from easy_gpt.cpp_amd import kernels

    tuned = kernels.library_tuning
    if tuned:
        kernels.tune_library_products(False)       # (no measurements for the shapes of this one untimed step)
    sched.step()                                   # the prompts
    if tuned:
        kernels.tune_library_products(True)
    assert len(sched.running) == batch and all(len(r.output) == 1 for r in sched.running)
    for _ in range(warmup):
        sched.step()
    arrivals = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        sched.step()                               # returns when the step's tokens are on the host
        arrivals.append(time.perf_counter())
    torch.cuda.synchronize()                       # (with the step that was launched ahead of the last return)
    sec = time.perf_counter() - t0
    assert sched.stats.generated == batch * (1 + warmup + steps) and not sched.stats.preemptions
    for r in list(sched.running):
        engine.finish(r.request_id)
    between = sorted(b - a for a, b in zip(arrivals, arrivals[1:]))
    return sec, (between[len(between) // 2] if between else sec / steps)


def decode_seconds(engine, sampler, rids, last, warmup: int, steps: int, no_lookahead: bool = False) -> tuple[float, float]:
    """Seconds of `steps` decode steps of the requests `rids` after `warmup` untimed ones, and the median time between
    the arrivals of two steps' tokens on the host.

    As the scheduler decodes: a step is launched before the host has seen the tokens of the step before it (its
    token ids go from the sampler to the step on the device), then the host waits for that earlier step's tokens.
    Every step's tokens reach the host inside the timed region."""
    import torch

    from easy_gpt.cpp_amd.engine import StepEntry
    from easy_gpt.cpp_amd.sampling import SamplingParams

    batch = len(rids)
    params, serials = [SamplingParams(greedy=True)] * batch, list(range(batch))

    def launch(pending, n):
        if pending is None or no_lookahead:
            tokens = last if pending is None else pending.result()
            logits = engine.step([StepEntry(rid, [tok], [0]) for rid, tok in zip(rids, tokens)])
        else:
            logits = engine.step_decode_ahead(rids, pending.device)
        return sampler.sample_async(logits, params, serials, [n] * batch)

    pending = None
    for i in range(warmup):
        nxt = launch(pending, i)
        if pending is not None:
            pending.result()
        pending = nxt
    if pending is not None:
        last[:] = pending.result()
    pending = None
    arrivals = []                                  # when each step's tokens reached the host
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        nxt = launch(pending, warmup + i)
        if pending is not None:
            pending.result()                       # the tokens of the step before, on the host
            arrivals.append(time.perf_counter())
        pending = nxt
    last[:] = pending.result()
    arrivals.append(time.perf_counter())
    torch.cuda.synchronize()
    sec = time.perf_counter() - t0
    between = sorted(b - a for a, b in zip(arrivals, arrivals[1:]))
    return sec, (between[len(between) // 2] if between else sec / steps)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=NEW_TOKENS - 16)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--shape", default="0.5b", choices=["0.5b"] + sorted(OTHER_SHAPES),
                    help="layer sizes: Qwen2.5-0.5B (the default, which the headline numbers are quoted on) or a larger one")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prefix", type=int, default=None,
                    help="tokens each request holds before decoding starts (default: 2,048; 4,096 at the 7B sizes)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-tune", action="store_true",
                    help="take the library's first choice for its matrix products instead of the measured one")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill measurements")
    ap.add_argument("--no-further-points", action="store_true",
                    help="skip the points at 8k and 32k prefixes and at the 1.5B and 7B layer sizes")
    ap.add_argument("--prefill-only", action="store_true", help="only the prefill (for profiling)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="tokens of the prompt that --prefill-only feeds in one step (the record's prefill is 2,048)")
    ap.add_argument("--serve-budget", type=int, default=2048, help="with --serve: the token budget of one step")
    ap.add_argument("--serve-requests", type=int, default=SERVE_REQUESTS, help="with --serve: requests, submitted together")
    ap.add_argument("--serve-prompts", default="128,2048", help="with --serve: prompt lengths are uniform in LOW,HIGH")
    ap.add_argument("--serve", action="store_true",
                    help="instead of fixed batches: 64 requests with prompts of 128 to 2,048 tokens and 256 new tokens "
                         "each through the scheduler, prompts in portions of 512 (the mixed serving workload)")
    ap.add_argument("--no-lookahead", action="store_true",
                    help="wait for a step's tokens on the host before the next step is launched (the scheduler with --serve, "
                         "the decode loop otherwise)")
    ap.add_argument("--direct-loop", action="store_true",
                    help="decode with the engine's step function in a loop of the benchmark's own instead of Scheduler.step")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path, --gpus {args.gpus} is not run")
        return 2
    global FULL_LAYERS, PREFIX, CONTEXT
    base, name = dict(QWEN25_05B), "Qwen2.5-0.5B"
    if args.shape != "0.5b":
        changes, FULL_LAYERS, PREFIX = OTHER_SHAPES[args.shape]
        base.update(changes)
        CONTEXT = PREFIX + 2048
        name = f"Qwen2.5-{args.shape.upper()}"
    if args.prefix is not None:
        if args.prefix < 1 or args.prefix + NEW_TOKENS > base["max_position_embeddings"]:
            print(f"--prefix must be between 1 and {base['max_position_embeddings'] - NEW_TOKENS}")
            return 2
        PREFIX, CONTEXT = args.prefix, args.prefix + 2048
    if args.layers is None:
        args.layers = FULL_LAYERS
    if args.warmup + args.steps > CONTEXT - PREFIX:
        print(f"--warmup + --steps must stay within the context of {CONTEXT} after a prefix of {PREFIX}")
        return 2

    import torch

    from easy_gpt.cpp_amd.engine import Engine, StepEntry
    from easy_gpt.cpp_amd.sampling import Sampler, SamplingParams
    from easy_gpt.cpp_amd.weights import write_random_model

    cfg = dict(base, num_hidden_layers=args.layers)
    dtype_key = "bf16" if args.dtype == "bfloat16" else "fp32"
    elem = 2 if args.dtype == "bfloat16" else 4
    h, nq, nkv, inter, vocab = (cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"],
                                cfg["intermediate_size"], cfg["vocab_size"])
    hd = cfg.get("head_dim", h // nq)
    layers = args.layers
    page_size = args.page_size
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})
    max_batch = max(batches)

    t_setup = time.time()
    tmp = tempfile.mkdtemp(prefix="egpt_bench_")
    write_random_model(tmp, cfg, seed=0, dtype=torch.bfloat16 if args.dtype == "bfloat16" else torch.float32)
    new_tokens = max(NEW_TOKENS, args.warmup + args.steps)        # a longer run than the default decodes further
    tokens_per_request = -(-(PREFIX + new_tokens) // page_size) * page_size
    if args.serve:
        longest = int(args.serve_prompts.split(",")[1])
        max_batch, tokens_per_request = args.serve_requests, -(-(longest + SERVE_NEW_TOKENS) // page_size) * page_size
    engine = Engine.from_dir(tmp, dtype=args.dtype, device="cuda:0", page_size=page_size,
                             max_tokens=max_batch * tokens_per_request + max(PREFILL_TOKENS, args.prefill_tokens),
                             max_requests=max_batch + 1, tune_products=not args.no_tune)
    sampler = Sampler(engine.device)
    g = torch.Generator().manual_seed(0)
    print(f"[bench] model ready in {time.time() - t_setup:.1f} s", file=sys.stderr, flush=True)

    if args.serve:
        remove_folder(tmp)
        print(json.dumps(serve_workload(engine, args, vocab, name)), flush=True)
        return 0
    # the further points stand beside the default run's record only
    further = not (args.no_points or args.no_further_points or args.shape != "0.5b" or args.prefix is not None
                   or args.layers != FULL_LAYERS or args.dtype != "bfloat16" or args.batch != 8)

    # per-step work of the model, for the rooflines
    layer_weights = (h * (nq + 2 * nkv) * hd + (nq + 2 * nkv) * hd + nq * hd * h + 3 * h * inter + 2 * h) * elem
    weight_bytes = layers * layer_weights + vocab * h * elem + h * elem          # output matrix read once, tied or not
    kv_bytes_per_token = layers * 2 * nkv * hd * elem

    def prefill_flops(t: int) -> float:
        linear = 2.0 * t * (h * (nq + 2 * nkv) * hd + nq * hd * h + 3 * h * inter)
        attention = 2.0 * t * (t + 1) * hd * nq                                  # QK^T and PV over the causal half
        return layers * (linear + attention) + 2.0 * vocab * h                   # logits at the last place only

    # ---------------------------------------------------------------- prefill of 2,048 tokens, one request, one step
    prefill = None
    if not args.no_points or args.prefill_only:
        n_prompt = args.prefill_tokens if args.prefill_only else PREFILL_TOKENS
        sec = prefill_seconds(engine, vocab, n_prompt, g, reps=10 if n_prompt <= 8192 else 3)
        prefill = {"value": round(n_prompt / sec, 1), "tokens": n_prompt, "ms": round(sec * 1e3, 3),
                   "frac": round(prefill_flops(n_prompt) / sec / (PEAK_TFLOPS[dtype_key] * 1e12), 5)}
        print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)
    if args.prefill_only:
        print(json.dumps({"metric": f"prefill tok/s at {n_prompt:,} tokens ({name})", "prefill": prefill}), flush=True)
        remove_folder(tmp)
        return 0

    # ---------------------------------------------------------------- decoding at each batch size
    def decode_run(batch: int, warmup: int, steps: int):
        if args.direct_loop:
            rids, last = fill_requests(engine, sampler, vocab, PREFIX, batch, g)
            sec, medians[batch] = decode_seconds(engine, sampler, rids, last, warmup, steps, args.no_lookahead)
            for rid in rids:
                engine.finish(rid)
        else:
            sec, medians[batch] = scheduler_decode_seconds(engine, vocab, PREFIX, batch, warmup, steps, g, args.no_lookahead)
        mean_ctx = PREFIX + warmup + (steps + 1) / 2.0
        step_bytes = weight_bytes + batch * mean_ctx * kv_bytes_per_token
        return sec, step_bytes

    results, medians = {}, {}
    for b in batches:
        sec, step_bytes = decode_run(b, args.warmup, args.steps)
        results[b] = (sec, step_bytes)
        print(f"[bench] decode batch {b}: {b * args.steps / sec:.1f} tok/s, {sec / args.steps * 1e3:.3f} ms/step, "
              f"{step_bytes / (sec / args.steps) / 1e9:.1f} GB/s", file=sys.stderr, flush=True)

    sec, step_bytes = results[args.batch]
    achieved = step_bytes / (sec / args.steps) / 1e9
    line = {
        "metric": f"decode tok/s at batch {args.batch} ({name}, prefix {PREFIX})",
        "value": round(args.batch * args.steps / sec, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(sec / args.steps * 1e3, 4),
        "ms_per_step_median": round(medians[args.batch] * 1e3, 4),      # between the arrivals of two steps' tokens on the host
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_key,
        "data": "synthetic: uniform-random token ids, random weights N(0, 0.02) from seed 0",
        "config": {
            "model": f"{name} layer sizes", "layers": layers, "layers_of_model": FULL_LAYERS, "hidden": h,
            "heads": nq, "kv_heads": nkv, "head_dim": hd, "intermediate": inter, "vocab": vocab, "tied": bool(cfg["tie_word_embeddings"]),
            "global_batch": args.batch, "seq_len": CONTEXT, "prefix_len": PREFIX, "new_tokens": new_tokens,
            "page_size": page_size, "rope_theta": cfg["rope_theta"], "rms_norm_eps": cfg["rms_norm_eps"],
            "sampling": "greedy", "library_products": "first choice" if args.no_tune else "measured",
            "parallelism": "single GPU, decode steps run by " + ("a loop over Engine.step" if args.direct_loop else "Scheduler.step"),
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 5)},
    }
    if prefill is not None:
        line["prefill"] = prefill
    points = {f"decode_b{b}": round(b * args.steps / results[b][0], 1) for b in batches if b != args.batch}
    del engine
    if further:
        # (the record above stands whatever happens to the points beside it: a failure there is named in the line)
        try:
            further_points(args, tmp, cfg, g, points)
        except Exception as e:      # noqa: BLE001
            line["points_error"] = f"{type(e).__name__}: {str(e)[:200]}"
            print(f"[bench] the further points stopped: {line['points_error']}", file=sys.stderr, flush=True)
    remove_folder(tmp)
    if points:
        line["points"] = points
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
