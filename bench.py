#!/usr/bin/env python3
"""Benchmark of the serving step on one MI355X: decode tokens/s at batch 8 (value), batch 1 and 64 (points),
and a 2,048-token prefill, for the Qwen2.5-0.5B layer sizes with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole batch: the engine's step function on one token per request, greedy
sampling on the device, and the sampled tokens brought to the host (a server needs them there to detect the
end of a request).  Steps are launched as the scheduler launches them: one step ahead of the host, the token ids
going from the sampler to the next step on the device (--no-lookahead waits for every step's tokens first).
Prints one JSON line.  The default run adds the same quantities at further context lengths and at the 1.5B and 7B
layer sizes to `points` (see FURTHER_CONTEXTS below; --no-further-points skips them).
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

# The larger Qwen2.5 layer sizes, for --shape (the default run and its record stay the 0.5B ones):
# (config changes, layers of the model, prefix length of the decode runs)
OTHER_SHAPES = {
    "1.5b": (dict(hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960,
                  vocab_size=151936, tie_word_embeddings=True), 28, 2048),
    "7b": (dict(hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944,
                vocab_size=152064, tie_word_embeddings=False), 28, 4096),
}


SERVE_REQUESTS, SERVE_NEW_TOKENS, SERVE_CHUNK = 64, 256, 512


def serve_workload(engine, name: str, args, vocab: int) -> int:
    """64 requests, submitted together, prompt lengths uniform in [128, 2048], 256 new tokens each (greedy, end token
    ignored), through the scheduler with prompts in portions of 512 tokens: total tokens a second."""
    import random

    import torch

    from easy_gpt.cpp_amd.engine.scheduler import Request, Scheduler, SchedulerConfig
    from easy_gpt.cpp_amd.sampling import SamplingParams

    rnd = random.Random(0)
    lens = [rnd.randint(128, 2048) for _ in range(SERVE_REQUESTS)]
    g = torch.Generator().manual_seed(0)
    results = []
    for rep in range(2):                                       # the first pass warms up (graphs, library choices)
        sched = Scheduler(engine, SchedulerConfig(max_active=SERVE_REQUESTS, max_admit_per_step=8,
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
    total = sum(lens) + SERVE_REQUESTS * SERVE_NEW_TOKENS
    print(json.dumps({
        "metric": f"tokens/s through the scheduler, prompts and generated ({name})", "value": round(total / sec, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": st.steps, "ms_per_step": round(sec / st.steps * 1e3, 3),
        "higher_is_better": True, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "generated_per_s": round(SERVE_REQUESTS * SERVE_NEW_TOKENS / sec, 1), "seconds": round(sec, 3),
        "data": "synthetic: uniform-random token ids, random weights N(0, 0.02) from seed 0",
        "config": {"model": f"{name} layer sizes", "requests": SERVE_REQUESTS, "prompt_tokens": sum(lens),
                   "new_tokens_each": SERVE_NEW_TOKENS, "prefill_chunk": min(SERVE_CHUNK, args.serve_budget),
                   "max_tokens_per_step": args.serve_budget,
                   "preemptions": st.preemptions, "steps_launched_ahead": st.steps_ahead, "sampling": "greedy"},
    }), flush=True)
    return 0


def link_floor() -> int:
    """What a chain of dependent kernels costs apart from its work: graphs of 125 links that each do next to nothing
    (every thread one load of what the link before wrote, `trips - 1` further loads that depend on each other, one
    store), replayed; microseconds per link by number of workgroups and of dependent round trips to memory, with
    the further loads near (within the few kilobytes that the link before wrote: L2) or far (anywhere in 1 GiB: HBM).
    Then the same chain with flags in memory in place of kernel boundaries."""
    import torch

    from easy_gpt.cpp_amd import kernels

    k = kernels.backend()
    links, table = 125, {}
    far = 1 << 28                                       # floats: dependent loads that range over 1 GiB miss every cache
    far_a, far_b = torch.zeros(far, device="cuda"), torch.zeros(far, device="cuda")
    for where in ("near", "far"):
        for groups in (1, 64, 256, 1024, 4096):
            n = groups * 256
            if where == "near":
                a, b = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
            else:
                a, b = far_a, far_b
            for trips in (1, 2, 3, 5):
                def chain():
                    src, dst = a, b
                    for _ in range(links):
                        k.probe_link(src, dst, trips, n)
                        src, dst = dst, src
                chain()
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    chain()
                for _ in range(3):
                    graph.replay()
                torch.cuda.synchronize()
                reps = 20
                t0 = time.perf_counter()
                for _ in range(reps):
                    graph.replay()
                torch.cuda.synchronize()
                key = f"{where}_wg{groups}_trips{trips}"
                table[key] = round((time.perf_counter() - t0) / reps / links * 1e6, 3)
                print(f"[bench] {groups:5d} workgroups, {trips} dependent loads ({where}): {table[key]:.2f} us a link",
                      file=sys.stderr, flush=True)
    # The same chain with its links handed over through flags in memory: the links alternate between two streams of
    # one graph (two hardware queues), so a link is resident and waiting while the link before runs; its first thread
    # polls the flag past the caches, then all threads read what the link before wrote past the caches.
    del far_a, far_b
    side = torch.cuda.Stream()
    main = torch.cuda.Stream()
    links = 124
    for groups in (1, 64, 128, 256, 512):
        n = groups * 256
        a, b = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
        flags = torch.zeros(links, dtype=torch.int32, device="cuda")
        gave_up = torch.zeros(1, dtype=torch.int32, device="cuda")

        def chain():
            first = torch.cuda.current_stream()
            flags.zero_()
            a.zero_()
            side.wait_stream(first)
            src, dst = a, b
            for link in range(links):
                k.probe_handoff(src, dst, n, flags[link - 1 : link] if link else None, groups, flags[link : link + 1], gave_up,
                                first if link % 2 == 0 else side)
                src, dst = dst, src
            first.wait_stream(side)
            return src

        with torch.cuda.stream(main):
            chain()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=main):
                result = chain()
            for _ in range(3):
                graph.replay()
            torch.cuda.synchronize()
            reps = 20
            t0 = time.perf_counter()
            for _ in range(reps):
                graph.replay()
            torch.cuda.synchronize()
            us = (time.perf_counter() - t0) / reps / links * 1e6
        right = float(result.min()) == links and float(result.max()) == links and int(gave_up.item()) == 0
        table[f"handoff_wg{groups}"] = round(us, 3)
        print(f"[bench] {groups:5d} workgroups, handed over through a flag, links on two streams in turn: {us:.2f} us a link"
              f"{'' if right else ' (WRONG RESULT or a wait ran out)'}", file=sys.stderr, flush=True)
    print(json.dumps({"metric": "microseconds per link of a replayed graph of 125 dependent near-empty kernels",
                      "unit": "us", "links": 125, "table": table}), flush=True)
    return 0


def anatomy(args, base: dict, name: str) -> int:
    """What the kernels of one decode step spend their time on, seen from inside: the step is replayed from its graph
    with the library's trace build, whose product and decode-attention kernels write the wall clock of four phases per
    workgroup (start; operands staged or queries made; matrix products done; results stored).  Per kind of kernel,
    medians over the layers, in microseconds: the gap from the end of the kernel before to the first workgroup's
    start, the ramp until the last workgroup has started, the phases of the median workgroup, and the span from the
    first start to the last end.  Timestamps cost a little: the step takes a few per cent longer than in bench runs."""
    import statistics
    import tempfile

    import torch

    from easy_gpt.cpp_amd import kernels
    from easy_gpt.cpp_amd.engine import Engine, StepEntry
    from easy_gpt.cpp_amd.kernels.hip import HipKernels
    from easy_gpt.cpp_amd.weights import write_random_model

    k = HipKernels(trace=True)
    kernels.use_backend(k)
    batch, prefix = args.batch, PREFIX
    tmp = tempfile.mkdtemp(prefix="egpt_bench_")
    write_random_model(tmp, base, seed=0, dtype=torch.bfloat16)
    engine = Engine.from_dir(tmp, dtype="bfloat16", device="cuda:0", page_size=args.page_size,
                             max_tokens=batch * (prefix + 256) + 2048, max_requests=batch + 1)
    g = torch.Generator().manual_seed(0)
    rids = [f"d{i}" for i in range(batch)]
    for rid in rids:
        engine.add_request(rid)
        engine.step([StepEntry(rid, torch.randint(0, base["vocab_size"], (prefix,), generator=g).tolist(), [prefix - 1])])
    for i in range(6):
        engine.step([StepEntry(rid, [5 + i], [0]) for rid in rids])
    buf = k.trace_attach()
    for rep in range(3):
        buf.zero_()
        torch.cuda.synchronize()
        engine.step([StepEntry(rid, [77 + rep], [0]) for rid in rids])
        torch.cuda.synchronize()
    launches = k.trace_records(buf)
    kinds: dict = {}
    prev_end, rates = None, []
    for launch in launches:
        wgs = [w["us"] for w in launch["workgroups"]]
        first, last_start = min(w[0] for w in wgs), max(w[0] for w in wgs)
        end = max(w[3] for w in wgs)
        med = lambda j: statistics.median(w[j] - w[0] for w in wgs if w[j]) if any(w[j] for w in wgs) else None
        key = (k.TRACED_KERNELS.get(launch["kernel"], str(launch["kernel"])), len(wgs))
        kinds.setdefault(key, []).append((first - prev_end if prev_end is not None else 0.0, last_start - first,
                                          med(1), med(2), med(3), end - first))
        prev_end = end
        for w in launch["workgroups"]:
            if w["us"][3] > w["us"][0] + 0.5:
                rates.append(((w["cycles"][3] - w["cycles"][0]) & 0xffffffff) / (w["us"][3] - w["us"][0]))
    rows = []
    print(f"{'kernel':46s} {'wgs':>5s} {'calls':>5s} | {'gap':>5s} {'ramp':>5s} {'staged':>6s} {'mfma':>5s} {'stored':>6s} {'span':>5s}",
          file=sys.stderr)
    for (kind, n_wgs), v in kinds.items():
        m = [None if any(x[i] is None for x in v) else round(statistics.median(x[i] for x in v), 2) for i in range(6)]
        rows.append({"kernel": kind, "workgroups": n_wgs, "calls": len(v), "gap": m[0], "ramp": m[1], "staged": m[2],
                     "mfma": m[3], "stored": m[4], "span": m[5]})
        f = lambda x: "    -" if x is None else f"{x:5.2f}"
        print(f"{kind:46s} {n_wgs:5d} {len(v):5d} | {f(m[0])} {f(m[1])} {f(m[2]):>6s} {f(m[3])} {f(m[4]):>6s} {f(m[5])}", file=sys.stderr)
    marks = [w["us"] for launch in launches for w in launch["workgroups"]]
    total = max(w[3] for w in marks) - min(w[0] for w in marks)
    rates.sort()
    print(json.dumps({"metric": f"anatomy of a decode step at batch {batch} ({name}, prefix {prefix}), microseconds",
                      "first_start_to_last_end_us": round(total, 1), "shader_clock_mhz": round(rates[len(rates) // 2]),
                      "kernels": rows}), flush=True)
    return 0


# The further points of the default run, beside decode_b1 and decode_b64.  Each name starts with what differs from the
# headline shape, then the quantity as there (decode_b<batch>: decoded tokens a second; prefill: tokens a second):
#   ctx8k_, ctx32k_  the 0.5B sizes with prefixes of 8,192 and 32,640 tokens (prefill: one prompt of that length in one step)
#   q1p5b_           Qwen2.5-1.5B layer sizes (28 layers, hidden 1536, 12 / 2 heads of 128, intermediate 8960, vocabulary
#                    151936, tied), prefixes of 2,048 tokens, a 2,048-token prefill
#   q7b_             Qwen2.5-7B layer sizes (28 layers, hidden 3584, 28 / 4 heads of 128, intermediate 18944, vocabulary
#                    152064, untied), prefixes of 4,096 tokens, a 2,048-token prefill
FURTHER_CONTEXTS = (("ctx8k", 8192), ("ctx32k", 32640))
FURTHER_SHAPES = (("q1p5b", "1.5b"), ("q7b", "7b"))
FURTHER_WARMUP, FURTHER_STEPS = 4, 32


def remove_folder(path: str) -> None:
    for f in os.listdir(path):
        os.remove(os.path.join(path, f))
    os.rmdir(path)


def further_points(args, model_dir: str, cfg: dict, g) -> dict:
    """Decode at batch 1 / 8 / 64 and a prefill at further context lengths (the model in `model_dir`) and at the larger
    layer sizes (random weights drawn on the GPU), all layers of each model: a flat dict of tokens a second."""
    import torch

    from easy_gpt.cpp_amd.engine import Engine
    from easy_gpt.cpp_amd.sampling import Sampler
    from easy_gpt.cpp_amd.weights import write_random_model

    points, page = {}, args.page_size
    warm, steps = FURTHER_WARMUP, FURTHER_STEPS
    room = 3 * (warm + steps) + page                    # the first request decodes in all three runs

    def rate(label, what, tokens, sec):
        points[f"{label}_{what}"] = round(tokens / sec, 1)
        print(f"[bench] {label} {what}: {tokens / sec:.1f} tok/s, {sec / (steps if what != 'prefill' else 1) * 1e3:.3f} ms",
              file=sys.stderr, flush=True)

    longest = max(p for _, p in FURTHER_CONTEXTS)
    engine = Engine.from_dir(model_dir, dtype=args.dtype, device="cuda:0", page_size=page,
                             max_tokens=65 * (-(-(longest + room) // page) * page), max_requests=66,
                             tune_products=not args.no_tune)
    sampler = Sampler(engine.device)
    for label, prefix in FURTHER_CONTEXTS:              # the prefixes are filled once and decoded as 64, 8 and 1
        rate(label, "prefill", prefix, prefill_seconds(engine, cfg["vocab_size"], prefix, g, reps=3))
        rids, last = fill_requests(engine, sampler, cfg["vocab_size"], prefix, 64, g)
        for b in (64, 8, 1):
            sub = last[:b]
            rate(label, f"decode_b{b}", b * steps, decode_seconds(engine, sampler, rids[:b], sub, warm, steps, args.no_lookahead)[0])
            last[:b] = sub
        for rid in rids:
            engine.finish(rid)
    del engine, sampler
    torch.cuda.empty_cache()

    for label, shape in FURTHER_SHAPES:
        changes, n_layers, prefix = OTHER_SHAPES[shape]
        other = dict(QWEN25_05B, **changes, num_hidden_layers=n_layers)
        t0 = time.time()
        tmp = tempfile.mkdtemp(prefix="egpt_bench_")
        write_random_model(tmp, other, seed=0, dtype=torch.bfloat16, device="cuda:0")
        engine = Engine.from_dir(tmp, dtype=args.dtype, device="cuda:0", page_size=page,
                                 max_tokens=64 * (-(-(prefix + warm + steps) // page) * page) + PREFILL_TOKENS,
                                 max_requests=65, tune_products=not args.no_tune)
        remove_folder(tmp)
        sampler = Sampler(engine.device)
        print(f"[bench] {label} model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
        rate(label, "prefill", PREFILL_TOKENS, prefill_seconds(engine, other["vocab_size"], PREFILL_TOKENS, g, reps=5))
        for b in (1, 8, 64):
            rids, last = fill_requests(engine, sampler, other["vocab_size"], prefix, b, g)
            rate(label, f"decode_b{b}", b * steps, decode_seconds(engine, sampler, rids, last, warm, steps, args.no_lookahead)[0])
            for rid in rids:
                engine.finish(rid)
        del engine, sampler
        torch.cuda.empty_cache()
    return points


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


def fill_requests(engine, sampler, vocab: int, prefix: int, batch: int, g):
    """`batch` requests with prefixes of `prefix` random tokens in the cache (untimed); their ids and next tokens."""
    import torch

    from easy_gpt.cpp_amd.engine import StepEntry
    from easy_gpt.cpp_amd.sampling import SamplingParams

    greedy = SamplingParams(greedy=True)
    rids, last = [f"d{i}" for i in range(batch)], []
    for rid in rids:
        engine.add_request(rid)
        p = torch.randint(0, vocab, (prefix,), generator=g).tolist()
        out = engine.step([StepEntry(rid, p, [prefix - 1])])
        last.append(sampler.sample(out, [greedy], [0], [0])[0])
    return rids, last


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
                    help="layer sizes: Qwen2.5-0.5B (the default, which the headline numbers are quoted on), 1.5B or 7B")
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
    ap.add_argument("--prefill-only", action="store_true", help="only the 2,048-token prefill (for profiling)")
    ap.add_argument("--serve-budget", type=int, default=2048, help="with --serve: the token budget of one step")
    ap.add_argument("--serve", action="store_true",
                    help="instead of fixed batches: 64 requests with prompts of 128 to 2,048 tokens and 256 new tokens "
                         "each through the scheduler, prompts in portions of 512 (the mixed serving workload)")
    ap.add_argument("--no-lookahead", action="store_true",
                    help="wait for a step's tokens on the host before the next step is launched (the scheduler with --serve, "
                         "the decode loop otherwise)")
    ap.add_argument("--anatomy", action="store_true",
                    help="instead of timing: one decode step at --batch seen from inside its kernels (the library's trace "
                         "build, compiled at the first call)")
    ap.add_argument("--link-floor", action="store_true",
                    help="instead of the model: what a link of a chain of dependent, near-empty kernels costs in a graph")
    args = ap.parse_args()
    if args.link_floor:
        return link_floor()
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
    if args.anatomy:
        return anatomy(args, dict(base, num_hidden_layers=args.layers), name)
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
    hd = h // nq
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
        max_batch, tokens_per_request = SERVE_REQUESTS, -(-(2048 + SERVE_NEW_TOKENS) // page_size) * page_size
    engine = Engine.from_dir(tmp, dtype=args.dtype, device="cuda:0", page_size=page_size,
                             max_tokens=max_batch * tokens_per_request + PREFILL_TOKENS, max_requests=max_batch + 1,
                             tune_products=not args.no_tune)
    sampler = Sampler(engine.device)
    g = torch.Generator().manual_seed(0)
    print(f"[bench] model ready in {time.time() - t_setup:.1f} s", file=sys.stderr, flush=True)

    if args.serve:
        remove_folder(tmp)
        return serve_workload(engine, name, args, vocab)
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
        sec = prefill_seconds(engine, vocab, PREFILL_TOKENS, g)
        prefill = {"value": round(PREFILL_TOKENS / sec, 1), "tokens": PREFILL_TOKENS, "ms": round(sec * 1e3, 3),
                   "frac": round(prefill_flops(PREFILL_TOKENS) / sec / (PEAK_TFLOPS[dtype_key] * 1e12), 5)}
        print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)
    if args.prefill_only:
        print(json.dumps({"metric": f"prefill tok/s at 2,048 tokens ({name})", "prefill": prefill}), flush=True)
        remove_folder(tmp)
        return 0

    # ---------------------------------------------------------------- decoding at each batch size
    def decode_run(batch: int, warmup: int, steps: int):
        rids, last = fill_requests(engine, sampler, vocab, PREFIX, batch, g)
        sec, medians[batch] = decode_seconds(engine, sampler, rids, last, warmup, steps, args.no_lookahead)
        for rid in rids:
            engine.finish(rid)
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
            "sampling": "greedy", "parallelism": "single GPU", "library_products": "first choice" if args.no_tune else "measured",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 5)},
    }
    if prefill is not None:
        line["prefill"] = prefill
    points = {f"decode_b{b}": round(b * args.steps / results[b][0], 1) for b in batches if b != args.batch}
    del engine
    if further:
        points.update(further_points(args, tmp, cfg, g))
    remove_folder(tmp)
    if points:
        line["points"] = points
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
