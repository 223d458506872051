"""Command line in the manner of the reference's `easy_llm`
(/root/reference/include/cli_options.hpp:9-24, /root/reference/src/cli_options.cpp:23-47,86-286,
/root/reference/src/main.cpp:24-125): the same option names, defaults, meanings and error
messages where it has them.  Prompts are token ids (the tokenizer is outside this engine):
a positional prompt is a list of ids separated by commas or blanks, and a prompt file has one
such prompt per non-empty line; with a prompt file the generated ids go to <stem>_output<ext>
beside it, as main.cpp:113-120 does for text.
"""
from __future__ import annotations

import os
import sys
import time
from dataclasses import dataclass

USAGE = """Usage: easy_llm [--model <dir>] [--prompt-file <path>] [--max-steps <n>]
                [--temperature <float>] [--top-p <float>] [--top-k <int>] [--seed <int>] [--greedy]
                [--serve-max-active <n>] [--serve-prefill-batch <n>] [--serve-stats-ms <n>]
                ["prompt token ids"]
  -f, --prompt-file <path>  Read prompts from file (one per line of token ids, ignore empty lines)
  -m, --max-steps <n>        Maximum generation steps per request: cap on its total length (default: 100)
      --temperature <float> Sampling temperature (default: 0.8)
      --top-p <float>        Nucleus sampling cutoff in (0,1] (default: 0.95)
      --top-k <int>          Top-K sampling cutoff, 0 disables (default: 20)
      --seed <int>           RNG seed for sampling (default: 42)
      --greedy               Use greedy decoding (override sampling)
      --serve-max-active <n> Max concurrent active requests (default: 16)
      --serve-prefill-batch <n> Max requests admitted per step (default: 4)
      --serve-idle-ms <n>    Accepted for compatibility; there is no stdin service to idle in (default: 2)
      --serve-stats-ms <n>   Stats log interval in milliseconds, 0 disables periodic logs (default: 1000)
      --model <dir>          Folder with config.json and model.safetensors (default: data/model)
      --allow-unexpected-tensors  Only warn about tensors in the file that the model does not use, as the
                             reference does; without it they are an error, listed with missing and misshapen ones
      --dtype <name>         bfloat16 or float32 (default: bfloat16)
      --device <name>        torch device that holds the model (default: cuda:0; the kernels are for MI355X only)
      --random-weights <config.json>  Write a model folder with random weights from this config (to --model), then run
      --max-new-tokens <n>   Cap on new tokens per request instead of --max-steps
      --ignore-eos           Do not stop at the end token
      --max-tokens-per-step <n>  Token budget of one step (default: 2048)
      --prefill-chunk <n>    Largest prompt portion in one step (default: 512)
      --cache-tokens <n>     Tokens the paged cache holds (default: 65536)
      --page-size <n>        Tokens per cache page (default: 16)
      --tune-products        Choose the library's matrix products by measurement (about a second per new shape)
  -h, --help                Show this help message
Examples:
  bin/easy_llm --model data/model --max-steps 128 "1 2 3"
  bin/easy_llm --temperature 0.7 --top-p 0.9 --top-k 40 "1,2,3"
  bin/easy_llm --greedy -f prompts.txt
"""


@dataclass
class CliOptions:
    prompt: str = ""
    prompt_file: str = ""
    max_steps: int = 100
    temperature: float = 0.8
    top_p: float = 0.95
    top_k: int = 20
    seed: int = 42
    use_greedy: bool = False
    serve: bool = False
    serve_max_active: int = 16
    serve_prefill_batch: int = 4
    serve_idle_ms: int = 2
    serve_stats_ms: int = 1000
    show_help: bool = False
    # beyond the reference
    model: str = "data/model"
    dtype: str = "bfloat16"
    device: str = "cuda:0"
    random_weights: str = ""
    max_new_tokens: int = 0
    ignore_eos: bool = False
    max_tokens_per_step: int = 2048
    prefill_chunk: int = 512
    cache_tokens: int = 65536
    page_size: int = 16
    tune_products: bool = False
    allow_unexpected_tensors: bool = False


class CliError(ValueError):
    pass


def _number(kind, value: str, what: str):
    try:
        if kind is int and not value.lstrip("+-").isdigit():
            raise ValueError
        return kind(value)
    except ValueError:
        raise CliError(f"Invalid number for {what}: {value}") from None


def parse_args(argv: list[str]) -> CliOptions:
    """argv without the program name.  Raises CliError with the reference's messages."""
    o = CliOptions()
    i = 0

    def value(arg: str, noun: str = "number") -> str:
        nonlocal i
        if i + 1 >= len(argv):
            raise CliError(f"Missing {noun} after {arg}")
        i += 1
        return argv[i]

    while i < len(argv):
        arg = argv[i]
        if arg in ("-h", "--help"):
            o.show_help = True
            return o
        elif arg in ("-f", "--prompt-file"):
            v = value(arg, "path")
            if o.prompt_file:
                raise CliError("Prompt file option specified multiple times")
            o.prompt_file = v
        elif arg in ("-m", "--max-steps"):
            o.max_steps = _number(int, value(arg), "max steps")
            if o.max_steps <= 0:
                raise CliError("Max steps must be greater than 0")
        elif arg == "--temperature":
            o.temperature = _number(float, value(arg), "temperature")
            if not o.temperature > 0:
                raise CliError("Temperature must be greater than 0")
        elif arg == "--top-p":
            o.top_p = _number(float, value(arg), "top-p")
            if not 0.0 < o.top_p <= 1.0:
                raise CliError("Top-p must be in (0, 1]")
        elif arg == "--top-k":
            o.top_k = _number(int, value(arg), "top-k")
            if o.top_k < 0:
                raise CliError("Top-k must be >= 0")
        elif arg == "--seed":
            o.seed = _number(int, value(arg), "seed")
            if o.seed < 0:
                raise CliError("Seed must be >= 0")
        elif arg == "--greedy":
            o.use_greedy = True
        elif arg == "--serve":
            o.serve = True
        elif arg == "--serve-max-active":
            o.serve_max_active = _number(int, value(arg), "serve max active")
            if o.serve_max_active <= 0:
                raise CliError("serve-max-active must be greater than 0")
        elif arg == "--serve-prefill-batch":
            o.serve_prefill_batch = _number(int, value(arg), "serve prefill batch")
            if o.serve_prefill_batch <= 0:
                raise CliError("serve-prefill-batch must be greater than 0")
        elif arg == "--serve-idle-ms":
            o.serve_idle_ms = _number(int, value(arg), "serve idle ms")
            if o.serve_idle_ms < 0:
                raise CliError("serve-idle-ms must be >= 0")
        elif arg == "--serve-stats-ms":
            o.serve_stats_ms = _number(int, value(arg), "serve stats ms")
            if o.serve_stats_ms < 0:
                raise CliError("serve-stats-ms must be >= 0")
        elif arg == "--model":
            o.model = value(arg, "path")
        elif arg == "--dtype":
            o.dtype = value(arg, "name")
            if o.dtype not in ("bfloat16", "float32", "bf16", "fp32"):
                raise CliError(f"Unknown dtype: {o.dtype}")
        elif arg == "--device":
            o.device = value(arg, "name")
        elif arg == "--random-weights":
            o.random_weights = value(arg, "path")
        elif arg == "--max-new-tokens":
            o.max_new_tokens = _number(int, value(arg), "max new tokens")
            if o.max_new_tokens <= 0:
                raise CliError("max-new-tokens must be greater than 0")
        elif arg == "--ignore-eos":
            o.ignore_eos = True
        elif arg == "--tune-products":
            o.tune_products = True
        elif arg == "--allow-unexpected-tensors":
            o.allow_unexpected_tensors = True
        elif arg in ("--max-tokens-per-step", "--prefill-chunk", "--cache-tokens", "--page-size"):
            name = arg[2:].replace("-", "_")
            v = _number(int, value(arg), arg[2:].replace("-", " "))
            if v <= 0:
                raise CliError(f"{arg[2:]} must be greater than 0")
            setattr(o, name, v)
        elif arg.startswith("-") and len(arg) > 1 and not arg.lstrip("-").replace(",", "").replace(" ", "").isdigit():
            raise CliError(f"Unknown option: {arg}")
        else:
            if o.prompt:
                raise CliError("Multiple prompts provided; use a single prompt or --prompt-file")
            o.prompt = arg
        i += 1
    return o


def parse_prompt(text: str) -> list[int]:
    parts = text.replace(",", " ").split()
    try:
        ids = [int(p) for p in parts]
    except ValueError:
        raise CliError(f"A prompt must be a list of token ids, got: {text!r}") from None
    if not ids:
        raise CliError("Empty prompt")
    return ids


def read_prompts_file(path: str) -> list[list[int]]:
    """One prompt per non-empty line (/root/reference/src/cli_options.cpp:66-84)."""
    try:
        with open(path, "r", encoding="utf-8") as f:
            lines = [ln.strip() for ln in f]
    except OSError:
        raise CliError(f"Failed to open prompt file: {path}") from None
    return [parse_prompt(ln) for ln in lines if ln]


def output_path_for(prompt_file: str) -> str:
    d, base = os.path.split(prompt_file)
    stem, ext = os.path.splitext(base)
    return os.path.join(d, f"{stem}_output{ext}")


def main(argv: list[str] | None = None) -> int:
    argv = sys.argv[1:] if argv is None else argv
    try:
        o = parse_args(argv)
        if o.show_help:
            sys.stdout.write(USAGE)
            return 0
        if o.serve:
            raise CliError("--serve (the stdin service) is not part of this engine; "
                           "give prompts on the command line or with --prompt-file")
        prompts: list[list[int]] = []
        if o.prompt_file:
            prompts += read_prompts_file(o.prompt_file)
        if o.prompt:
            prompts.append(parse_prompt(o.prompt))
        if not prompts:
            raise CliError("No prompts provided")
    except CliError as e:
        sys.stderr.write(f"error: {e}\n")
        sys.stderr.write(USAGE)
        return 1

    if o.random_weights:
        from .config.base import read_json
        from .weights import write_random_model

        write_random_model(o.model, read_json(o.random_weights), o.seed)
        print(f"[easy_llm] wrote random weights (seed {o.seed}) to {o.model}", file=sys.stderr)

    from .generate import LLM

    llm = LLM(o.model, dtype=o.dtype, device=o.device, cache_tokens=o.cache_tokens, page_size=o.page_size,
              max_active=o.serve_max_active, max_admit_per_step=o.serve_prefill_batch,
              max_tokens_per_step=o.max_tokens_per_step, prefill_chunk=o.prefill_chunk, tune_products=o.tune_products,
              allow_unexpected_tensors=o.allow_unexpected_tensors)
    last = [time.perf_counter()]

    def on_step(sched):
        if o.serve_stats_ms and (time.perf_counter() - last[0]) * 1000.0 >= o.serve_stats_ms:
            last[0] = time.perf_counter()
            s = sched.stats
            print(f"[stats] steps={s.steps} running={len(sched.running)} waiting={len(sched.waiting)} "
                  f"finished={s.finished} prompt_tokens={s.prompt_tokens} generated={s.generated} "
                  f"preemptions={s.preemptions}", file=sys.stderr, flush=True)

    t0 = time.perf_counter()
    requests = llm.generate_requests(
        prompts, max_new_tokens=o.max_new_tokens or 100, max_steps=None if o.max_new_tokens else o.max_steps,
        temperature=o.temperature, top_p=o.top_p, top_k=o.top_k, greedy=o.use_greedy, seed=o.seed,
        ignore_eos=o.ignore_eos, on_step=on_step,
    )
    dt = time.perf_counter() - t0
    # a request that failed leaves an empty line (and its reason on stderr); the others keep their outputs
    failed = [r for r in requests if r.status == "failed"]
    for r in failed:
        print(f"error: request {r.request_id} failed: {r.finish_reason}", file=sys.stderr)
    lines = ["" if r.status == "failed" else " ".join(str(t) for t in r.output) for r in requests]
    if o.prompt_file:
        path = output_path_for(o.prompt_file)
        with open(path, "w", encoding="utf-8") as f:
            f.write("\n".join(lines) + "\n")
        print(f"[easy_llm] wrote {len(lines)} outputs to {path}", file=sys.stderr)
    else:
        for ln in lines:
            print(ln)
    s = llm.last_stats
    print(f"[summary] requests={len(requests)} failed={len(failed)} steps={s.steps} prompt_tokens={s.prompt_tokens} "
          f"generated={s.generated} preemptions={s.preemptions} seconds={dt:.3f} "
          f"tok_per_s={s.generated / dt if dt > 0 else 0:.1f}", file=sys.stderr)
    return 1 if failed else 0
