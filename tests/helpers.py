"""Shared test equipment: requests of random tokens, the ways of cutting them into steps, replaying a
trace through an engine, and comparing with the plain implementation."""
from __future__ import annotations

import json
import os
import random

import torch

import plain_qwen2 as plain
from easy_gpt.cpp_amd.engine import StepEntry
from easy_gpt.cpp_amd.weights import SafetensorsFile, write_safetensors

# Tolerances, as fractions of the largest logit magnitude of the compared rows.
# float32: the engine's rounding is that of float32 sums in another order than the plain model's float64.
FP32_TOL = 2e-5
# bfloat16: the engine rounds activations between kernels (normed inputs, queries, keys, values, probabilities,
# attention outputs, the activated inner values; never the residual stream, partial sums or the logits), and the
# plain model rounds nothing but the weights.  Measured once over 60 seeded traces (mixed, portions, last tokens
# decoded; page sizes 4, 16, 32) for each of the five tiny configurations, as the worst error of a trace:
#   random weights:   median 1.5e-3 to 4.0e-3, largest 5.4e-3 (configuration B)
#   peaked attention: median 1.8e-3 to 1.4e-2, largest 1.9e-2 (configurations D and E, head sizes 64 and 128, where
#                     a score of size s is off by about s / 256 and the softmax turns that into per cents of a
#                     weight); an earlier run of 700 traces had its largest at 2.1e-2
# The lines stand a factor of 1.4 to 1.8 above the largest error seen; a wrong or stale key in a model with peaked
# attention moves a logit by tenths of the scale.
BF16_TOL = 3e-2            # models with peaked attention (`sharpen_attention`)
BF16_TOL_RANDOM = 1e-2     # models with random weights as they are drawn


def make_requests(vocab: int, lengths, seed: int) -> dict[str, list[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def step_record(step, entries, end=()):
    return {"step": step, "entries": [{"id": i, "tokens": t, "want": w} for i, t, w in entries], "end": list(end)}


def trace_whole(reqs):
    """Each request alone and whole: one step per request."""
    return [step_record(s, [(rid, ids, list(range(len(ids))))], [rid]) for s, (rid, ids) in enumerate(reqs.items())]


def trace_last_decoded(reqs, n_last=32):
    """Most of a request in one step, the last n_last tokens one by one."""
    trace, s = [], 0
    for rid, ids in reqs.items():
        head = max(1, len(ids) - n_last)
        trace.append(step_record(s, [(rid, ids[:head], list(range(head)))]))
        s += 1
        for i in range(head, len(ids)):
            trace.append(step_record(s, [(rid, [ids[i]], [0])], [rid] if i == len(ids) - 1 else []))
            s += 1
        if head == len(ids):
            trace[-1]["end"] = [rid]
    return trace


def trace_portions(reqs, seed=0):
    """Portions of changing size, down to two tokens (and single ones)."""
    rng = random.Random(seed)
    trace, s = [], 0
    for rid, ids in reqs.items():
        pos = 0
        sizes = [7, 2, 16, 3, 2, 1, 33, 2, 5, 1, 1, 64, 2]
        k = 0
        while pos < len(ids):
            n = min(sizes[k % len(sizes)] if k < len(sizes) else rng.choice([1, 2, 3, 9, 17, 40]), len(ids) - pos)
            k += 1
            trace.append(step_record(s, [(rid, ids[pos : pos + n], list(range(n)))], [rid] if pos + n == len(ids) else []))
            pos += n
            s += 1
    return trace


def trace_mixed(reqs, seed=0, max_live=4, decode_tail=12, want_all=True):
    """Up to max_live live requests: prompt portions of some beside single decoded tokens of others;
    a request may sit out a step; requests end while others go on, so their pages are used again."""
    rng = random.Random(seed)
    pending = list(reqs.items())
    live: dict[str, list] = {}          # id -> [ids, pos]
    trace, s = [], 0
    while pending or live:
        while pending and len(live) < max_live and (not live or rng.random() < 0.6):
            rid, ids = pending.pop(0)
            live[rid] = [ids, 0]
        entries, end = [], []
        for rid, (ids, pos) in list(live.items()):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                     # left out of this step, goes on later
            remaining = len(ids) - pos
            if remaining <= decode_tail:
                n = 1
            else:
                n = min(rng.choice([2, 2, 3, 5, 8, 13, 16, 21, 31]), remaining - decode_tail)
            toks = ids[pos : pos + n]
            want = list(range(n)) if want_all or n == 1 else ([n - 1] if rng.random() < 0.5 else [])
            entries.append((rid, toks, want))
            live[rid][1] = pos + n
            if pos + n == len(ids):
                end.append(rid)
                del live[rid]
        if entries:
            trace.append(step_record(s, entries, end))
            s += 1
    return trace


def max_live_tokens(trace, round_to=64) -> int:
    """The --max-tokens a trace needs: the most tokens live requests hold at any time, each request's
    count rounded up to a multiple of `round_to`."""
    held: dict[str, int] = {}
    worst = 0
    for rec in trace:
        for e in rec["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in rec["end"]:
            held.pop(rid, None)
    return worst


def replay(engine, trace) -> dict[tuple[str, int], torch.Tensor]:
    """Run a trace through an engine; returns {(request id, position): logits row (float32, CPU)}."""
    rows: dict[tuple[str, int], torch.Tensor] = {}
    fed: dict[str, int] = {}
    for rec in trace:
        entries = []
        for e in rec["entries"]:
            if not engine.has_request(e["id"]):
                engine.add_request(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        out = engine.step(entries)
        if out is not None:
            out = out.float().cpu()
        r = 0
        for e in rec["entries"]:
            base = fed.get(e["id"], 0)
            for w in e["want"]:
                rows[(e["id"], base + w)] = out[r]
                r += 1
            fed[e["id"]] = base + len(e["tokens"])
        assert out is None or r == out.shape[0]
        for rid in rec["end"]:
            engine.finish(rid)
        engine.cache.check()
    return rows


def plain_rows(model_dir, reqs, bf16_weights=False):
    cfg, w = plain.read_model(model_dir, round_to_bf16=bf16_weights)
    return {rid: plain.forward_logits(cfg, w, ids) for rid, ids in reqs.items()}


def worst_error(rows, ref) -> tuple[float, float, tuple]:
    """Largest absolute difference over all rows, the reference's largest magnitude, and where."""
    worst, where, scale = 0.0, None, 0.0
    for (rid, pos), row in rows.items():
        r = ref[rid][pos]
        d = float((row.double() - r).abs().max())
        scale = max(scale, float(r.abs().max()))
        if d > worst:
            worst, where = d, (rid, pos)
    return worst, scale, where


def assert_rows_match(rows, ref, tol, what=""):
    assert rows, "nothing was compared"
    worst, scale, where = worst_error(rows, ref)
    assert worst <= tol * scale, f"{what}: max |diff| {worst:.3e} at {where} exceeds {tol:g} x {scale:.3f}"
    return worst / scale


def sharpen_attention(src_dir: str, dst_dir: str, factor: float = 14.0) -> str:
    """A copy of a model folder whose query and key projections are scaled so that attention is peaked:
    with N(0, 0.02) weights every key gets nearly the same weight, and a fault that touches one far key
    (a page's edge, a stale page) would hardly move the logits."""
    os.makedirs(dst_dir, exist_ok=True)
    with open(os.path.join(src_dir, "config.json")) as f:
        cfg = json.load(f)
    with open(os.path.join(dst_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    with SafetensorsFile(os.path.join(src_dir, "model.safetensors")) as sf:
        tensors = {}
        for name in sf.names():
            t = sf.read(name)
            if ".q_proj." in name or ".k_proj." in name:
                t = t * factor
            tensors[name] = t
    write_safetensors(os.path.join(dst_dir, "model.safetensors"), tensors)
    return dst_dir
