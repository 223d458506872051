"""bin/trace_run as a user runs it: a subprocess fed with JSON lines, logits files compared with the plain model."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers as H
from conftest import TINY

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_trace(model_dir, dtype, trace, out_dir, max_tokens, vocab, page_size=None):
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens)]
    if page_size is not None:
        cmd += ["--page-size", str(page_size)]
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    rows, fed = {}, {}
    for rec in trace:
        p.stdin.write(json.dumps(rec) + "\n")
        p.stdin.flush()
        line = p.stdout.readline().strip()
        assert line == f"done {rec['step']}", line
        wanted = sum(len(e["want"]) for e in rec["entries"])
        path = os.path.join(out_dir, f"{rec['step']}.f32")
        if wanted:
            data = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
            r = 0
            for e in rec["entries"]:
                for w in e["want"]:
                    rows[(e["id"], fed.get(e["id"], 0) + w)] = torch.from_numpy(data[r].copy())
                    r += 1
        else:
            assert not os.path.exists(path)
        for e in rec["entries"]:
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    # the index written at the end names the same rows by (request, position)
    with open(os.path.join(out_dir, "index.json")) as f:
        index = json.load(f)
    assert index["vocab"] == vocab and len(index["rows"]) == len(rows)
    for item in index["rows"]:
        data = np.fromfile(os.path.join(out_dir, item["file"]), dtype="<f4").reshape(-1, vocab)
        assert torch.equal(torch.from_numpy(data[item["row"]].copy()), rows[(item["id"], item["position"])])
    return rows


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_mixed_trace(tiny_models, tmp_path, dtype):
    name = "B"
    cfg = TINY[name][0]
    reqs = H.make_requests(cfg["vocab_size"], [70, 23, 110, 64, 37, 90], seed=91)
    ref = H.plain_rows(tiny_models[name], reqs, bf16_weights=(dtype == "bfloat16"))
    trace = H.trace_mixed(reqs, seed=4, decode_tail=32, want_all=False)
    rows = run_trace(tiny_models[name], dtype, trace, str(tmp_path / "out"), H.max_live_tokens(trace, 64), cfg["vocab_size"])
    assert len(rows) > 150
    H.assert_rows_match(rows, ref, H.FP32_TOL if dtype == "float32" else H.BF16_TOL_RANDOM, f"trace_run {dtype}")
    # a page size that is no divisor of 64 (requests counted in whole pages of it)
    rows = run_trace(tiny_models[name], dtype, trace, str(tmp_path / "out48"), H.max_live_tokens(trace, 48), cfg["vocab_size"],
                     page_size=48)
    H.assert_rows_match(rows, ref, H.FP32_TOL if dtype == "float32" else H.BF16_TOL_RANDOM, f"trace_run {dtype}, pages of 48")


def test_trace_run_whole_and_last32(tiny_models, tmp_path):
    name = "A"
    cfg = TINY[name][0]
    reqs = H.make_requests(cfg["vocab_size"], [5, 128, 33], seed=92)
    ref = H.plain_rows(tiny_models[name], reqs)
    for i, trace in enumerate((H.trace_whole(reqs), H.trace_last_decoded(reqs, 32))):
        for s, rec in enumerate(trace):
            rec["step"] = s
        rows = run_trace(tiny_models[name], "float32", trace, str(tmp_path / f"out{i}"), 128, cfg["vocab_size"])
        assert len(rows) == 166
        H.assert_rows_match(rows, ref, H.FP32_TOL, "trace_run float32")
