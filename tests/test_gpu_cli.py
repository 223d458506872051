"""The command line as a user runs it on the GPU: bin/easy_llm and `python -m easy_gpt.cpp_amd` as subprocesses,
their tokens compared with the plain implementation's greedy generation."""
import json
import os
import subprocess
import sys

import pytest

import plain_qwen2 as plain
from conftest import TINY_A, TINY_B

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(cmd, **kw):
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=110, cwd=kw.pop("cwd", ROOT), **kw)
    assert p.returncode == 0, p.stderr[-2000:]
    return p


def test_easy_llm_with_random_weights_and_a_prompt(tmp_path):
    # float32 with random weights has no near-ties at these sizes: the tokens are exactly the plain model's
    cfg_path, model = tmp_path / "cfg.json", tmp_path / "model"
    cfg_path.write_text(json.dumps(TINY_A))
    p = run([sys.executable, os.path.join(ROOT, "bin", "easy_llm"), "--random-weights", str(cfg_path), "--model", str(model),
             "--dtype", "float32", "--greedy", "--ignore-eos", "--max-new-tokens", "16", "--seed", "0", "5 17 3 250 9"])
    cfg, w = plain.read_model(str(model))
    assert [int(t) for t in p.stdout.split()] == plain.greedy_generate(cfg, w, [5, 17, 3, 250, 9], 16)
    assert "wrote random weights (seed 0)" in p.stderr and "[summary] requests=1 failed=0" in p.stderr
    assert os.path.isfile(model / "config.json") and os.path.isfile(model / "model.safetensors")


def test_module_entry_with_a_prompt_file(tmp_path):
    # `python -m easy_gpt.cpp_amd -f prompts.txt` from another working folder: one line of token ids per prompt in
    # prompts_output.txt beside the prompt file (/root/reference/src/main.cpp:105-125), empty lines of the file
    # skipped (/root/reference/src/cli_options.cpp:66-84); prompts in portions of 16, four requests at a time
    from easy_gpt.cpp_amd.weights import write_random_model

    model = str(tmp_path / "model")
    write_random_model(model, TINY_B, seed=1)
    prompts = [[3, 4, 5], list(range(10, 60)), [999], [7] * 33, [1, 2]]
    (tmp_path / "prompts.txt").write_text("\n\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    env = dict(os.environ, PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", ""))
    p = run([sys.executable, "-m", "easy_gpt.cpp_amd", "-f", str(tmp_path / "prompts.txt"), "--model", model, "--dtype", "float32",
             "--greedy", "--ignore-eos", "--max-new-tokens", "8", "--prefill-chunk", "16", "--serve-max-active", "4",
             "--cache-tokens", "1024"], cwd=str(tmp_path), env=env)
    assert p.stdout.strip() == ""                                         # with a prompt file nothing goes to stdout
    lines = (tmp_path / "prompts_output.txt").read_text().splitlines()
    cfg, w = plain.read_model(model)
    assert [[int(t) for t in ln.split()] for ln in lines] == [plain.greedy_generate(cfg, w, pr, 8) for pr in prompts]
    assert "wrote 5 outputs" in p.stderr


def test_sampling_options_through_the_command_line(tmp_path):
    # the reference's defaults (temperature 0.8, top-p 0.95, top-k 20, seed 42) and --max-steps as the cap on the whole
    # length: the same command gives the same tokens twice, another seed gives others
    from easy_gpt.cpp_amd.weights import write_random_model

    model = str(tmp_path / "model")
    write_random_model(model, TINY_A, seed=2)
    base = [sys.executable, os.path.join(ROOT, "bin", "easy_llm"), "--model", model, "--ignore-eos", "-m", "40", "9 8 7 6"]
    a, b = run(base).stdout.split(), run(base).stdout.split()
    c = run(base + ["--seed", "43"]).stdout.split()
    assert len(a) == 40 - 4 + 1 and a == b and a != c
    assert all(0 <= int(t) < TINY_A["vocab_size"] for t in a + c)
