"""Command line parsing in the reference's manner (no GPU); vectors of /root/reference/test/cli_options_test.cpp."""
import pytest

from easy_gpt.cpp_amd.cli import CliError, main, output_path_for, parse_args, parse_prompt, read_prompts_file


def test_defaults_are_the_reference_s():
    o = parse_args(["1 2 3"])
    assert (o.max_steps, o.temperature, o.top_p, o.top_k, o.seed, o.use_greedy) == (100, 0.8, 0.95, 20, 42, False)
    assert (o.serve_max_active, o.serve_prefill_batch, o.serve_idle_ms, o.serve_stats_ms) == (16, 4, 2, 1000)
    assert o.prompt == "1 2 3"


def test_serve_flags_parse():
    # /root/reference/test/cli_options_test.cpp:12-43
    o = parse_args(["--serve", "--serve-max-active", "12", "--serve-prefill-batch", "3", "--serve-idle-ms", "5",
                    "--serve-stats-ms", "250"])
    assert o.serve and (o.serve_max_active, o.serve_prefill_batch, o.serve_idle_ms, o.serve_stats_ms) == (12, 3, 5, 250)


def test_negative_stats_interval_names_the_flag():
    # /root/reference/test/cli_options_test.cpp:45-62
    with pytest.raises(CliError, match="serve-stats-ms"):
        parse_args(["--serve", "--serve-stats-ms", "-1"])


@pytest.mark.parametrize("argv,msg", [
    (["-x"], "Unknown option: -x"),
    (["--max-steps"], "Missing number after --max-steps"),
    (["-m", "abc"], "Invalid number for max steps: abc"),
    (["-m", "0"], "Max steps must be greater than 0"),
    (["--temperature", "0"], "Temperature must be greater than 0"),
    (["--top-p", "1.5"], r"Top-p must be in \(0, 1\]"),
    (["--top-k", "-2"], "Top-k must be >= 0"),
    (["--seed", "-1"], "Seed must be >= 0"),
    (["-f"], "Missing path after -f"),
    (["-f", "a", "-f", "b"], "Prompt file option specified multiple times"),
    (["1 2", "3 4"], "Multiple prompts provided"),
    (["--serve-max-active", "0"], "serve-max-active must be greater than 0"),
    (["--serve-prefill-batch", "x"], "Invalid number for serve prefill batch: x"),
])
def test_error_messages(argv, msg):
    with pytest.raises(CliError, match=msg):
        parse_args(argv)


def test_short_and_long_options():
    o = parse_args(["-m", "64", "--temperature", "0.7", "--top-p", "0.9", "--top-k", "40", "--seed", "7", "--greedy",
                    "-f", "p.txt", "--model", "dir", "--dtype", "float32", "--max-new-tokens", "5", "--ignore-eos"])
    assert (o.max_steps, o.temperature, o.top_p, o.top_k, o.seed, o.use_greedy) == (64, 0.7, 0.9, 40, 7, True)
    assert (o.prompt_file, o.model, o.dtype, o.max_new_tokens, o.ignore_eos) == ("p.txt", "dir", "float32", 5, True)
    assert parse_args(["--tune-products", "1 2"]).tune_products and not parse_args(["1 2"]).tune_products
    assert parse_args(["-h", "--bogus"]).show_help


def test_prompts(tmp_path):
    assert parse_prompt("1, 2,3  4") == [1, 2, 3, 4]
    with pytest.raises(CliError):
        parse_prompt("hello")
    f = tmp_path / "prompts.txt"
    f.write_text("1 2 3\n\n  \n4,5\n")
    assert read_prompts_file(str(f)) == [[1, 2, 3], [4, 5]]          # empty lines are ignored
    with pytest.raises(CliError, match="Failed to open prompt file"):
        read_prompts_file(str(tmp_path / "none.txt"))
    assert output_path_for("/a/b/test_batch.txt") == "/a/b/test_batch_output.txt"


def test_main_errors_return_one(capsys):
    assert main(["--top-k", "-1"]) == 1
    assert "Top-k must be >= 0" in capsys.readouterr().err
    assert main([]) == 1
    assert "No prompts provided" in capsys.readouterr().err
    assert main(["--help"]) == 0
    assert "Usage: easy_llm" in capsys.readouterr().out


# ----------------------------------------------------------------------------- the body of main(), on the CPU
@pytest.fixture()
def emulated_backend():
    from emulated_kernels import EmulatedKernels
    from easy_gpt.cpp_amd import kernels

    kernels.use_backend(EmulatedKernels())
    yield
    kernels.use_backend(None)


def test_main_writes_random_weights_and_generates(tmp_path, capsys, emulated_backend):
    # the whole command line with the tests' stand-in for the kernels: the model folder is written from a config and
    # the seed, loaded, and the greedy tokens are the plain implementation's
    import json

    import plain_qwen2 as plain
    from conftest import TINY_A

    cfg_path, model = tmp_path / "cfg.json", tmp_path / "model"
    cfg_path.write_text(json.dumps(TINY_A))
    common = ["--model", str(model), "--dtype", "float32", "--device", "cpu", "--greedy", "--ignore-eos",
              "--serve-stats-ms", "0", "--cache-tokens", "512"]
    assert main(["--random-weights", str(cfg_path), "--seed", "3", "--max-new-tokens", "6", "5 17 3 99"] + common) == 0
    out = capsys.readouterr()
    cfg, w = plain.read_model(str(model))
    assert [int(t) for t in out.out.split()] == plain.greedy_generate(cfg, w, [5, 17, 3, 99], 6)
    assert "wrote random weights (seed 3)" in out.err and "[summary] requests=1 failed=0" in out.err
    # a prompt file: one line of output per prompt in <stem>_output<ext> beside it (/root/reference/src/main.cpp:105-125),
    # --max-steps as the cap on a request's whole length (/root/reference/src/continuous_batch_server.cpp:313)
    prompts = tmp_path / "prompts.txt"
    prompts.write_text("1 2 3\n\n  \n7,8,9,10,11\n400\n")
    assert main(["-f", str(prompts), "-m", "8"] + common) == 0
    capsys.readouterr()
    lines = (tmp_path / "prompts_output.txt").read_text().splitlines()
    expected = [plain.greedy_generate(cfg, w, p, max(1, 8 - len(p) + 1)) for p in ([1, 2, 3], [7, 8, 9, 10, 11], [400])]
    assert [[int(t) for t in ln.split()] for ln in lines] == expected
    assert [len(e) for e in expected] == [6, 4, 8]


def test_main_reports_a_request_that_failed_and_keeps_the_others(tmp_path, capsys, emulated_backend):
    import json

    import plain_qwen2 as plain
    from conftest import TINY_A
    from easy_gpt.cpp_amd.weights import write_random_model

    model = str(tmp_path / "model")
    write_random_model(model, TINY_A, seed=0)
    prompts = tmp_path / "p.txt"
    prompts.write_text("1 2 3\n" + " ".join(str(i % 500) for i in range(100)) + "\n4 5\n")
    # a cache of 64 tokens cannot hold the second request (100 tokens) even alone; the others are generated
    rc = main(["-f", str(prompts), "--model", model, "--dtype", "float32", "--device", "cpu", "--greedy", "--ignore-eos",
               "--max-new-tokens", "4", "--cache-tokens", "64", "--serve-stats-ms", "0"])
    err = capsys.readouterr().err
    assert rc == 1 and "request 1 failed" in err and "even alone" in err and "failed=1" in err
    cfg, w = plain.read_model(model)
    lines = (tmp_path / "p_output.txt").read_text().split("\n")
    assert [int(t) for t in lines[0].split()] == plain.greedy_generate(cfg, w, [1, 2, 3], 4)
    assert lines[1] == "" and [int(t) for t in lines[2].split()] == plain.greedy_generate(cfg, w, [4, 5], 4)


def test_unexpected_tensors_are_an_error_unless_allowed(tmp_path, capsys, emulated_backend):
    import torch

    from conftest import TINY_A
    from easy_gpt.cpp_amd.weights import SafetensorsFile, WeightsError, write_random_model, write_safetensors

    model = str(tmp_path / "model")
    write_random_model(model, TINY_A, seed=0)
    path = str(tmp_path / "model" / "model.safetensors")
    with SafetensorsFile(path) as f:
        tensors = {n: f.read(n) for n in f.names()}
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(8)
    write_safetensors(path, tensors)
    args = ["--model", model, "--dtype", "float32", "--device", "cpu", "--greedy", "--max-new-tokens", "2",
            "--serve-stats-ms", "0", "--cache-tokens", "64", "1 2 3"]
    with pytest.raises(WeightsError, match="unexpected tensors"):
        main(args)
    assert main(["--allow-unexpected-tensors"] + args) == 0
    assert "rotary_emb.inv_freq' is not used by this model and was ignored" in capsys.readouterr().err
