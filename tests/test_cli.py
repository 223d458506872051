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
