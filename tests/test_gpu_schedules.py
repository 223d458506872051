"""Schedules that the other GPU tests do not reach: decode steps launched ahead of the host for more requests than a
graph's rows follow one by one (batches beyond 16 are padded to a multiple of 8) on a model with windowed layers, a
device given without its index, and models made without a file."""
import pytest
import torch

import helpers as H
import plain_qwen2 as plain
from conftest import TINY

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.mark.parametrize("dtype", DTYPES)
def test_many_requests_decode_ahead_on_windowed_layers(tiny_models, dtype):
    # 21 requests on configuration D (a windowed layer: pages are given back while decoding runs ahead), so the decode
    # batches are padded (24 rows for 21 to 17 requests) and shrink as requests end: on their limits, and one on an
    # end token while the batch is padded.  Steps launched ahead give the tokens of a scheduler that waits for every
    # step, greedy and with temperature; and every greedy token is the plain model's argmax at its place (or ties
    # with it within the tolerance)
    from easy_gpt.cpp_amd import kernels
    from easy_gpt.cpp_amd.engine import Engine
    from easy_gpt.cpp_amd.engine.scheduler import Request, Scheduler, SchedulerConfig
    from easy_gpt.cpp_amd.sampling import SamplingParams

    kernels.use_backend(None)
    cfg = TINY["D"][0]
    n_req = 21
    eng = Engine.from_dir(tiny_models["D"], dtype=dtype, device="cuda:0", page_size=16, max_tokens=n_req * 160,
                          max_requests=n_req + 1)
    assert eng._has_windows
    prompts = list(H.make_requests(cfg["vocab_size"], [5 + (7 * i) % 60 for i in range(n_req)], seed=95).values())

    def run(lookahead, eos, params):
        sched = Scheduler(eng, SchedulerConfig(max_active=n_req, max_admit_per_step=n_req, prefill_chunk=64,
                                               max_tokens_per_step=512), eos_token_id=eos)
        sched.lookahead = lookahead
        reqs = [sched.add(Request(i, p, params, max_new_tokens=30 + i)) for i, p in enumerate(prompts)]
        sched.run()
        assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]
        return [r.output for r in reqs], [r.finish_reason for r in reqs], sched.stats

    for params in (SamplingParams(greedy=True), SamplingParams(temperature=0.8, top_k=40, top_p=0.95, seed=11)):
        free_run, _, _ = run(False, -1, params)
        # an end token that one request alone produces, within its first tokens: 21 rows become 20 while the batch is
        # padded to 24 either way.  (A request that ends on an end token is in one more step when steps are launched
        # ahead; were that the step in which 17 rows become 16, the two runs would take different kernels there, and
        # bfloat16 logits would differ by their rounding.)
        others = lambda i: {t for j, o in enumerate(free_run) if j != i for t in o}
        which, eos = next((i, t) for i in range(n_req - 1, -1, -1) for t in free_run[i][:14] if t not in others(i))
        waiting, why_w, st_w = run(False, eos, params)
        ahead, why_a, st_a = run(True, eos, params)
        assert ahead == waiting and why_a == why_w and why_a.count("eos") == 1 and why_a[which] == "eos"
        assert st_w.steps_ahead == 0 and st_a.steps_ahead > 20 and st_a.discarded == 1
        assert st_a.generated == sum(len(o) for o in ahead)
        assert (st_a.decode_tokens, st_a.prompt_tokens) == (st_w.decode_tokens, st_w.prompt_tokens)
        assert any(rows == 24 for (rows, _, _) in eng._decode_plans)            # padded batches ran
        if params.greedy:
            pcfg, w = plain.read_model(tiny_models["D"], round_to_bf16=(dtype == "bfloat16"))
            tol = H.FP32_TOL if dtype == "float32" else H.BF16_TOL_RANDOM
            for prompt, out in zip(prompts, ahead):
                logits = plain.forward_logits(pcfg, w, prompt + out)
                for i, tok in enumerate(out):
                    row = logits[len(prompt) + i - 1]
                    gap = float(row.max() - row[tok])
                    assert gap <= tol * float(row.abs().max()), (i, tok, gap)


def test_a_device_without_an_index(tiny_models):
    # "cuda" names the current GPU; tensors made there call themselves "cuda:0", and steps launched ahead compare the
    # device of the sampler's tokens with the engine's
    from easy_gpt.cpp_amd.generate import LLM

    cfg = TINY["A"][0]
    prompts = list(H.make_requests(cfg["vocab_size"], [5, 17], seed=96).values())
    outs = {}
    for device in ("cuda", "cuda:0"):
        llm = LLM(tiny_models["A"], dtype="float32", device=device, cache_tokens=512)
        assert llm.engine.device == torch.device("cuda:0")
        outs[device] = llm.generate(prompts, max_new_tokens=12, temperature=0.8, seed=3, ignore_eos=True)
        assert llm.last_stats.steps_ahead > 5
    assert outs["cuda"] == outs["cuda:0"]


def test_random_weights_are_the_same_on_every_device_and_without_a_file(tmp_path):
    # a tensor's values are a function of (seed, name, index) in integer arithmetic: the GPU draws what the CPU draws;
    # and a model loaded from the generator gives the logits of the model loaded from the folder that was written
    from easy_gpt.cpp_amd.engine import Engine, StepEntry
    from easy_gpt.cpp_amd.engine.engine import load_random_model
    from easy_gpt.cpp_amd.parts.spec import ParamSpec
    from easy_gpt.cpp_amd.weights import random_tensor, write_random_model

    for spec in (ParamSpec("w", (301, 77)), ParamSpec("n", (1000,), role="norm_scale"),
                 ParamSpec("t", (50,), role="int_table", dtype="int32")):
        for dtype in (torch.float32, torch.bfloat16):
            assert torch.equal(random_tensor(spec, 4, dtype, device="cpu"), random_tensor(spec, 4, dtype, device="cuda:0"))
    cfg = TINY["B"][0]
    write_random_model(str(tmp_path), cfg, seed=8, dtype=torch.bfloat16, device="cpu")
    ids = H.make_requests(cfg["vocab_size"], [40], seed=97)["r0"]
    rows = []
    for model in (None, load_random_model(cfg, seed=8, dtype="bfloat16", device="cuda:0")):
        eng = (Engine.from_dir(str(tmp_path), dtype="bfloat16", device="cuda:0", max_tokens=64, max_requests=2)
               if model is None else Engine(model, max_tokens=64, max_requests=2))
        eng.add_request("r")
        rows.append(eng.step([StepEntry("r", ids, [0, 39])]).clone())
    assert torch.equal(rows[0], rows[1])


def test_generation_under_page_pressure_gives_the_same_tokens_in_float32():
    # 40 requests with prompts of 20 to 6,000 tokens on four layers of the 0.5B sizes, greedy: with room for all of them,
    # and with so few pages that requests are preempted dozens of times (freed, queued again, their prompt and what
    # they had generated computed again in other portions, beside other requests, on other pages).  In float32 a
    # row's logits are the same bits however the work is cut and batched, so every request must get exactly the
    # tokens it got with room
    import random

    from easy_gpt.cpp_amd import kernels
    from easy_gpt.cpp_amd.engine import Engine
    from easy_gpt.cpp_amd.engine.engine import load_random_model
    from easy_gpt.cpp_amd.engine.scheduler import Request, Scheduler, SchedulerConfig
    from easy_gpt.cpp_amd.sampling import SamplingParams

    kernels.use_backend(None)
    cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 4, "hidden_size": 896,
           "num_attention_heads": 14, "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 151936,
           "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 32768,
           "hidden_act": "silu", "torch_dtype": "bfloat16"}
    model = load_random_model(cfg, seed=3, dtype="float32", device="cuda:0")
    rnd = random.Random(5)
    lens = [rnd.choice([rnd.randint(20, 300), rnd.randint(500, 3000), rnd.randint(4000, 6000)]) for _ in range(40)]
    new = [rnd.choice([8, 40, 100]) for _ in lens]
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in lens]
    outputs = {}
    for label, max_tokens in (("room", sum(lens) + sum(new) + 4096), ("pressure", 10000)):
        eng = Engine(model, page_size=16, max_tokens=max_tokens, max_requests=33)
        sched = Scheduler(eng, SchedulerConfig(max_active=32, max_admit_per_step=4, max_tokens_per_step=2048,
                                               prefill_chunk=512), eos_token_id=-1)
        reqs = [sched.add(Request(i, p, SamplingParams(greedy=True), max_new_tokens=n, ignore_eos=True))
                for i, (p, n) in enumerate(zip(prompts, new))]
        sched.run()
        assert all(r.finish_reason == "length" and len(r.output) == n for r, n in zip(reqs, new))
        assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools] and not eng.cache.requests
        assert (sched.stats.preemptions > 20) == (label == "pressure")
        outputs[label] = [list(r.output) for r in reqs]
        del eng, sched
    assert outputs["pressure"] == outputs["room"]
