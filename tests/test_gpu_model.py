"""The whole engine on the GPU against the plain implementation, in float32 and bfloat16: every way of
cutting the work, mixed batches with page reuse, long decoding, first tokens, greedy generation."""
import pytest
import torch

import helpers as H
import plain_qwen2 as plain
from conftest import TINY

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


def engine_for(model_dir, dtype, **kw):
    from easy_gpt.cpp_amd import kernels
    from easy_gpt.cpp_amd.engine import Engine

    kernels.use_backend(None)
    kw.setdefault("page_size", 16)
    kw.setdefault("max_requests", 4)
    return Engine.from_dir(model_dir, dtype=dtype, device="cuda:0", **kw)


def tol_of(dtype, random_weights=False):
    if dtype == "float32":
        return H.FP32_TOL
    return H.BF16_TOL_RANDOM if random_weights else H.BF16_TOL


@pytest.fixture(scope="module")
def sharp_by_dtype(tiny_models, tmp_path_factory):
    """Models with peaked attention.  Scores of the random models have a spread of about 0.04, so every key
    weighs the same; scaling q and k projections by f multiplies that by f^2.  float32 gets f = 10 (spread
    about 4: single keys decide; larger scores would amplify float32 rounding of q and k, about 1e-6 of a
    score, beyond the tolerance).  bfloat16 rounds q and k to 8 bits, which moves a score s by about s / 256,
    so it gets f = 6 (spread about 1.5): still peaked, but its own rounding stays inside its tolerance."""
    out = {}
    for dtype, f in (("float32", 10.0), ("bfloat16", 6.0)):
        out[dtype] = {n: H.sharpen_attention(d, str(tmp_path_factory.mktemp(f"sharp_{n}_{dtype}")), f)
                      for n, d in tiny_models.items()}
    return out


@pytest.fixture()
def sharp_models(sharp_by_dtype, request):
    dtype = request.node.callspec.params.get("dtype", "float32") if hasattr(request.node, "callspec") else "float32"
    return sharp_by_dtype[dtype]


def lengths_for(name):
    cap = TINY[name][0]["max_position_embeddings"]
    return [min(n, cap) for n in (5, 100, 33, 77)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_every_cutting_agrees_with_plain(tiny_models, sharp_models, name, dtype):
    cfg = TINY[name][0]
    reqs = H.make_requests(cfg["vocab_size"], lengths_for(name), seed=21)
    for models, label in ((tiny_models, "random"), (sharp_models, "sharp")):
        ref = H.plain_rows(models[name], reqs, bf16_weights=(dtype == "bfloat16"))
        results = {}
        for cut, trace in [("whole", H.trace_whole(reqs)), ("last32", H.trace_last_decoded(reqs, 32)),
                           ("portions", H.trace_portions(reqs))]:
            eng = engine_for(models[name], dtype, max_tokens=128)
            rows = H.replay(eng, trace)
            assert len(rows) == sum(len(v) for v in reqs.values())
            H.assert_rows_match(rows, ref, tol_of(dtype, label == "random"), f"{name} {label} {dtype} {cut}")
            results[cut] = rows
            assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]
        # the cuttings also agree with each other, more tightly than with the plain model
        for cut in ("last32", "portions"):
            worst = max(float((results[cut][key] - results["whole"][key]).abs().max()) for key in results["whole"])
            scale = max(float(r.abs().max()) for r in ref.values())
            assert worst <= (1e-5 if dtype == "float32" else tol_of(dtype, label == "random")) * scale, (cut, worst)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_mixed_batches_with_page_reuse(sharp_models, name, dtype):
    cfg = TINY[name][0]
    cap = cfg["max_position_embeddings"]
    reqs = H.make_requests(cfg["vocab_size"], [min(n, cap) for n in (70, 23, 110, 64, 37, 90, 128, 16)], seed=31)
    ref = H.plain_rows(sharp_models[name], reqs, bf16_weights=(dtype == "bfloat16"))
    for page_size, seed in ((16, 1), (4, 2)):
        trace = H.trace_mixed(reqs, seed=seed, decode_tail=20)
        need = H.max_live_tokens(trace, round_to=page_size)
        eng = engine_for(sharp_models[name], dtype, page_size=page_size, max_tokens=need)
        rows = H.replay(eng, trace)
        H.assert_rows_match(rows, ref, tol_of(dtype), f"{name} {dtype} mixed page {page_size}")
        assert max(len(r["entries"]) for r in trace) == 4
        pool = eng.cache.pools[0]
        assert sum(-(-len(v) // page_size) for v in reqs.values()) > pool.num_pages      # pages were used again
        assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


@pytest.mark.parametrize("dtype", ["bfloat16"])
@pytest.mark.parametrize("name", ["D", "E"])
def test_mixed_batches_whose_single_tokens_go_to_the_decode_kernel(sharp_models, name, dtype, monkeypatch):
    # what steps with contexts beyond some thousand tokens do, here at every length: the requests that bring one
    # token are left out by the kernel of the portions and taken by the decode kernel in a launch of its own
    from easy_gpt.cpp_amd.kernels import hip

    monkeypatch.setattr(hip.HipKernels, "singles_apart_beyond", 0)
    cfg = TINY[name][0]
    cap = cfg["max_position_embeddings"]
    reqs = H.make_requests(cfg["vocab_size"], [min(n, cap) for n in (70, 23, 110, 64, 37, 90, 128, 16)], seed=33)
    ref = H.plain_rows(sharp_models[name], reqs, bf16_weights=True)
    trace = H.trace_mixed(reqs, seed=3, decode_tail=20)
    eng = engine_for(sharp_models[name], dtype, max_tokens=H.max_live_tokens(trace, round_to=16))
    H.assert_rows_match(H.replay(eng, trace), ref, tol_of(dtype), f"{name} mixed, single tokens apart")
    assert any(len(r["entries"]) > 1 and {len(e["tokens"]) for e in r["entries"]} > {1} for r in trace)
    # the same steps kernel by kernel, not from replayed graphs
    eng = engine_for(sharp_models[name], dtype, max_tokens=H.max_live_tokens(trace, round_to=16), use_graphs=False)
    H.assert_rows_match(H.replay(eng, trace), ref, tol_of(dtype), f"{name} mixed, single tokens apart, no graphs")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "D"])
def test_the_general_step_kernel_by_kernel(sharp_models, name, dtype):
    # no graphs at all: every step builds its own metadata (one packed upload, nothing padded) and runs kernel by
    # kernel, which is what steps of more than `graph_tokens` tokens and models with per-request state do
    cfg = TINY[name][0]
    cap = cfg["max_position_embeddings"]
    reqs = H.make_requests(cfg["vocab_size"], [min(n, cap) for n in (5, 100, 33, 77, 128, 60)], seed=23)
    ref = H.plain_rows(sharp_models[name], reqs, bf16_weights=(dtype == "bfloat16"))
    for cut, trace in [("whole", H.trace_whole(reqs)), ("last32", H.trace_last_decoded(reqs, 32)),
                       ("portions", H.trace_portions(reqs)), ("mixed", H.trace_mixed(reqs, seed=5, decode_tail=20))]:
        eng = engine_for(sharp_models[name], dtype, page_size=16 if cut != "mixed" else 4, use_graphs=False,
                         max_tokens=H.max_live_tokens(trace, 16))
        rows = H.replay(eng, trace)
        assert len(rows) == sum(len(v) for v in reqs.values())
        H.assert_rows_match(rows, ref, tol_of(dtype), f"{name} {dtype} {cut}, no graphs")
        assert not eng._decode_plans and not eng._row_plans and not eng._padded_plans
        assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


@pytest.mark.parametrize("dtype", DTYPES)
def test_steps_beyond_the_graphs_sizes_take_the_general_step(sharp_models, dtype):
    # graphs only up to 64 tokens a step here: the larger portions of the same trace take the general step, the
    # smaller ones the graphs, and decoded tokens ride beside both
    name = "D"
    cfg = TINY[name][0]
    reqs = H.make_requests(cfg["vocab_size"], [300, 200, 90], seed=24)
    ref = H.plain_rows(sharp_models[name], reqs, bf16_weights=(dtype == "bfloat16"))
    a, b, c = reqs["r0"], reqs["r1"], reqs["r2"]
    trace = [H.step_record(0, [("r0", a[:130], [0, 129])]),                                   # general
             H.step_record(1, [("r0", a[130:131], [0]), ("r1", b[:100], [99])]),              # general, mixed
             H.step_record(2, [("r1", b[100:140], [0, 39]), ("r0", a[131:132], [0])]),        # 41 tokens: rows graph
             H.step_record(3, [("r0", a[132:133], [0]), ("r1", b[140:141], [0])]),            # decode graph
             H.step_record(4, [("r2", c, list(range(90))), ("r0", a[133:134], [0]), ("r1", b[141:], [58])], ["r1", "r2"]),
             H.step_record(5, [("r0", a[134:], list(range(166)))], ["r0"])]
    eng = engine_for(sharp_models[name], dtype, max_tokens=H.max_live_tokens(trace, 16))
    eng.graph_tokens = 64
    rows = H.replay(eng, trace)
    H.assert_rows_match(rows, ref, tol_of(dtype), f"steps beyond the graphs {dtype}")
    assert not eng._padded_plans and eng._row_plans and eng._decode_plans


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(sharp_models, dtype):
    # one request decoded token by token over many pages, another joining half way
    name = "C" if dtype == "float32" else "D"
    cfg = TINY[name][0]
    reqs = H.make_requests(cfg["vocab_size"], [400, 150], seed=41)
    ref = H.plain_rows(sharp_models[name], reqs, bf16_weights=(dtype == "bfloat16"))
    a, b = reqs["r0"], reqs["r1"]
    trace = [H.step_record(0, [("r0", a[:3], [0, 1, 2])])]
    for i in range(3, 400):
        entries = [("r0", [a[i]], [0])]
        j = i - 200
        if 0 <= j < 150:
            entries.append(("r1", [b[j]], [0]))
        trace.append(H.step_record(i, entries, (["r0"] if i == 399 else []) + (["r1"] if j == 149 else [])))
    eng = engine_for(sharp_models[name], dtype, max_tokens=H.max_live_tokens(trace, 16))
    rows = H.replay(eng, trace)
    assert len(rows) == 550
    H.assert_rows_match(rows, ref, tol_of(dtype), f"long decoding {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_decoding_across_the_context_steps_of_the_captured_graphs(sharp_models, dtype):
    # two requests decoded side by side from 490 and 400 tokens on: the decode graphs are captured per step of the
    # longest context (512 tokens) and per width of the block tables, and both change on the way
    name = "D"
    cfg = TINY[name][0]
    reqs = H.make_requests(cfg["vocab_size"], [620, 530], seed=43)
    ref = H.plain_rows(sharp_models[name], reqs, bf16_weights=(dtype == "bfloat16"))
    a, b = reqs["r0"], reqs["r1"]
    trace = [H.step_record(0, [("r0", a[:490], [489])]), H.step_record(1, [("r1", b[:400], [0, 399])])]
    for i in range(130):
        trace.append(H.step_record(2 + i, [("r0", [a[490 + i]], [0]), ("r1", [b[400 + i]], [0])],
                                   ["r0", "r1"] if i == 129 else []))
    eng = engine_for(sharp_models[name], dtype, max_tokens=H.max_live_tokens(trace, 16))
    rows = H.replay(eng, trace)
    assert len(rows) == 3 + 260
    H.assert_rows_match(rows, ref, tol_of(dtype), f"decoding across graph steps {dtype}")
    assert len({key[2] for key in eng._decode_plans}) >= 2 and len({key[1] for key in eng._decode_plans}) >= 2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "D"])
def test_short_portions_run_as_rows_from_a_replayed_graph(sharp_models, name, dtype):
    # a prompt fed five tokens a step beside another request's decoded tokens: six tokens in every step, laid out as six
    # rows of one token, captured at the second step and replayed from then on; every step is compared with the plain model
    cfg = TINY[name][0]
    reqs = H.make_requests(cfg["vocab_size"], [90, 96], seed=47)
    ref = H.plain_rows(sharp_models[name], reqs, bf16_weights=(dtype == "bfloat16"))
    a, b = reqs["r0"], reqs["r1"]
    trace = [H.step_record(0, [("r0", a[:70], [69])])]                       # 70 tokens: the step of many tokens
    for i in range(19):
        entries = [("r1", b[5 * i : 5 * i + 5], [0, 4] if i % 2 else [4]), ("r0", [a[70 + i]], [0])]
        trace.append(H.step_record(1 + i, entries[::-1] if i % 3 == 0 else entries))
    trace.append(H.step_record(20, [("r1", b[95:], [0]), ("r0", [a[89]], [])], ["r0", "r1"]))
    eng = engine_for(sharp_models[name], dtype, max_tokens=H.max_live_tokens(trace, 16))
    rows = H.replay(eng, trace)
    H.assert_rows_match(rows, ref, tol_of(dtype), f"rows from a graph {name} {dtype}")
    plans = eng._row_plans
    assert any(key[0] == 6 and p.graph is not None for key, p in plans.items())
    assert not eng._decode_plans                                              # no step was one token per request


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "D"])
def test_steps_of_some_hundred_tokens_replay_the_graph_of_their_padded_size(sharp_models, name, dtype):
    # steps of 97 to 112 tokens in changing mixes of three requests (portions, single tokens, a request left out): all of
    # them run from the graph for 112 tokens and four requests, captured at its second visit and replayed after; one of
    # them has exactly 112 tokens and so no padding at all; one step wants every row and has a graph of its own
    cfg = TINY[name][0]
    cap = cfg["max_position_embeddings"]
    reqs = H.make_requests(cfg["vocab_size"], [min(250, cap), 230, 240], seed=49)
    ref = H.plain_rows(sharp_models[name], reqs, bf16_weights=(dtype == "bfloat16"))
    plan = [  # tokens of (r0, r1, r2) in each step
        (70, 30, 0), (1, 5, 95), (1, 100, 1), (0, 1, 99), (97, 1, 0), (1, 1, 110), (60, 50, 1), (20, 30, 16), (1, 3, 1),
    ]
    fed = {rid: 0 for rid in reqs}
    trace = []
    for s_i, counts in enumerate(plan):
        entries = []
        for rid, n in zip(reqs, counts):
            n = min(n, len(reqs[rid]) - fed[rid])
            if n == 0:
                continue
            want = list(range(n)) if s_i == 3 else ([n - 1] if (s_i + len(entries)) % 2 else [0, n - 1])
            entries.append((rid, reqs[rid][fed[rid] : fed[rid] + n], want))
            fed[rid] += n
        trace.append(H.step_record(s_i, entries))
    rest = {rid: ids[fed[rid]:] for rid, ids in reqs.items() if fed[rid] < len(ids)}
    eng = engine_for(sharp_models[name], dtype, max_tokens=H.max_live_tokens(trace, 16) + 3 * 256)
    rows = H.replay(eng, trace)
    assert sum(plan[5]) == 112 and len(rows) > 110
    for rid, ids in rest.items():                                   # what is left, whole
        out = eng.step([H.StepEntry(rid, ids, list(range(len(ids))))]).float().cpu()
        for j in range(len(ids)):
            rows[(rid, fed[rid] + j)] = out[j]
    for rid in reqs:
        eng.finish(rid)
    H.assert_rows_match(rows, ref, tol_of(dtype), f"padded graphs {name} {dtype}")
    visits = {key: (p.runs, p.graph is not None) for key, p in eng._padded_plans.items()}
    assert any(key[0] == 112 and key[1] == 4 and captured for key, (runs, captured) in visits.items()), visits
    assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


def test_graph_replays_of_large_steps_equal_the_steps_run_kernel_by_kernel(tmp_path):
    # layer sizes of the 0.5B model (the library's products at their real shapes), two layers: steps of 2,048 and of 300
    # tokens replayed from their graphs several times, with other work between the replays, against the same steps of an
    # engine that runs the same padded steps kernel by kernel: the same kernels, so the same bits
    from easy_gpt.cpp_amd.engine import StepEntry
    from easy_gpt.cpp_amd.weights import write_random_model

    cfg = {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 2, "hidden_size": 896,
        "num_attention_heads": 14, "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 9001,
        "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 4096,
    }
    write_random_model(str(tmp_path), cfg, seed=13, dtype=torch.bfloat16)
    graphs = engine_for(str(tmp_path), "bfloat16", max_tokens=4096 + 1024)
    plain_steps = engine_for(str(tmp_path), "bfloat16", max_tokens=4096 + 1024)
    plain_steps.capture_after = None                     # the same steps on the same padded shapes, never captured
    g = torch.Generator().manual_seed(5)
    for rep in range(5):
        big = torch.randint(0, 9001, (2048,), generator=g).tolist()
        small = torch.randint(0, 9001, (300,), generator=g).tolist()
        outs = []
        for eng in (graphs, plain_steps):
            eng.add_request("big"), eng.add_request("small")
            a = eng.step([StepEntry("big", big, [0, 1000, 2047])]).clone()
            b = eng.step([StepEntry("small", small[:290], [289]), StepEntry("big", [7], [0])]).clone()
            c = eng.step([StepEntry("small", small[290:], [9])]).clone()              # rows of one token
            eng.finish("big"), eng.finish("small")
            outs.append((a, b, c))
        for x, y in zip(*outs):
            assert torch.equal(x, y), rep
    assert all(p.graph is not None for p in graphs._padded_plans.values()) and len(graphs._padded_plans) == 2
    assert all(p.graph is None for p in plain_steps._padded_plans.values()) and len(plain_steps._padded_plans) == 2


def test_plans_are_dropped_and_made_again_when_there_are_too_many(sharp_by_dtype):
    # at most two graphs of a kind are kept here: steps of five sizes in turn drop and re-capture them all the time
    name, dtype = "D", "bfloat16"
    cfg = TINY[name][0]
    model_dir = sharp_by_dtype[dtype][name]
    reqs = H.make_requests(cfg["vocab_size"], [400, 360], seed=52)
    ref = H.plain_rows(model_dir, reqs, bf16_weights=True)
    eng = engine_for(model_dir, dtype, max_tokens=1280)
    eng.MAX_PLANS = 2
    sizes = [70, 20, 100, 3, 130]
    fed = {"r0": 0, "r1": 0}
    trace, s_i = [], 0
    while any(fed[r] < len(reqs[r]) for r in reqs):
        entries = []
        for j, rid in enumerate(reqs):
            n = min(sizes[(s_i + 2 * j) % len(sizes)], len(reqs[rid]) - fed[rid])
            if n:
                entries.append((rid, reqs[rid][fed[rid] : fed[rid] + n], [0, n - 1]))
                fed[rid] += n
        trace.append(H.step_record(s_i, entries))
        s_i += 1
    rows = H.replay(eng, trace)
    H.assert_rows_match(rows, ref, H.BF16_TOL, "plans dropped and made again")
    assert len(eng._padded_plans) <= 2 and len(eng._row_plans) <= 2 and s_i >= 6


def test_a_graph_is_captured_after_every_earlier_one_was_dropped(sharp_by_dtype):
    # one graph kept per kind of step: every new shape drops the only graph there is, and the next capture starts
    # from nothing again (the pool that the dropped graphs shared went with the last of them)
    cfg = TINY["D"][0]
    model_dir = sharp_by_dtype["bfloat16"]["D"]
    reqs = H.make_requests(cfg["vocab_size"], [300], seed=53)
    ref = H.plain_rows(model_dir, reqs, bf16_weights=True)
    eng = engine_for(model_dir, "bfloat16", max_tokens=640)
    eng.MAX_PLANS = 1
    sizes, fed, trace = [70, 130, 70, 30], 0, []
    while fed < 300:
        n = min(sizes[len(trace) % len(sizes)], 300 - fed)
        trace.append(H.step_record(len(trace), [("r0", reqs["r0"][fed : fed + n], [0, n - 1])]))
        fed += n
    rows = H.replay(eng, trace)
    H.assert_rows_match(rows, ref, H.BF16_TOL, "one graph kept")
    assert len(eng._padded_plans) == 1 and len(trace) >= 4


def test_an_engine_is_freed_when_its_last_reference_goes(tiny_models):
    # its plans hold no reference back to it: if they did, its device memory and graphs would be freed whenever the
    # collector of reference cycles runs, which may be in the middle of another engine's graph capture
    import gc
    import weakref

    from easy_gpt.cpp_amd.engine import StepEntry

    reqs = H.make_requests(TINY["A"][0]["vocab_size"], [100, 30, 9], seed=50)
    gc.collect()
    gc.disable()
    try:
        eng = engine_for(tiny_models["A"], "bfloat16", max_tokens=512)
        for rid, ids in reqs.items():
            eng.add_request(rid)
            eng.step([StepEntry(rid, ids[:-3], [])])                      # a padded step and two steps as rows
        for i in (3, 2, 1):
            eng.step([StepEntry(rid, [ids[-i]], [0]) for rid, ids in reqs.items()])     # decode steps, captured
        assert eng._padded_plans and eng._row_plans and eng._decode_plans
        ref = weakref.ref(eng)
        del eng
        assert ref() is None
    finally:
        gc.enable()


def test_portions_behind_a_long_context_are_not_laid_out_as_rows(tiny_models):
    eng = engine_for(tiny_models["D"], "bfloat16", max_tokens=640)
    eng.graph_row_reads = 2000
    reqs = H.make_requests(TINY["D"][0]["vocab_size"], [600], seed=48)
    from easy_gpt.cpp_amd.engine import StepEntry
    eng.add_request("r")
    eng.step([StepEntry("r", reqs["r0"][:500], [])])
    eng.step([StepEntry("r", reqs["r0"][500:510], [9])])                      # 10 tokens x 510 keys > 2000
    assert not eng._row_plans
    eng.graph_row_reads = 1 << 18
    eng.step([StepEntry("r", reqs["r0"][510:520], [9])])
    assert len(eng._row_plans) == 1


def test_wide_layers_with_many_requests_replay_the_library_products_in_the_graph(tmp_path):
    # 40 requests decoded side by side in a model whose gate/up and output matrices are wide enough for the library's
    # product at this many rows: the captured graph then holds library nodes, is replayed step after step with the
    # program's own work in between, and every replay is compared with the plain implementation
    from easy_gpt.cpp_amd import kernels
    from easy_gpt.cpp_amd.weights import write_random_model

    cfg = {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 2, "hidden_size": 512,
        "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 64, "intermediate_size": 6160, "vocab_size": 12400,
        "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 64,
    }
    kernels.use_backend(None)
    k = kernels.backend()
    assert k._library_rows(40, 2 * 6160, 512) and k._library_rows(40, 12400, 512) and not k._library_rows(40, 512, 6160)
    sharp = str(tmp_path)              # plain random weights: this test is about the replays, not about far keys
    write_random_model(sharp, cfg, seed=9)
    n_req, prompt, steps = 40, 9, 7
    reqs = H.make_requests(cfg["vocab_size"], [prompt + steps + i % 3 for i in range(n_req)], seed=61)
    ref = H.plain_rows(sharp, reqs, bf16_weights=True)
    ids = list(reqs)
    trace = [H.step_record(0, [(rid, reqs[rid][:prompt + i % 3], [prompt + i % 3 - 1]) for i, rid in enumerate(ids)])]
    for s in range(steps):
        trace.append(H.step_record(1 + s, [(rid, [reqs[rid][prompt + i % 3 + s]], [0]) for i, rid in enumerate(ids)],
                                   ids if s == steps - 1 else []))
    eng = engine_for(sharp, "bfloat16", max_tokens=n_req * 64, max_requests=n_req)
    rows = H.replay(eng, trace)
    assert len(rows) == n_req * (1 + steps)
    H.assert_rows_match(rows, ref, H.BF16_TOL, "library products in the decode graph")
    plans = list(eng._decode_plans.values())
    assert len(plans) == 1 and plans[0].graph is not None          # an eager visit, then replays


@pytest.mark.parametrize("dtype", DTYPES)
def test_batches_that_shrink_share_the_graph_of_their_padded_size(sharp_models, dtype):
    # 23 requests decode side by side and end one by one: batches of 23 down to 17 run from one graph of 24 rows
    # (rows that were a request become padding and the other way round), 16 and fewer from graphs of their own size;
    # every step is compared with the plain implementation
    m = sharp_models["D"]
    n_req, prompt = 23, 6
    lens = [prompt + 4 + i for i in range(n_req)]                    # request i decodes 4 + i tokens after its prompt
    reqs = H.make_requests(TINY["D"][0]["vocab_size"], lens, seed=71)
    ref = H.plain_rows(m, reqs, bf16_weights=(dtype == "bfloat16"))
    ids = list(reqs)
    trace = [H.step_record(0, [(rid, reqs[rid][:prompt], [prompt - 1]) for rid in ids])]
    fed = {rid: prompt for rid in ids}
    live = list(ids)
    step = 1
    while live:
        # a request that is put in front of the others now and then: rows change their owners
        order = live[step % 3:] + live[:step % 3]
        entries = [(rid, [reqs[rid][fed[rid]]], [0]) for rid in order]
        for rid in order:
            fed[rid] += 1
        ended = [rid for rid in order if fed[rid] == len(reqs[rid])]
        trace.append(H.step_record(step, entries, ended))
        live = [rid for rid in live if rid not in ended]
        step += 1
    eng = engine_for(m, dtype, max_tokens=n_req * 64, max_requests=n_req)
    rows = H.replay(eng, trace)
    assert len(rows) == n_req + sum(n - prompt for n in lens)
    H.assert_rows_match(rows, ref, tol_of(dtype), "decode batches padded to the size of a graph")
    sizes = sorted({key[0] for key in eng._decode_plans})
    assert 24 in sizes and not any(16 < b < 24 for b in sizes), sizes
    padded = [p for key, p in eng._decode_plans.items() if key[0] == 24]
    assert all(p.graph is not None for p in padded)                  # visited often enough to be captured and replayed
    assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


def test_a_layer_with_large_matrices_takes_the_kernels_that_are_not_folded(tmp_path):
    # one layer whose gate/up matrix has 67M elements and whose width is 2,048: with few rows the norm before gate/up
    # and SwiGLU before down then run as kernels of their own (folded into the products they would be computed again
    # by hundreds of workgroups), the QKV and output projections keep their folded prologues with wide workgroups
    from easy_gpt.cpp_amd import kernels
    from easy_gpt.cpp_amd.weights import write_random_model

    cfg = {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 1, "hidden_size": 2048,
        "num_attention_heads": 16, "num_key_value_heads": 2, "intermediate_size": 16384, "vocab_size": 600,
        "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 128,
    }
    kernels.use_backend(None)
    k = kernels.backend()
    h = torch.zeros(3, 2048, device="cuda")
    nw = torch.ones(2048, dtype=torch.bfloat16, device="cuda")
    big = torch.zeros(2 * 16384, 2048, dtype=torch.bfloat16, device="cuda")
    assert k.product_normed(h, None, nw, big) is None and k.product_normed(h, None, nw, big[:2560]) is not None
    del big
    write_random_model(str(tmp_path), cfg, seed=12)
    reqs = H.make_requests(cfg["vocab_size"], [40, 23, 31], seed=71)
    ref = H.plain_rows(str(tmp_path), reqs, bf16_weights=True)
    ids = list(reqs)
    trace = [H.step_record(0, [(rid, reqs[rid][:-6], [len(reqs[rid]) - 7]) for rid in ids])]
    for s in range(6):
        trace.append(H.step_record(1 + s, [(rid, [reqs[rid][len(reqs[rid]) - 6 + s]], [0]) for rid in ids], ids if s == 5 else []))
    eng = engine_for(str(tmp_path), "bfloat16", max_tokens=256)
    rows = H.replay(eng, trace)
    assert len(rows) == 3 * 7
    H.assert_rows_match(rows, ref, H.BF16_TOL, "large matrices, few rows")


def test_library_products_chosen_by_measurement(sharp_by_dtype):
    # with tune_products the library's many-row products are measured at their first visit and the fastest candidate
    # kept; the products with float32 output stay with the library's first choice.  Whatever is chosen, the logits
    # are the plain implementation's, on the first visit (kernel by kernel) and from the replayed graph
    from easy_gpt.cpp_amd import kernels

    m = sharp_by_dtype["bfloat16"]["D"]
    reqs = H.make_requests(TINY["D"][0]["vocab_size"], [200, 150], seed=81)
    ref = H.plain_rows(m, reqs, bf16_weights=True)
    try:
        eng = engine_for(m, "bfloat16", max_tokens=1024, tune_products=True)
        assert kernels.library_tuning and torch.cuda.tunable.is_enabled()
        for visit in range(3):                               # the same shapes again: the graph of the first visit
            trace = [H.step_record(0, [(rid, ids, list(range(len(ids)))) for rid, ids in reqs.items()], list(reqs))]
            rows = H.replay(eng, trace)
            H.assert_rows_match(rows, ref, H.BF16_TOL, f"tuned library products, visit {visit}")
        assert any(p.graph is not None for p in eng._padded_plans.values())
        assert torch.cuda.tunable.is_enabled()               # switched back on after every float32-output product
    finally:
        kernels.tune_library_products(False)
    assert not kernels.library_tuning and not torch.cuda.tunable.is_enabled()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_of_a_sequence(tiny_models, name, dtype):
    cfg = TINY[name][0]
    reqs = H.make_requests(cfg["vocab_size"], [1, 2, 3], seed=51)
    ref = H.plain_rows(tiny_models[name], reqs, bf16_weights=(dtype == "bfloat16"))
    eng = engine_for(tiny_models[name], dtype, max_tokens=192)
    # all three at once, as one batch; then the two-token one again token by token
    trace = [H.step_record(0, [(rid, ids, list(range(len(ids)))) for rid, ids in reqs.items()], list(reqs))]
    rows = H.replay(eng, trace)
    H.assert_rows_match(rows, ref, tol_of(dtype, True), "first tokens, batched")
    rows = H.replay(eng, H.trace_last_decoded({"r2": reqs["r2"]}, 32))
    H.assert_rows_match(rows, ref, tol_of(dtype, True), "first tokens, one by one")


def test_logits_do_not_depend_on_neighbours_or_pages(sharp_models):
    # the same request alone, and among others on different pages: equal up to rounding (here: exactly,
    # float32 kernels reduce in an order that does not depend on the batch)
    name = "B"
    cfg = TINY[name][0]
    reqs = H.make_requests(cfg["vocab_size"], [60, 45, 80], seed=61)
    eng = engine_for(sharp_models[name], "float32", max_tokens=64 * 4)
    alone = H.replay(eng, H.trace_whole({"r0": reqs["r0"]}))
    eng.add_request("filler")                       # shifts which pages r0 gets
    from easy_gpt.cpp_amd.engine import StepEntry
    eng.step([StepEntry("filler", reqs["r1"][:20], [])])
    trace = [H.step_record(0, [("r1", reqs["r1"], []), ("r0", reqs["r0"][:33], list(range(33))), ("r2", reqs["r2"], [5])]),
             H.step_record(1, [("r0", reqs["r0"][33:], list(range(27)))], ["r0", "r1", "r2"])]
    among = H.replay(eng, trace)
    for pos in range(60):
        assert torch.equal(alone[("r0", pos)], among[("r0", pos)]), pos


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_entry_point(tiny_models, dtype):
    from easy_gpt.cpp_amd.generate import LLM

    for name, lens, n_new in (("A", [5, 17, 33], 16), ("B", [1, 9, 40, 100], 24)):
        cfg, w = plain.read_model(tiny_models[name], round_to_bf16=(dtype == "bfloat16"))
        prompts = list(H.make_requests(cfg["vocab_size"], lens, seed=71).values())
        llm = LLM(tiny_models[name], dtype=dtype, cache_tokens=1024, prefill_chunk=16, max_tokens_per_step=48)
        outs = llm.generate(prompts, max_new_tokens=n_new, greedy=True, ignore_eos=True)
        assert [len(o) for o in outs] == [n_new] * len(prompts)
        for prompt, out in zip(prompts, outs):
            # walk the plain model along the engine's tokens; each must be the plain argmax, or tie with it
            # within the tolerance (a near-tie may legitimately fall the other way)
            logits = plain.forward_logits(cfg, w, prompt + out)
            for i, tok in enumerate(out):
                row = logits[len(prompt) + i - 1]
                gap = float(row.max() - row[tok])
                assert gap <= tol_of(dtype, True) * float(row.abs().max()), (name, i, tok, gap)
        assert llm.last_stats.generated == n_new * len(prompts)
        assert llm.engine.cache.free_pages() == [p.num_pages for p in llm.engine.cache.pools]
    # float32 with random weights has no near-ties here: the tokens are exactly the plain model's
    if dtype == "float32":
        cfg, w = plain.read_model(tiny_models["A"])
        prompt = list(H.make_requests(cfg["vocab_size"], [17], seed=72).values())[0]
        llm = LLM(tiny_models["A"], dtype="float32", cache_tokens=256)
        assert llm.generate([prompt], max_new_tokens=16, greedy=True, ignore_eos=True)[0] == plain.greedy_generate(cfg, w, prompt, 16)


def test_temperature_generation_and_preemption(tiny_models):
    from easy_gpt.cpp_amd.generate import LLM

    cfg = TINY["B"][0]
    prompts = list(H.make_requests(cfg["vocab_size"], [1, 9, 40, 100], seed=81).values())
    kw = dict(max_new_tokens=24, temperature=0.8, top_k=20, top_p=0.95, seed=5, ignore_eos=True)
    roomy = LLM(tiny_models["B"], dtype="float32", cache_tokens=2048, prefill_chunk=16, max_tokens_per_step=40)
    a = roomy.generate(prompts, **kw)
    again = roomy.generate(prompts, **kw)
    other_seed = roomy.generate(prompts, **dict(kw, seed=6))
    assert [len(o) for o in a] == [24] * 4
    assert all(0 <= t < cfg["vocab_size"] for o in a for t in o)
    # a pool so small that requests are preempted and recomputed: same tokens (the draw of a request's n-th
    # token depends on (seed, request, n) only; here requests keep their serial numbers)
    tight = LLM(tiny_models["B"], dtype="float32", cache_tokens=192, prefill_chunk=16, max_tokens_per_step=40)
    b = tight.generate(prompts, **kw)
    assert tight.last_stats.preemptions > 0
    assert a == b
    assert again == a              # the seed decides: the same engine gives the same tokens again
    assert other_seed != a         # and another seed other ones (96 draws at temperature 0.8)


@pytest.mark.parametrize("dtype", DTYPES)
def test_decoding_one_step_ahead_of_the_host_gives_the_same_tokens(tiny_models, dtype):
    # the scheduler launches a decode step before it has seen the tokens of the step before it (the token ids go from
    # the sampler to the next step on the device); with greedy and with temperature sampling, with requests that end
    # on an end token (one token too many is computed for them and thrown away) and on their limits, the tokens are
    # those of a scheduler that waits for every step
    from easy_gpt.cpp_amd.engine.scheduler import Request, Scheduler, SchedulerConfig
    from easy_gpt.cpp_amd.sampling import SamplingParams

    cfg = TINY["B"][0]
    eng = engine_for(tiny_models["B"], dtype, max_tokens=2048, max_requests=8)
    prompts = list(H.make_requests(cfg["vocab_size"], [3, 40, 17, 9, 1], seed=91).values())

    def run(lookahead, eos, params):
        sched = Scheduler(eng, SchedulerConfig(max_active=8, prefill_chunk=16, max_tokens_per_step=64), eos_token_id=eos)
        sched.lookahead = lookahead
        reqs = [sched.add(Request(i, p, params, max_new_tokens=20 + 3 * i)) for i, p in enumerate(prompts)]
        sched.run()
        assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]
        return [r.output for r in reqs], [r.finish_reason for r in reqs], sched.stats

    for params in (SamplingParams(greedy=True), SamplingParams(temperature=0.9, top_k=50, top_p=0.9, seed=3)):
        free_run, _, _ = run(False, -1, params)
        eos = free_run[2][7]                                  # the third request ends on its eighth token (or before)
        waiting, why_w, st_w = run(False, eos, params)
        ahead, why_a, st_a = run(True, eos, params)
        assert ahead == waiting and why_a == why_w and "eos" in why_a and "length" in why_a
        assert st_w.steps_ahead == 0 and st_a.steps_ahead > 10 and st_a.discarded >= 1
        assert st_a.generated == st_w.generated == sum(len(o) for o in ahead)
