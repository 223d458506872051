"""The engine at the layer sizes of Qwen2.5-0.5B (width 896, 14 query and 2 kv heads of 64, inner width 4,864, the
whole vocabulary of 151,936, tied, theta 1e6; two layers) against the plain implementation, in float32 and in
bfloat16: the four cuttings on requests of a few hundred tokens, and the shape that the benchmark measures: eight
requests with prefixes of about 2,100 tokens, decoded from the captured graph, and one request decoded alone behind
such a prefix.  The kernels take other paths at these sizes than at the tiny ones (folded products with a k range
of 896, key ranges of the decode attention split over workgroups, the tiled prefill attention with 14 query heads on
2 kv heads, the two-stage argmax, products of the library).

The plain implementation is the same float64 torch code as everywhere, computed on the GPU here (on the CPU these
shapes take minutes); logits are compared at chosen places only (a row is 151,936 numbers).
"""
import pytest
import torch

import helpers as H
import plain_qwen2 as plain

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]

SIZES_0P5B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 2, "hidden_size": 896,
    "num_attention_heads": 14, "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 151936,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 32768,
    "use_sliding_window": False, "hidden_act": "silu", "torch_dtype": "bfloat16",
}
VOCAB = SIZES_0P5B["vocab_size"]


@pytest.fixture(scope="module")
def models_0p5b(tmp_path_factory):
    """dtype -> (model folder, plain config, plain weights on the GPU).  The files hold bfloat16 values, so the
    engine in either precision and the plain model compute with the same weights.  Attention is peaked as in the
    tiny models' tests (a wrong or stale key must move the logits): scores of the random model have a spread of
    about 0.4 here; the query and key projections are scaled so that it becomes about 3.5 for float32 and about 1.5
    for bfloat16, whose own rounding of queries and keys moves a score by 1/256 of its size."""
    from easy_gpt.cpp_amd.weights import write_random_model

    d = str(tmp_path_factory.mktemp("sizes_0p5b"))
    write_random_model(d, SIZES_0P5B, seed=5, dtype=torch.bfloat16)
    made = {}

    def get(dtype):
        if dtype not in made:
            sharp = H.sharpen_attention(d, str(tmp_path_factory.mktemp(f"sizes_0p5b_{dtype}")), 3.0 if dtype == "float32" else 2.0)
            made[dtype] = (sharp,) + plain.read_model(sharp, device="cuda:0")
        return made[dtype]

    return get


def engine_for(model_dir, dtype, **kw):
    from easy_gpt.cpp_amd import kernels
    from easy_gpt.cpp_amd.engine import Engine

    kernels.use_backend(None)
    kw.setdefault("page_size", 16)
    kw.setdefault("max_requests", 8)
    return Engine.from_dir(model_dir, dtype=dtype, device="cuda:0", **kw)


def tol_of(dtype):
    return H.FP32_TOL if dtype == "float32" else H.BF16_TOL


def only_wanted(trace, keep):
    """The trace with logits asked for only at the positions in keep[request id]."""
    fed: dict[str, int] = {}
    out = []
    for rec in trace:
        entries = []
        for e in rec["entries"]:
            base = fed.get(e["id"], 0)
            entries.append({"id": e["id"], "tokens": e["tokens"], "want": [w for w in e["want"] if base + w in keep[e["id"]]]})
            fed[e["id"]] = base + len(e["tokens"])
        out.append({"step": rec["step"], "entries": entries, "end": rec["end"]})
    return out


def compare(rows, cfg, w, reqs, tol, what):
    """rows {(request, position): logits row on the CPU} against the plain model's rows at the same places."""
    assert rows, "nothing was compared"
    worst, scale, where = 0.0, 0.0, None
    for rid, ids in reqs.items():
        places = sorted(pos for (r, pos) in rows if r == rid)
        if not places:
            continue
        ref = plain.forward_logits(cfg, w, ids[: places[-1] + 1], rows=places).cpu()
        for i, pos in enumerate(places):
            d = float((rows[(rid, pos)].double() - ref[i]).abs().max())
            scale = max(scale, float(ref[i].abs().max()))
            if d > worst:
                worst, where = d, (rid, pos)
    print(f"{what}: {len(rows)} rows, largest error {worst / scale:.2e} of the logit scale {scale:.2f}", flush=True)
    assert worst <= tol * scale, f"{what}: max |diff| {worst:.3e} at {where} exceeds {tol:g} x {scale:.3f}"
    return worst / scale


@pytest.mark.parametrize("dtype", DTYPES)
def test_every_cutting_at_the_0p5b_sizes(models_0p5b, dtype):
    model_dir, cfg, w = models_0p5b(dtype)
    reqs = H.make_requests(VOCAB, [300, 70, 181, 33], seed=61)
    keep = {rid: set(range(0, len(ids), 11)) | set(range(max(0, len(ids) - 34), len(ids))) for rid, ids in reqs.items()}
    for cut, trace in [("whole", H.trace_whole(reqs)), ("last32", H.trace_last_decoded(reqs, 32)),
                       ("portions", H.trace_portions(reqs)), ("mixed", H.trace_mixed(reqs, seed=3, decode_tail=20))]:
        trace = only_wanted(trace, keep)
        need = H.max_live_tokens(trace, 16)
        eng = engine_for(model_dir, dtype, max_tokens=need if cut == "mixed" else 512)
        rows = H.replay(eng, trace)
        assert len(rows) == sum(len(k) for k in keep.values())
        compare(rows, cfg, w, reqs, tol_of(dtype), f"0.5B sizes {dtype} {cut}")
        assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_benchmarks_shape_decoding_behind_long_prefixes(models_0p5b, dtype):
    # eight requests with prefixes of 2,089 to 2,110 tokens (each fed in one step of more than 2,048 tokens, which no
    # graph covers), then 16 decode steps of all eight (the first run kernel by kernel, the others replayed from its
    # graph), then one of them alone for four steps more, and a mixed step: a portion of a new prompt beside decoded
    # tokens of two others
    from easy_gpt.cpp_amd.engine import StepEntry

    model_dir, cfg, w = models_0p5b(dtype)
    lens = [2110, 2089, 2100, 2095, 2105, 2091, 2108, 2099]
    n_decoded, n_alone = 16, 4
    reqs = H.make_requests(VOCAB, [n + n_decoded + n_alone for n in lens], seed=62)
    reqs["late"] = H.make_requests(VOCAB, [150], seed=63)["r0"]
    eng = engine_for(model_dir, dtype, max_tokens=9 * 2176, max_requests=9)
    rows = {}
    for (rid, ids), n in zip(reqs.items(), lens):
        eng.add_request(rid)
        out = eng.step([StepEntry(rid, ids[:n], [0, n - 1])]).float().cpu()
        rows[(rid, 0)], rows[(rid, n - 1)] = out[0], out[1]
    assert not eng._padded_plans and not eng._decode_plans              # those steps took the general path
    rids = list(reqs)[:8]
    for i in range(n_decoded):
        out = eng.step([StepEntry(rid, [reqs[rid][n + i]], [0]) for rid, n in zip(rids, lens)]).float().cpu()
        for j, (rid, n) in enumerate(zip(rids, lens)):
            rows[(rid, n + i)] = out[j]
    assert any(p.graph is not None for p in eng._decode_plans.values())
    first, n0 = rids[0], lens[0] + n_decoded
    for i in range(n_alone):
        rows[(first, n0 + i)] = eng.step([StepEntry(first, [reqs[first][n0 + i]], [0])]).float().cpu()[0]
    eng.add_request("late")
    mixed = [StepEntry("late", reqs["late"][:120], [0, 119]),
             StepEntry(rids[1], [reqs[rids[1]][lens[1] + n_decoded]], [0]),
             StepEntry(rids[2], [reqs[rids[2]][lens[2] + n_decoded]], [0])]
    out = eng.step(mixed).float().cpu()
    rows[("late", 0)], rows[("late", 119)] = out[0], out[1]
    rows[(rids[1], lens[1] + n_decoded)], rows[(rids[2], lens[2] + n_decoded)] = out[2], out[3]
    for rid in list(reqs):
        eng.finish(rid)
    compare(rows, cfg, w, reqs, tol_of(dtype), f"0.5B sizes {dtype} decoding behind 2,100 tokens")
    assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


@pytest.mark.parametrize("dtype", DTYPES)
def test_decoding_behind_a_long_prefix_splits_the_keys_many_times(models_0p5b, dtype):
    # one request behind 9,000 tokens decodes alone: its keys are split over more workgroups than the output
    # projection combines in registers (its wide path); then beside two requests with 3,000-token prefixes
    from easy_gpt.cpp_amd import kernels
    from easy_gpt.cpp_amd.engine import StepEntry

    model_dir, cfg, w = models_0p5b(dtype)
    lens = {"long": 9000, "b": 3011, "c": 2990}
    n_new = 9
    reqs = {rid: H.make_requests(VOCAB, [n + n_new], seed=64 + i)["r0"] for i, (rid, n) in enumerate(lens.items())}
    eng = engine_for(model_dir, dtype, max_tokens=9216 + 2 * 3072, max_requests=3)
    if dtype == "bfloat16":
        assert kernels.backend()._decode_shape(1, 2, 64, 9216, False)[0] > 16
    rows, fed = {}, {}

    def prefill(rid):
        eng.add_request(rid)
        ids, n, pos = reqs[rid], lens[rid], 0
        while pos < n:
            step = min(2048, n - pos)
            out = eng.step([StepEntry(rid, ids[pos : pos + step], [step - 1] if pos + step == n else [])])
            pos += step
        rows[(rid, n - 1)] = out.float().cpu()[0]
        fed[rid] = n

    def decode(which):
        out = eng.step([StepEntry(rid, [reqs[rid][fed[rid]]], [0]) for rid in which]).float().cpu()
        for j, rid in enumerate(which):
            rows[(rid, fed[rid])] = out[j].clone()
            fed[rid] += 1

    prefill("long")
    for _ in range(5):
        decode(["long"])
    prefill("b")
    prefill("c")
    for _ in range(4):
        decode(["long", "b", "c"])
    for rid in reqs:
        eng.finish(rid)
    compare(rows, cfg, w, reqs, tol_of(dtype), f"0.5B sizes {dtype} decoding behind 9,000 tokens")
    assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_of_a_long_prompt_beside_decoded_tokens(models_0p5b, dtype):
    # a prompt of 9,000 tokens in portions of 512 and less, every step beside the decoded tokens of two requests behind
    # 3,000 tokens: in bfloat16 the portions' blocks of rows share their keys among several workgroups once the
    # prefix is long, and the requests of one token go to the decode kernel; the steps replay the graphs of their
    # padded sizes
    from easy_gpt.cpp_amd.engine import StepEntry

    model_dir, cfg, w = models_0p5b(dtype)
    n_long, lens = 9000, {"b": 3011, "c": 2990}
    cuts = [512] * 9 + [300, 512, 64, 512, 2, 512, 16] + [512] * 4
    cuts.append(n_long - sum(cuts))
    assert 0 < cuts[-1] <= 512
    reqs = {"long": H.make_requests(VOCAB, [n_long], seed=80)["r0"]}
    for i, (rid, n) in enumerate(lens.items()):
        reqs[rid] = H.make_requests(VOCAB, [n + len(cuts)], seed=81 + i)["r0"]
    eng = engine_for(model_dir, dtype, max_tokens=9216 + 2 * 3072, max_requests=3)
    rows, fed = {}, {}
    for rid, n in lens.items():
        eng.add_request(rid)
        for pos in range(0, n, 2048):
            step = min(2048, n - pos)
            eng.step([StepEntry(rid, reqs[rid][pos : pos + step], [])])
        fed[rid] = n
    eng.add_request("long")
    pos = 0
    for i, n in enumerate(cuts):
        want = [0, n - 1] if i % 4 == 1 or i >= len(cuts) - 2 or n < 100 else []
        entries = [StepEntry("long", reqs["long"][pos : pos + n], want)]
        entries += [StepEntry(rid, [reqs[rid][fed[rid]]], [0]) for rid in lens]
        out = eng.step(entries).float().cpu()
        for j, at in enumerate(want):
            rows[("long", pos + at)] = out[j].clone()
        for j, rid in enumerate(lens):
            rows[(rid, fed[rid])] = out[len(want) + j].clone()
            fed[rid] += 1
        pos += n
    assert pos == n_long
    assert any(p.graph is not None for p in eng._padded_plans.values())
    for rid in reqs:
        eng.finish(rid)
    compare(rows, cfg, w, reqs, tol_of(dtype), f"0.5B sizes {dtype} portions of a long prompt beside decoded tokens")
    assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


@pytest.mark.parametrize("dtype", DTYPES)
def test_decoding_behind_32000_tokens(models_0p5b, dtype):
    # the longest context of the benchmark's record: a request of 32,000 tokens, its prompt fed in one step of that
    # many tokens (no graph covers it) and, again, in portions of 2,048 (replayed from the graph of that size); then
    # decoded alone (the keys split over dozens of workgroups) and beside seven requests behind 4,000 tokens
    from easy_gpt.cpp_amd.engine import StepEntry

    model_dir, cfg, w = models_0p5b(dtype)
    n_long, n_short, n_alone, n_beside = 32000, 4000, 3, 3
    reqs = {"long": H.make_requests(VOCAB, [n_long + n_alone + n_beside], seed=70)["r0"]}
    for i in range(7):
        reqs[f"s{i}"] = H.make_requests(VOCAB, [n_short - 11 * i + n_beside], seed=71 + i)["r0"]
    eng = engine_for(model_dir, dtype, max_tokens=2 * 32768 + 7 * 4096, max_requests=9)
    rows, fed = {}, {}

    def decode(which):
        out = eng.step([StepEntry(rid, [reqs[rid][fed[rid]]], [0]) for rid in which]).float().cpu()
        for j, rid in enumerate(which):
            rows[(rid, fed[rid])] = out[j].clone()
            fed[rid] += 1

    # in portions of 2,048 (a second request with the same tokens), logits at the last place and inside
    eng.add_request("portions")
    ids, pos = reqs["long"], 0
    while pos < n_long:
        step = min(2048, n_long - pos)
        out = eng.step([StepEntry("portions", ids[pos : pos + step], [step - 1] if pos + step == n_long else [])])
        pos += step
    in_portions = out.float().cpu()[0].clone()
    assert any(p.graph is not None for p in eng._padded_plans.values())
    eng.finish("portions")
    # in one step
    eng.add_request("long")
    out = eng.step([StepEntry("long", ids[:n_long], [999, n_long - 1])]).float().cpu()
    rows[("long", 999)], rows[("long", n_long - 1)] = out[0].clone(), out[1].clone()
    fed["long"] = n_long
    scale = float(rows[("long", n_long - 1)].abs().max())
    assert float((in_portions - rows[("long", n_long - 1)]).abs().max()) <= 2 * tol_of(dtype) * scale
    for _ in range(n_alone):
        decode(["long"])
    for i in range(7):
        rid = f"s{i}"
        n = len(reqs[rid]) - n_beside
        eng.add_request(rid)
        for pos in range(0, n, 2048):
            step = min(2048, n - pos)
            out = eng.step([StepEntry(rid, reqs[rid][pos : pos + step], [step - 1] if pos + step == n else [])])
        rows[(rid, n - 1)] = out.float().cpu()[0].clone()
        fed[rid] = n
    for _ in range(n_beside):
        decode(["long"] + [f"s{i}" for i in range(7)])
    for rid in reqs:
        eng.finish(rid)
    rows[("long2", n_long - 1)] = in_portions
    reqs["long2"] = reqs["long"][:n_long]
    compare(rows, cfg, w, reqs, tol_of(dtype), f"0.5B sizes {dtype} decoding behind 32,000 tokens")
    assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]
