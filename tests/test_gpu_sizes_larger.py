"""One layer at the layer sizes of Qwen2.5-1.5B (width 1,536, 12 query and 2 kv heads of 128, inner width 8,960, tied)
and of Qwen2.5-7B (width 3,584, 28 query and 4 kv heads of 128, inner width 18,944, a separate output matrix) against
the plain implementation, in float32 and in bfloat16.  At these sizes the kernels take paths that neither the tiny
configurations nor the 0.5B sizes reach: products with the norm folded in in workgroups of sixteen wavefronts and a
norm kernel of its own before the gate/up product, rows of the residual stream too wide for one pass of a workgroup,
the decode attention at head size 128 in workgroups of eight wavefronts (more LDS than a kernel may take unasked),
the library's products for a few dozen rows.

The plain implementation runs in float64 on the GPU; logits are compared at chosen places only."""
import pytest
import torch

import helpers as H
import plain_qwen2 as plain
from test_gpu_sizes_0p5b import compare, engine_for, only_wanted, tol_of

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]

BASE = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 1, "rope_theta": 1000000.0,
        "rms_norm_eps": 1e-6, "max_position_embeddings": 4096, "use_sliding_window": False, "hidden_act": "silu",
        "torch_dtype": "bfloat16"}
SIZES = {
    "1.5b": dict(BASE, hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960,
                 vocab_size=151936, tie_word_embeddings=True),
    "7b": dict(BASE, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944,
               vocab_size=152064, tie_word_embeddings=False),
}


@pytest.fixture(scope="module")
def larger_models(tmp_path_factory):
    """(size, dtype) -> (model folder, plain config, plain weights on the GPU); one size's weights at a time are kept.
    Attention is peaked as in the other tests (the scores' spread grows with the width: the gain is set by it)."""
    from easy_gpt.cpp_amd.weights import write_random_model

    kept = {}

    def get(size, dtype):
        if (size, dtype) not in kept:
            kept.clear()
            torch.cuda.empty_cache()
            cfg = SIZES[size]
            d = str(tmp_path_factory.mktemp(f"sizes_{size.replace('.', 'p')}"))
            write_random_model(d, cfg, seed=7, dtype=torch.bfloat16, device="cuda:0")
            gain = ((2.5 if dtype == "float32" else 0.9) / (0.0004 * cfg["hidden_size"])) ** 0.5
            sharp = H.sharpen_attention(d, d + "_sharp", gain)
            kept[(size, dtype)] = (sharp,) + plain.read_model(sharp, device="cuda:0")
        return kept[(size, dtype)]

    return get


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("size", ["1.5b", "7b"])
def test_cuttings_and_decoding_at_larger_sizes(larger_models, size, dtype):
    from easy_gpt.cpp_amd.engine import StepEntry

    model_dir, cfg, w = larger_models(size, dtype)
    vocab = cfg["vocab_size"]
    # the four cuttings on short requests
    reqs = H.make_requests(vocab, [150, 41, 97], seed=71)
    keep = {rid: set(range(0, len(ids), 13)) | set(range(max(0, len(ids) - 34), len(ids))) for rid, ids in reqs.items()}
    for cut, trace in [("whole", H.trace_whole(reqs)), ("last32", H.trace_last_decoded(reqs, 32)),
                       ("portions", H.trace_portions(reqs)), ("mixed", H.trace_mixed(reqs, seed=5, decode_tail=12))]:
        trace = only_wanted(trace, keep)
        eng = engine_for(model_dir, dtype, max_tokens=max(H.max_live_tokens(trace, 16), 512))
        rows = H.replay(eng, trace)
        assert len(rows) == sum(len(k) for k in keep.values())
        compare(rows, cfg, w, reqs, tol_of(dtype), f"{size} sizes {dtype} {cut}")
        assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]
        del eng
    # eight requests behind prefixes of about 1,100 tokens, decoded from the captured graph; then twenty (rows padded
    # to 24: the products of 17 to 64 rows) for two steps; then one alone
    lens = [1110, 1089, 1100, 1095, 1105, 1091, 1108, 1099] + [40 + 7 * i for i in range(12)]
    n_decoded = 8
    reqs = H.make_requests(vocab, [n + n_decoded + 4 for n in lens], seed=72)
    eng = engine_for(model_dir, dtype, max_tokens=8 * 1184 + 12 * 192, max_requests=20)
    rows, rids = {}, list(reqs)
    for rid, n in zip(rids, lens):
        eng.add_request(rid)
        out = eng.step([StepEntry(rid, reqs[rid][:n], [n - 1])]).float().cpu()
        rows[(rid, n - 1)] = out[0]
    fed = dict(zip(rids, lens))

    def decode(which):
        out = eng.step([StepEntry(rid, [reqs[rid][fed[rid]]], [0]) for rid in which]).float().cpu()
        for j, rid in enumerate(which):
            rows[(rid, fed[rid])] = out[j].clone()
            fed[rid] += 1

    for _ in range(n_decoded - 2):
        decode(rids[:8])
    for _ in range(2):
        decode(rids)
    for _ in range(2):
        decode(rids[:1])
    assert sum(p.graph is not None for p in eng._decode_plans.values()) >= 2
    for rid in rids:
        eng.finish(rid)
    compare(rows, cfg, w, reqs, tol_of(dtype), f"{size} sizes {dtype} decoding behind 1,100 tokens")
    assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("size", ["1.5b", "7b"])
def test_portions_behind_a_prefix_beside_decoded_tokens_at_larger_sizes(larger_models, size, dtype):
    # a prompt of 3,900 tokens in portions of up to 512, every step beside the decoded tokens of two requests behind
    # 2,300 tokens: at head size 128 the portions' blocks of rows share their keys among workgroups from 2,048 tokens
    # on, and the requests of one token go to the decode kernel
    from easy_gpt.cpp_amd.engine import StepEntry

    model_dir, cfg, w = larger_models(size, dtype)
    vocab = cfg["vocab_size"]
    n_long, lens = 3900, {"b": 2311, "c": 2290}
    cuts = [512] * 4 + [300, 512, 70, 2, 512]
    cuts.append(n_long - sum(cuts))
    assert 0 < cuts[-1] <= 512
    reqs = {"long": H.make_requests(vocab, [n_long], seed=90)["r0"]}
    for i, (rid, n) in enumerate(lens.items()):
        reqs[rid] = H.make_requests(vocab, [n + len(cuts)], seed=91 + i)["r0"]
    eng = engine_for(model_dir, dtype, max_tokens=4096 + 2 * 2432, max_requests=3)
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
        want = [0, n - 1] if i % 3 == 1 or i >= len(cuts) - 2 or n < 100 else []
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
    for rid in reqs:
        eng.finish(rid)
    compare(rows, cfg, w, reqs, tol_of(dtype), f"{size} sizes {dtype} portions behind a prefix beside decoded tokens")
    assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]
