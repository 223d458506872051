"""The engine's bookkeeping on the CPU: the step function, block tables, slots and page reuse are run with
the tests' slow stand-in for the kernels and compared with the plain implementation.  The kernels
themselves are tested on the GPU (-m gpu)."""
import pytest
import torch

import helpers as H
from conftest import TINY
from emulated_kernels import EmulatedKernels
from easy_gpt.cpp_amd import kernels
from easy_gpt.cpp_amd.cache import OutOfPages
from easy_gpt.cpp_amd.engine import Engine, StepEntry


@pytest.fixture(autouse=True)
def emulated_backend():
    kernels.use_backend(EmulatedKernels())
    yield
    kernels.use_backend(None)


def test_no_cpu_path_in_the_product():
    kernels.use_backend(None)
    with pytest.raises(kernels.KernelsUnavailable):
        kernels.backend()


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_cuttings_agree_with_plain(tiny_models, name):
    cfg = TINY[name][0]
    reqs = H.make_requests(cfg["vocab_size"], [5, 41, 17], seed=11)
    ref = H.plain_rows(tiny_models[name], reqs)
    for page_size, trace in [(4, H.trace_whole(reqs)), (16, H.trace_last_decoded(reqs, 8)), (3, H.trace_portions(reqs))]:
        eng = Engine.from_dir(tiny_models[name], dtype="float32", device="cpu", page_size=page_size,
                              max_tokens=64, max_requests=2)
        rows = H.replay(eng, trace)
        assert len(rows) == sum(len(v) for v in reqs.values())
        H.assert_rows_match(rows, ref, 1e-6, f"{name} page {page_size}")
        assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


@pytest.mark.parametrize("name", ["B", "C"])
def test_mixed_batches_with_page_reuse(tiny_models, name):
    cfg = TINY[name][0]
    reqs = H.make_requests(cfg["vocab_size"], [23, 9, 37, 30, 14, 26], seed=3)
    ref = H.plain_rows(tiny_models[name], reqs)
    trace = H.trace_mixed(reqs, seed=1, decode_tail=5)
    need = H.max_live_tokens(trace, round_to=4)
    eng = Engine.from_dir(tiny_models[name], dtype="float32", device="cpu", page_size=4, max_tokens=need, max_requests=4)
    rows = H.replay(eng, trace)
    H.assert_rows_match(rows, ref, 1e-6, name)
    assert max(len(r["entries"]) for r in trace) >= 3
    total_pages = sum(-(-len(v) // 4) for v in reqs.values())
    assert total_pages > eng.cache.pools[0].num_pages            # so pages were used again
    assert eng.cache.pools[0].high_water <= eng.cache.pools[0].num_pages


def test_step_checks_and_out_of_pages_leaves_the_cache_unchanged(tiny_models):
    eng = Engine.from_dir(tiny_models["A"], dtype="float32", device="cpu", page_size=4, num_pages=4, max_requests=2)
    eng.add_request("a")
    eng.add_request("b")
    with pytest.raises(IndexError, match="token id"):
        eng.step([StepEntry("a", [512], [0])])
    with pytest.raises(IndexError, match="wanted place"):
        eng.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(KeyError):
        eng.step([StepEntry("zz", [1], [0])])
    with pytest.raises(ValueError, match="twice"):
        eng.step([StepEntry("a", [1], [0]), StepEntry("a", [2], [0])])
    assert eng.step([StepEntry("a", list(range(9)), [])]) is None          # nothing wanted
    with pytest.raises(OutOfPages):
        eng.step([StepEntry("a", [1], [0]), StepEntry("b", list(range(8)), [0])])   # b needs 2 pages, 1 free
    assert eng.cache.requests["a"].num_tokens == 9 and eng.cache.requests["b"].tables == [[]]
    assert eng.cache.free_pages() == [1]
    eng.cache.check()
    out = eng.step([StepEntry("a", [1], [0]), StepEntry("b", [3, 4], [1, 0])])
    assert out.shape == (3, 512) and out.dtype == torch.float32
    with pytest.raises(ValueError, match="max_position_embeddings"):
        eng.finish("b")
        eng.step([StepEntry("a", list(range(200)), [])])


def test_a_step_that_fails_leaves_the_cache_as_it_found_it(tiny_models):
    # an error between the reservation of a step's pages and their commit (here: the model raises) gives the pages
    # back, and the same step can be run again
    cfg = TINY["A"][0]
    reqs = H.make_requests(cfg["vocab_size"], [23, 9], seed=5)
    ref = H.plain_rows(tiny_models["A"], reqs)
    eng = Engine.from_dir(tiny_models["A"], dtype="float32", device="cpu", page_size=4, max_tokens=64, max_requests=2)
    ids = list(reqs)
    for rid in ids:
        eng.add_request(rid)
    eng.step([StepEntry(rid, reqs[rid][:5], [4]) for rid in ids])
    free = eng.cache.free_pages()
    forward = eng.model.forward

    def broken(ctx):
        raise RuntimeError("the device is gone")

    eng.model.forward = broken
    second = [StepEntry(ids[0], reqs[ids[0]][5:], [0]), StepEntry(ids[1], reqs[ids[1]][5:6], [0])]
    with pytest.raises(RuntimeError, match="gone"):
        eng.step(second)
    assert eng.cache.free_pages() == free
    eng.cache.check()
    eng.model.forward = forward
    logits = eng.step(second)
    for row, rid in zip(logits, ids):
        assert float((row.double().cpu() - ref[rid][5]).abs().max()) <= 1e-5 * float(ref[rid][5].abs().max())
    for rid in ids:
        eng.finish(rid)
    assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]
