"""Rules of a model's description that need no GPU: what a block arrangement may be given, layers without a mixer,
the shapes of paged tensors, distributions of random weights by role; and the toy model with four norms, a
mixer-only layer and a windowed cache of latents stepped on the CPU with the tests' stand-in for the kernels."""
import pytest
import torch

import helpers as H
import test_gpu_toy_shapes as toys
from test_gpu_toy_shapes import toys_registered  # noqa: F401  (fixture)
from emulated_kernels import EmulatedKernels
from easy_gpt.cpp_amd import kernels
from easy_gpt.cpp_amd.cache import PagedStorage
from easy_gpt.cpp_amd.parts import (
    BLOCKS, CacheNeed, LayerSpec, ModelSpec, PagedTensor, ParamSpec, PartSpec, RunSpec, build_model, make_part,
)
from easy_gpt.cpp_amd.weights import random_tensor, register_role
from easy_gpt.cpp_amd.weights import random_init


def norm(p):
    return PartSpec("rmsnorm", dict(eps=1e-5), prefix=p)


def test_a_block_takes_exactly_the_norms_it_places():
    ff = make_part("feed_forward", PartSpec("swiglu", dict(intermediate_size=24), "f."), hidden_size=16)
    att = make_part("mixer", PartSpec("gq_attention", dict(n_heads=1, n_kv_heads=1, head_dim=16, qkv_bias=False, out_bias=False,
                                                            window=None, position=PartSpec("none", {})), "a."), hidden_size=16)
    n = lambda p: make_part("norm", norm(p), hidden_size=16)
    block = BLOCKS["pre_norm"](att, ff, {"mixer": n("n1."), "feed_forward": n("n2.")})
    assert [type(p).__name__ for p in block.parts()] == ["RMSNorm", "RMSNorm", "GQAttention", "SwiGLU"]
    with pytest.raises(ValueError, match="places the norms"):
        BLOCKS["pre_norm"](att, ff, {"mixer": n("n1.")})
    with pytest.raises(ValueError, match="places the norms"):
        BLOCKS["pre_norm"](att, ff, {"mixer": n("n1."), "feed_forward": n("n2."), "after": n("n3.")})
    with pytest.raises(ValueError, match="arranges a mixer and a feed-forward"):
        BLOCKS["pre_norm"](att, None, {"mixer": n("n1."), "feed_forward": n("n2.")})


def test_a_layer_without_a_mixer_has_neither_cache_nor_state(toys_registered):
    class FeedForwardOnly(BLOCKS["toy_mixer_only"].__mro__[1]):          # parts.Block
        norm_slots = ("feed_forward",)
        uses_mixer = False

    BLOCKS["toy_ff_only"] = FeedForwardOnly
    try:
        def spec(run):
            return ModelSpec(hidden_size=16, vocab_size=32, max_position=64, embedding=PartSpec("token_embedding", {}, "e."),
                             layers=(LayerSpec("toy_ff_only", None, PartSpec("swiglu", dict(intermediate_size=24), "f."),
                                               {"feed_forward": norm("n.")}),),
                             run_order=(run,), final_norm=norm("fn."), output_head=PartSpec("linear_head", dict(tied=True), "h."))

        model = build_model(spec(RunSpec(0)))
        assert model.cache_groups == [] and model.state_needs == {}
        assert [s.name for s in model.param_specs()] == ["e.weight", "n.weight", "f.gate_proj.weight", "f.up_proj.weight",
                                                          "f.down_proj.weight", "fn.weight"]
        with pytest.raises(ValueError, match="has no mixer"):
            build_model(spec(RunSpec(0, cache=0)))
    finally:
        BLOCKS.pop("toy_ff_only")


def test_paged_tensor_shapes_and_storage():
    kv = CacheNeed.keys_and_values(n_kv_heads=3, head_dim=32, window=9)
    assert [t.page_shape(8) for t in kv.tensors] == [(3, 8, 32), (3, 32, 8)] and kv.window == 9
    latent = CacheNeed((PagedTensor("latent", (12,), 0, dtype="float32"), PagedTensor("gate", (2, 5), 2)), None)
    assert [t.page_shape(4) for t in latent.tensors] == [(4, 12), (2, 5, 4)]
    with pytest.raises(ValueError, match="token_axis"):
        PagedTensor("x", (4,), 2).page_shape(4)
    store = PagedStorage([kv, latent], [2, 1], [10, 6], 4, torch.bfloat16, "cpu")
    assert store.tensors[0]["k"].shape == (2, 10, 3, 4, 32) and store.tensors[0]["v"].shape == (2, 10, 3, 32, 4)
    assert store.tensors[1]["latent"].shape == (1, 6, 4, 12) and store.tensors[1]["latent"].dtype == torch.float32
    assert store.tensors[1]["gate"].dtype == torch.bfloat16 and set(store.slab(1, 0)) == {"latent", "gate"}
    assert store.slab(0, 1)["k"].data_ptr() == store.tensors[0]["k"][1].data_ptr()
    with pytest.raises(ValueError, match="names a tensor twice"):
        PagedStorage([CacheNeed((PagedTensor("a", (2,)), PagedTensor("a", (3,))))], [1], [2], 4, torch.float32, "cpu")
    # needs are compared by value: mixers with equal needs share a pool
    assert CacheNeed.keys_and_values(3, 32, 9) == kv and CacheNeed.keys_and_values(3, 32, None) != kv


def test_random_weights_by_role():
    spec = ParamSpec("x.rate", (64,), role="toy_rate", dtype="float32")
    with pytest.raises(KeyError, match="toy_rate"):
        random_tensor(spec, seed=1)
    register_role("toy_rate", lambda shape, g, device: 0.9 + 0.09 * torch.rand(shape, generator=g, device=device))
    try:
        t = random_tensor(spec, seed=1)
        assert t.dtype == torch.float32 and 0.9 <= float(t.min()) and float(t.max()) < 0.99
        assert torch.equal(t, random_tensor(spec, seed=1)) and not torch.equal(t, random_tensor(spec, seed=2))
        with pytest.raises(ValueError, match="already registered"):
            register_role("toy_rate", lambda *a: None)
    finally:
        random_init.ROLES.pop("toy_rate")
    assert random_tensor(ParamSpec("m", (4, 4)), seed=1, dtype=torch.bfloat16).dtype == torch.bfloat16
    assert random_tensor(ParamSpec("t", (4,), role="int_table", dtype="int32"), seed=1).dtype == torch.int32


def test_the_toy_shapes_step_on_the_cpu(toys_registered, tmp_path):
    from easy_gpt.cpp_amd.engine import Engine
    from easy_gpt.cpp_amd.weights import write_random_model

    kernels.use_backend(EmulatedKernels())
    try:
        d = write_random_model(str(tmp_path / "toy"), toys.SHAPES_CONFIG, seed=11)
        eng = Engine.from_dir(d, dtype="float32", device="cpu", page_size=4, num_pages=40, max_requests=3)
        w = toys.weights_as_engine_sees_them(d, "float32")
        reqs = H.make_requests(toys.SHAPES_CONFIG["vocab_size"], [21, 9, 33], seed=6)
        ref = {rid: toys.shapes_plain(w, toys.SHAPES_CONFIG, ids) for rid, ids in reqs.items()}
        for trace in (H.trace_portions(reqs), H.trace_mixed(reqs, seed=4, max_live=3, decode_tail=5)):
            H.assert_rows_match(H.replay(eng, trace), ref, 1e-6, "toy shapes on the CPU")
        assert eng.cache.free_pages() == [40, 40]
    finally:
        kernels.use_backend(None)
