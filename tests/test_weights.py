"""Weights file reading, validation errors and the random-weights mode (no GPU)."""
import json
import os
import struct

import pytest
import torch

from conftest import TINY_A, TINY_B
from easy_gpt.cpp_amd.config import resolve_architecture
from easy_gpt.cpp_amd.parts import build_model
from easy_gpt.cpp_amd.weights import (
    CheckedWeights, SafetensorsError, SafetensorsFile, WeightsError, random_tensors, write_random_model,
    write_safetensors,
)


def model_for(cfg):
    arch = resolve_architecture(cfg)
    return build_model(arch.build_spec(arch.config_class.from_dict(cfg)))


# fixture of the reference's validation test: 1 layer, H=4, nq=2, nkv=1, V=10
# (/root/reference/test/model_param_validation_test.cpp:201-215)
FIXTURE = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": 1, "hidden_size": 4,
    "num_attention_heads": 2, "num_key_value_heads": 1, "intermediate_size": 6, "vocab_size": 10,
    "rope_theta": 10000.0, "max_position_embeddings": 32, "tie_word_embeddings": True,
}


def write_fixture(d, mutate=None, dtype=torch.float32):
    model = model_for(FIXTURE)
    tensors = random_tensors(model.param_specs(), 0, dtype)
    if mutate:
        mutate(tensors)
    os.makedirs(d, exist_ok=True)
    write_safetensors(os.path.join(d, "model.safetensors"), tensors)
    return model


def test_roundtrip_and_dtypes(tmp_path):
    t = {
        "a": torch.randn(3, 5), "b": torch.randn(4).to(torch.bfloat16), "c": torch.randn(2, 2).to(torch.float16),
        "d": torch.arange(6, dtype=torch.int64).reshape(2, 3), "e": torch.arange(4, dtype=torch.int32),
    }
    p = str(tmp_path / "model.safetensors")
    write_safetensors(p, t, metadata={"format": "pt"})
    with SafetensorsFile(p) as f:
        assert set(f.names()) == set(t)                      # __metadata__ is skipped
        for k, v in t.items():
            got = f.read(k)
            assert got.dtype == v.dtype and got.shape == v.shape and torch.equal(got, v)


def test_stored_dtype_rules(tmp_path):
    # bfloat16 stays, float16 becomes float32 (exactly), float32 stays, int64 becomes int32
    from easy_gpt.cpp_amd.parts import ParamSpec

    t = {"w": torch.randn(3, 5).to(torch.bfloat16), "h": torch.randn(2).to(torch.float16), "f": torch.randn(2),
         "i": torch.arange(5, dtype=torch.int64)}
    write_safetensors(str(tmp_path / "model.safetensors"), t)
    specs = [ParamSpec("w", (3, 5)), ParamSpec("h", (2,)), ParamSpec("f", (2,)), ParamSpec("i", (5,), "int_table", "int32")]
    cw = CheckedWeights(str(tmp_path), specs)
    assert cw.get("w").dtype == torch.bfloat16 and torch.equal(cw.get("w"), t["w"])
    assert cw.get("h").dtype == torch.float32 and torch.equal(cw.get("h"), t["h"].float())
    assert cw.get("f").dtype == torch.float32 and torch.equal(cw.get("f"), t["f"])
    assert cw.get("i").dtype == torch.int32 and cw.get("i").tolist() == [0, 1, 2, 3, 4]
    cw.close()


def test_float16_checkpoint_is_rounded_once_on_the_way_to_the_engine(tmp_path):
    # The reference decodes every stored element through float32 into the build's dtype
    # (/root/reference/src/models/loader.cpp:173-198): a float32 engine holds the stored float16 values exactly,
    # a bfloat16 engine rounds them once.
    from easy_gpt.cpp_amd.parts import ParamSpec
    from easy_gpt.cpp_amd.parts.base import Part

    g = torch.Generator().manual_seed(3)
    h = (torch.randn(64, 7, generator=g) * 0.02).to(torch.float16)
    assert not torch.equal(h.to(torch.bfloat16).float(), h.float())      # these values do not fit bfloat16
    write_safetensors(str(tmp_path / "model.safetensors"), {"h": h})
    cw = CheckedWeights(str(tmp_path), [ParamSpec("h", (64, 7))])
    got = cw.get("h")
    cw.close()
    assert torch.equal(Part._to(got, "compute", torch.float32, "cpu"), h.float())
    assert torch.equal(Part._to(got, "compute", torch.bfloat16, "cpu"), h.float().to(torch.bfloat16))


def test_file_format_agrees_with_the_safetensors_library(tmp_path):
    # The format is pinned by something other than this repository's own writer: a file the library writes is
    # read the same by SafetensorsFile, and a file write_safetensors writes is read the same by the library.
    st = pytest.importorskip("safetensors.torch")
    g = torch.Generator().manual_seed(4)
    t = {
        "model.a": torch.randn(3, 5, generator=g), "b": torch.randn(17, generator=g).to(torch.bfloat16),
        "c.h": torch.randn(2, 2, 3, generator=g).to(torch.float16), "i": torch.arange(6, dtype=torch.int64).reshape(2, 3),
        "j": torch.arange(4, dtype=torch.int32),
    }
    theirs, ours = str(tmp_path / "theirs.safetensors"), str(tmp_path / "ours.safetensors")
    st.save_file(t, theirs, metadata={"format": "pt"})
    with SafetensorsFile(theirs) as f:
        assert set(f.names()) == set(t)
        for k, v in t.items():
            got = f.read(k)
            assert got.dtype == v.dtype and got.shape == v.shape and torch.equal(got, v), k
    write_safetensors(ours, t, metadata={"format": "pt", "seed": "4"})
    back = st.load_file(ours)
    assert set(back) == set(t)
    for k, v in t.items():
        assert back[k].dtype == v.dtype and torch.equal(back[k], v), k


def test_complete_set_validates(tmp_path):
    model = write_fixture(str(tmp_path))
    cw = CheckedWeights(str(tmp_path), model.param_specs())
    assert cw.get("model.embed_tokens.weight").shape == (10, 4)
    cw.close()


def test_checkpoint_in_several_files_with_an_index(tmp_path):
    model = model_for(FIXTURE)
    tensors = random_tensors(model.param_specs(), 0, torch.float32)
    names = list(tensors)
    parts = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    for fname, part in parts.items():
        write_safetensors(str(tmp_path / fname), {n: tensors[n] for n in part})
    index = {"metadata": {}, "weight_map": {n: f for f, part in parts.items() for n in part}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    cw = CheckedWeights(str(tmp_path), model.param_specs())
    for n in names:
        assert torch.equal(cw.get(n), tensors[n])
    cw.close()
    # a tensor that the index sends to the wrong file, a missing file, and a missing tensor
    bad = dict(index, weight_map=dict(index["weight_map"], **{names[0]: "model-00002-of-00002.safetensors"}))
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(bad))
    with pytest.raises(WeightsError, match="is not in"):
        CheckedWeights(str(tmp_path), model.param_specs())
    bad = dict(index, weight_map=dict(index["weight_map"], **{names[0]: "gone.safetensors"}))
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(bad))
    with pytest.raises(SafetensorsError, match="not found"):
        CheckedWeights(str(tmp_path), model.param_specs())
    os.remove(tmp_path / "model-00002-of-00002.safetensors")
    write_safetensors(str(tmp_path / "model-00002-of-00002.safetensors"), {n: tensors[n] for n in names[3::2]})
    short = {n: f for n, f in index["weight_map"].items() if n != names[1]}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": short}))
    with pytest.raises(WeightsError) as e:
        CheckedWeights(str(tmp_path), model.param_specs())
    assert e.value.missing == [names[1]]
    (tmp_path / "model.safetensors.index.json").write_text("{}")
    with pytest.raises(WeightsError, match="weight_map"):
        CheckedWeights(str(tmp_path), model.param_specs())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    def mutate(t):
        del t["model.layers.0.self_attn.k_proj.weight"]           # missing, as in the reference's test :372
        del t["model.layers.0.mlp.up_proj.weight"]
        t["model.embed_tokens.weight"] = torch.zeros(9, 4)         # wrong shape [9,4], reference :389
        t["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(3)
        t["model.layers.0.extra.weight"] = torch.zeros(2)          # unexpected
        t["something_else"] = torch.zeros(1)

    model = write_fixture(str(tmp_path), mutate)
    with pytest.raises(WeightsError) as e:
        CheckedWeights(str(tmp_path), model.param_specs())
    err = e.value
    assert sorted(err.missing) == ["model.layers.0.mlp.up_proj.weight", "model.layers.0.self_attn.k_proj.weight"]
    assert sorted(err.unexpected) == ["model.layers.0.extra.weight", "something_else"]
    assert sorted(n for n, _, _ in err.wrong_shape) == ["model.embed_tokens.weight", "model.layers.0.self_attn.q_proj.bias"]
    msg = str(err)
    for word in ["missing", "unexpected", "wrong shapes", "k_proj.weight", "something_else", "[9, 4]", "[10, 4]"]:
        assert word in msg


def test_tied_model_ignores_a_stray_output_matrix_but_untied_needs_it(tmp_path):
    def mutate(t):
        t["lm_head.weight"] = torch.zeros(10, 4)

    model = write_fixture(str(tmp_path / "tied"), mutate)
    cw = CheckedWeights(str(tmp_path / "tied"), model.param_specs(), model.spec.ignorable_tensors)
    assert cw.ignored == ["lm_head.weight"]
    cw.close()
    untied = model_for(dict(FIXTURE, tie_word_embeddings=False))
    write_fixture(str(tmp_path / "untied"))
    with pytest.raises(WeightsError) as e:
        CheckedWeights(str(tmp_path / "untied"), untied.param_specs(), untied.spec.ignorable_tensors)
    assert e.value.missing == ["lm_head.weight"]


def test_norm_weight_may_be_a_column(tmp_path):
    # [H, 1] is accepted for a norm weight (/root/reference/test/mlp_cuda_test.cpp:150-178)
    def mutate(t):
        t["model.norm.weight"] = t["model.norm.weight"].reshape(4, 1)

    model = write_fixture(str(tmp_path), mutate)
    CheckedWeights(str(tmp_path), model.param_specs()).close()


def _raw_file(path, header: dict, data: bytes):
    h = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + data)


def test_file_format_errors(tmp_path):
    p = str(tmp_path / "model.safetensors")
    _raw_file(p, {"x": {"dtype": "I8", "shape": [4], "data_offsets": [0, 4]}}, b"\0" * 4)
    with pytest.raises(SafetensorsError, match="unsupported dtype"):      # reference test :345 rejects I8
        SafetensorsFile(p)
    _raw_file(p, {"x": {"dtype": "F32", "shape": [4], "data_offsets": [0, 12]}}, b"\0" * 16)
    with pytest.raises(SafetensorsError, match="needs 16"):
        SafetensorsFile(p)
    _raw_file(p, {"x": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="outside"):
        SafetensorsFile(p)
    _raw_file(p, {"x": {"dtype": "F32", "shape": [-1], "data_offsets": [0, 4]}}, b"\0" * 4)
    with pytest.raises(SafetensorsError, match="invalid shape"):
        SafetensorsFile(p)
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(p)
    with pytest.raises(SafetensorsError, match="not found"):
        SafetensorsFile(str(tmp_path / "nothing.safetensors"))


def test_random_weights_folder(tmp_path):
    d1 = write_random_model(str(tmp_path / "m1"), TINY_B, seed=1)
    d2 = write_random_model(str(tmp_path / "m2"), TINY_B, seed=1)
    d3 = write_random_model(str(tmp_path / "m3"), TINY_B, seed=2)
    assert json.load(open(os.path.join(d1, "config.json"))) == TINY_B
    f1, f2, f3 = (SafetensorsFile(os.path.join(d, "model.safetensors")) for d in (d1, d2, d3))
    model = model_for(TINY_B)
    assert set(f1.names()) == {s.name for s in model.param_specs()}
    for s in model.param_specs():
        a, b, c = f1.read(s.name), f2.read(s.name), f3.read(s.name)
        assert a.dtype == torch.float32 and tuple(a.shape) == s.shape
        assert torch.equal(a, b) and not torch.equal(a, c)           # the seed decides, nothing else
    w = f1.read("model.layers.1.mlp.down_proj.weight")
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    n = f1.read("model.layers.2.input_layernorm.weight")
    assert abs(float(n.mean()) - 1.0) < 0.02
    b = f1.read("model.layers.0.self_attn.q_proj.bias")
    assert 0.005 < float(b.std()) < 0.04
    for f in (f1, f2, f3):
        f.close()
    bf = write_random_model(str(tmp_path / "m4"), TINY_A, seed=0, dtype=torch.bfloat16)
    with SafetensorsFile(os.path.join(bf, "model.safetensors")) as f:
        assert f.read("model.embed_tokens.weight").dtype == torch.bfloat16


def test_random_values_are_a_function_of_seed_name_and_index():
    # element i of a tensor depends on (seed, tensor name, i) and on nothing else: not on the tensor's shape, not on how
    # many elements are drawn at a time, and (integer arithmetic only) not on the device; pinned by a few values, so
    # that a change of the generator shows
    from easy_gpt.cpp_amd.parts.spec import ParamSpec
    from easy_gpt.cpp_amd.weights import RandomWeights, random_init, random_tensor

    a = random_tensor(ParamSpec("w", (7, 11)), seed=3, device="cpu")
    b = random_tensor(ParamSpec("w", (77,)), seed=3, device="cpu")
    assert torch.equal(a.flatten(), b)
    assert not torch.equal(b, random_tensor(ParamSpec("v", (77,)), seed=3, device="cpu"))
    chunk = random_init._CHUNK
    try:
        random_init._CHUNK = 13
        assert torch.equal(b, random_tensor(ParamSpec("w", (77,)), seed=3, device="cpu"))
    finally:
        random_init._CHUNK = chunk
    big = random_tensor(ParamSpec("m", (400, 500)), seed=1, device="cpu").double()
    assert abs(float(big.mean())) < 2e-4 and abs(float(big.std()) - 0.02) < 2e-4
    kurtosis = float((big ** 4).mean() / (big ** 2).mean() ** 2)
    assert 2.7 < kurtosis < 3.0 and float(big.abs().max()) < 4.9 * 0.02        # a sum of eight uniforms: nearly normal
    assert [round(v, 6) for v in big[0, :4].tolist()] == [0.03894, -0.020119, 0.008327, 0.003933]
    table = random_tensor(ParamSpec("t", (5,), role="int_table", dtype="int32"), seed=1, device="cpu")
    assert table.tolist() == [14619, 23638, 5612, 9413, 15729]
    # the source without a file hands out the same tensors, in the stored dtype
    specs = [ParamSpec("w", (7, 11)), ParamSpec("s", (9,), role="norm_scale")]
    src = RandomWeights(specs, seed=3, dtype=torch.bfloat16, device="cpu")
    assert torch.equal(src.get("w"), a.to(torch.bfloat16)) and src.get("s").dtype == torch.bfloat16
    with pytest.raises(KeyError):
        src.get("missing")
