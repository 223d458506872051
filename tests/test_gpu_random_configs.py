"""Configurations drawn at random (seeded): every size and option the configuration allows, in combinations that
no hand-made configuration has, through the four cuttings in both precisions against the plain implementation.
Head sizes in steps of 16 up to 256, any number of heads and groups, widths and vocabularies that are no power of
two, windows on some layers, tied or not, page sizes from 4 to 64."""
import random

import pytest

import helpers as H

pytestmark = pytest.mark.gpu


def drawn_config(seed: int) -> dict:
    rng = random.Random(7700 + seed)
    nkv = rng.choice([1, 1, 2, 3, 5])
    nq = nkv * rng.choice([1, 2, 3, 4, 7, 8])
    hd = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 256])
    if nq * hd > 1536:
        hd = 16
    hidden = nq * hd if rng.random() < 0.5 else rng.choice([40, 56, 72, 88, 100, 136, 200, 264, 328])
    return {
        "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
        "num_hidden_layers": rng.randint(1, 3), "hidden_size": hidden, "num_attention_heads": nq, "num_key_value_heads": nkv,
        "head_dim": hd, "intermediate_size": rng.choice([24, 100, 177, 200, 333, 520]),
        "vocab_size": rng.choice([97, 300, 777, 1001, 5003, 9001]),
        "rope_theta": rng.choice([1e4, 5e4, 1e6]), "rms_norm_eps": rng.choice([1e-6, 1e-5, 3e-6]),
        "tie_word_embeddings": rng.random() < 0.5, "max_position_embeddings": rng.choice([128, 256, 400]), "hidden_act": "silu",
        "use_sliding_window": rng.random() < 0.35, "sliding_window": rng.choice([8, 24, 50]), "max_window_layers": rng.randint(0, 2),
        "bos_token_id": 1, "eos_token_id": 2, "torch_dtype": "float32",
    }


@pytest.mark.parametrize("seed", range(10))
def test_a_drawn_configuration_agrees_with_plain(tmp_path, seed):
    from easy_gpt.cpp_amd.engine import Engine
    from easy_gpt.cpp_amd.weights import write_random_model

    cfg = drawn_config(seed)
    rng = random.Random(seed)
    what = {k: cfg[k] for k in ("num_hidden_layers", "hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim",
                                "intermediate_size", "vocab_size", "tie_word_embeddings", "use_sliding_window",
                                "sliding_window", "max_window_layers")}
    print(f"configuration {seed}: {what}", flush=True)
    folder = write_random_model(str(tmp_path / "drawn"), cfg, seed)
    cap = cfg["max_position_embeddings"]
    reqs = H.make_requests(cfg["vocab_size"], [rng.randint(1, cap) for _ in range(3)] + [min(cap, 100)], seed=seed)
    for dtype in ("float32", "bfloat16"):
        # (scores of a size that a wrong or stale key would show at, as in the hand-made configurations)
        gain = ((2.5 if dtype == "float32" else 0.9) / (0.0004 * cfg["hidden_size"])) ** 0.5
        model = H.sharpen_attention(folder, str(tmp_path / f"sharp_{dtype}"), gain)
        ref = H.plain_rows(model, reqs, bf16_weights=(dtype == "bfloat16"))
        for name, trace in (("whole", H.trace_whole(reqs)), ("last decoded", H.trace_last_decoded(reqs)),
                            ("portions", H.trace_portions(reqs, seed=seed)), ("mixed", H.trace_mixed(reqs, seed=seed))):
            page = rng.choice([16, 16, 32, 8, 64, 4])
            eng = Engine.from_dir(model, dtype=dtype, device="cuda:0", page_size=page,
                                  max_tokens=H.max_live_tokens(trace, max(page, 64)), max_requests=4)
            rows = H.replay(eng, trace)
            assert len(rows) == sum(len(v) for v in reqs.values())
            H.assert_rows_match(rows, ref, H.FP32_TOL if dtype == "float32" else H.BF16_TOL,
                                f"configuration {seed} {what}, {dtype}, {name}, page size {page}")
            assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]
            del eng
