"""What pins the plain model's composition (no GPU): where the residual additions, the three kinds of norm
and the output projection sit, beside the reference's text (/root/reference/src/models/block.cpp:23-29:
a = x + Attn(N1 x), y = a + MLP(N2 a); /root/reference/src/models/gpt_model.cpp:324-328: final norm, then the
output projection).

Each check builds weights for which the whole model reduces to a closed form of library routines
(`F.rms_norm`, `F.linear`, `F.silu`, `F.scaled_dot_product_attention`, a complex product for the rotation),
and the last test shows that every check does its work: models with one plausible mistake each (a dropped
residual, a norm after instead of before, a parallel block, swapped norm weights, no final norm) fail them.
"""
import torch
import torch.nn.functional as F

import plain_qwen2 as plain
from conftest import TINY_A, TINY_B, TINY_C

F64 = torch.float64


def weights_for(cfg, seed):
    """Random float64 weights under the reference's tensor names, norm weights far from one so that a norm
    weight in the wrong place shows."""
    g = torch.Generator().manual_seed(seed)
    h, nq, nkv = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim") or h // nq
    inter, vocab = cfg["intermediate_size"], cfg["vocab_size"]
    rnd = lambda *shape, std=0.3: torch.randn(*shape, generator=g, dtype=F64) * std
    w = {"model.embed_tokens.weight": rnd(vocab, h, std=1.0), "model.norm.weight": 1.0 + rnd(h, std=0.5)}
    if not cfg["tie_word_embeddings"]:
        w["lm_head.weight"] = rnd(vocab, h)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = 1.0 + rnd(h, std=0.5)
        w[p + "post_attention_layernorm.weight"] = 1.0 + rnd(h, std=0.5)
        for n, rows in (("q", nq * hd), ("k", nkv * hd), ("v", nkv * hd)):
            w[p + f"self_attn.{n}_proj.weight"] = rnd(rows, h)
            w[p + f"self_attn.{n}_proj.bias"] = rnd(rows)
        w[p + "self_attn.o_proj.weight"] = rnd(h, nq * hd)
        w[p + "mlp.gate_proj.weight"] = rnd(inter, h)
        w[p + "mlp.up_proj.weight"] = rnd(inter, h)
        w[p + "mlp.down_proj.weight"] = rnd(h, inter)
    return w


def zeroed(w, *suffixes):
    return {k: (torch.zeros_like(v) if k.endswith(suffixes) else v) for k, v in w.items()}


# ----------------------------------------------------------------------------- closed forms from library routines
def lib_norm(x, weight, cfg):
    return F.rms_norm(x, (x.shape[-1],), weight, cfg.get("rms_norm_eps", 1e-6))


def lib_head(x, w, cfg):
    x = lib_norm(x, w["model.norm.weight"], cfg)
    return F.linear(x, w["model.embed_tokens.weight" if cfg["tie_word_embeddings"] else "lm_head.weight"])


def lib_mlp(x, w, p):
    return F.linear(F.silu(F.linear(x, w[p + "gate_proj.weight"])) * F.linear(x, w[p + "up_proj.weight"]),
                    w[p + "down_proj.weight"])


def lib_attention_one_token(x, w, p, cfg):
    """A sequence of one token: its only key is its own, so the attention output is its value, query head h
    getting the value of kv head h // G; rotation and scores drop out."""
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim") or cfg["hidden_size"] // nq
    v = F.linear(x, w[p + "v_proj.weight"], w[p + "v_proj.bias"]).reshape(-1, nkv, hd)
    return F.linear(v.repeat_interleave(nq // nkv, dim=1).reshape(-1, nq * hd), w[p + "o_proj.weight"])


def lib_attention(x, w, p, cfg, window):
    """Whole sequence: the library's attention on rotated queries and keys, the rotation as a complex product."""
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim") or cfg["hidden_size"] // nq
    s, half = x.shape[0], hd // 2
    q = F.linear(x, w[p + "q_proj.weight"], w[p + "q_proj.bias"]).reshape(s, nq, hd)
    k = F.linear(x, w[p + "k_proj.weight"], w[p + "k_proj.bias"]).reshape(s, nkv, hd)
    v = F.linear(x, w[p + "v_proj.weight"], w[p + "v_proj.bias"]).reshape(s, nkv, hd)
    inv = torch.tensor([cfg["rope_theta"] ** (-2.0 * i / hd) for i in range(half)], dtype=F64)
    turn = torch.polar(torch.ones(s, half, dtype=F64), torch.arange(s, dtype=F64)[:, None] * inv)[:, None, :]

    def rotate(t):
        z = torch.complex(t[..., :half], t[..., half:]) * turn
        return torch.cat([z.real, z.imag], dim=-1)

    q, k = rotate(q), rotate(k)
    k, v = k.repeat_interleave(nq // nkv, dim=1), v.repeat_interleave(nq // nkv, dim=1)
    if window:
        i, j = torch.arange(s)[:, None], torch.arange(s)[None, :]
        mask = (j <= i) & (j > i - window)
        o = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), attn_mask=mask)
    else:
        o = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
    return F.linear(o.transpose(0, 1).reshape(s, nq * hd), w[p + "o_proj.weight"])


# ----------------------------------------------------------------------------- the checks
def composition_checks(forward, cfg, seed=0):
    """Raises AssertionError if `forward(cfg, w, ids)` does not compose the parts as the reference does."""
    w = weights_for(cfg, seed)
    layers = cfg["num_hidden_layers"]
    g = torch.Generator().manual_seed(100 + seed)
    ids = torch.randint(0, cfg["vocab_size"], (14,), generator=g).tolist()
    emb = w["model.embed_tokens.weight"][ids]
    close = lambda a, b: torch.allclose(a, b, atol=1e-9, rtol=1e-9)

    # 1. no attention output, no feed-forward output: the residual stream is the embedding, and the logits are
    #    head(final_norm(embedding)).  A dropped residual gives zeros, a missing final norm another scale.
    w0 = zeroed(w, "o_proj.weight", "down_proj.weight")
    assert close(forward(cfg, w0, ids), lib_head(emb, w0, cfg)), "embedding -> final norm -> head"

    # 2. no attention output: each layer adds MLP(N2(x)) to x, with its own post_attention_layernorm
    w1 = zeroed(w, "o_proj.weight")
    x = emb
    for i in range(layers):
        p = f"model.layers.{i}."
        x = x + lib_mlp(lib_norm(x, w1[p + "post_attention_layernorm.weight"], cfg), w1, p + "mlp.")
    assert close(forward(cfg, w1, ids), lib_head(x, w1, cfg)), "x + MLP(N2 x)"

    # 3. no feed-forward output, sequences of one token: each layer adds Wo v(N1(x)) to x, with its own
    #    input_layernorm and the value's bias
    w2 = zeroed(w, "down_proj.weight")
    for tok in ids[:3]:
        x = w2["model.embed_tokens.weight"][[tok]]
        for i in range(layers):
            p = f"model.layers.{i}."
            x = x + lib_attention_one_token(lib_norm(x, w2[p + "input_layernorm.weight"], cfg), w2, p + "self_attn.", cfg)
        assert close(forward(cfg, w2, [tok]), lib_head(x, w2, cfg)), "x + Attn(N1 x), one token"

    # 4. everything, one token: the feed-forward reads the stream after the attention's addition (a parallel
    #    block would read it before)
    for tok in ids[:3]:
        x = w["model.embed_tokens.weight"][[tok]]
        for i in range(layers):
            p = f"model.layers.{i}."
            a = x + lib_attention_one_token(lib_norm(x, w[p + "input_layernorm.weight"], cfg), w, p + "self_attn.", cfg)
            x = a + lib_mlp(lib_norm(a, w[p + "post_attention_layernorm.weight"], cfg), w, p + "mlp.")
        assert close(forward(cfg, w, [tok]), lib_head(x, w, cfg)), "a = x + Attn(N1 x); y = a + MLP(N2 a)"

    # 5. everything, the whole sequence, from library routines (windowed layers with an explicit mask)
    x = emb
    for i in range(layers):
        p = f"model.layers.{i}."
        a = x + lib_attention(lib_norm(x, w[p + "input_layernorm.weight"], cfg), w, p + "self_attn.", cfg,
                              plain.layer_window(cfg, i))
        x = a + lib_mlp(lib_norm(a, w[p + "post_attention_layernorm.weight"], cfg), w, p + "mlp.")
    got, ref = forward(cfg, w, ids), lib_head(x, w, cfg)
    # (the plain model makes its angles in float32 as the reference does, and these weights give peaked attention)
    assert float((got - ref).abs().max()) <= 1e-5 * float(ref.abs().max()), "whole sequence"

    # 6. the final norm is the last thing before the output matrix: twice its weight, twice the logits
    w3 = dict(w, **{"model.norm.weight": w["model.norm.weight"] * 2})
    assert close(forward(cfg, w3, ids), got * 2), "final norm feeds the head"


CONFIGS = [TINY_A, TINY_B, dict(TINY_C, sliding_window=5)]


def test_the_plain_model_composes_its_parts_as_the_reference_does():
    for seed, cfg in enumerate(CONFIGS):
        composition_checks(plain.forward_logits, cfg, seed)


# ----------------------------------------------------------------------------- the checks can fail
def flawed_forward(flaw):
    """plain.forward_logits with one mistake."""

    def forward(cfg, w, token_ids):
        ids = torch.as_tensor(token_ids, dtype=torch.long)
        eps = cfg.get("rms_norm_eps", 1e-6)
        x = w["model.embed_tokens.weight"][ids]
        positions = torch.arange(len(ids))
        for i in range(cfg["num_hidden_layers"]):
            p = f"model.layers.{i}."
            n1, n2 = p + "input_layernorm.weight", p + "post_attention_layernorm.weight"
            if flaw == "swapped_norm_weights":
                n1, n2 = n2, n1
            attn = lambda t: plain.self_attention_block(t, w, p + "self_attn.", cfg, positions, plain.layer_window(cfg, i))
            mlp = lambda t: plain.swiglu_mlp(t, w, p + "mlp.")
            if flaw == "post_norm":
                x = plain.rms_norm(x + attn(x), w[n1], eps)
                x = plain.rms_norm(x + mlp(x), w[n2], eps)
                continue
            if flaw == "parallel_block":
                x = x + attn(plain.rms_norm(x, w[n1], eps)) + mlp(plain.rms_norm(x, w[n2], eps))
                continue
            a = attn(plain.rms_norm(x, w[n1], eps))
            x = a if flaw == "no_attention_residual" else x + a
            m = mlp(plain.rms_norm(x, w[n2], eps))
            x = m if flaw == "no_feed_forward_residual" else x + m
        if flaw != "no_final_norm":
            x = plain.rms_norm(x, w["model.norm.weight"], eps)
        head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
        return plain.linear(x, head)

    return forward


def test_every_plausible_mistake_in_the_composition_fails_the_checks():
    composition_checks(flawed_forward(None), TINY_B, 1)          # the harness itself, without a flaw, passes
    for flaw in ("no_attention_residual", "no_feed_forward_residual", "post_norm", "parallel_block",
                 "swapped_norm_weights", "no_final_norm"):
        for seed, cfg in enumerate(CONFIGS):
            try:
                composition_checks(flawed_forward(flaw), cfg, seed)
            except AssertionError:
                continue
            raise AssertionError(f"a model with the flaw '{flaw}' passed the composition checks")
