"""Pins for the plain implementation (no GPU): vectors the reference's tests hold, special cases that
reduce to a library routine, and invariants, each chosen so that a plausible mistake fails it."""
import math

import torch
import torch.nn.functional as F

import plain_qwen2 as plain

F64 = torch.float64


# ----------------------------------------------------------------------------- linear
def test_linear_vector_of_the_reference():
    # /root/reference/test/matmul_3d_test.cpp:60-87: bias path == no-bias path + manual add
    x = torch.tensor([[1.0, 2, 3], [4, 5, 6]], dtype=F64)
    w = torch.tensor([[1.0, 0, -1], [2, 3, 4]], dtype=F64)
    b = torch.tensor([0.5, -1.0], dtype=F64)
    assert torch.equal(plain.linear(x, w, b), torch.tensor([[-1.5, 19.0], [-1.5, 46.0]], dtype=F64))
    assert torch.equal(plain.linear(x, w), plain.linear(x, w, b) - b)
    assert torch.allclose(plain.linear(x, w, b), F.linear(x, w, b))


# ----------------------------------------------------------------------------- rmsnorm
def test_rms_norm_matches_library_and_pins_eps_place():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 24, generator=g, dtype=F64)
    w = torch.randn(24, generator=g, dtype=F64)
    for eps in (1e-6, 1e-5, 0.3):
        assert torch.allclose(plain.rms_norm(x, w, eps), F.rms_norm(x, (24,), w, eps), atol=1e-14)
    # constant input c with unit weight gives c / sqrt(c^2 + eps): eps is inside the root, added to the mean
    c, eps = 0.01, 1e-3
    y = plain.rms_norm(torch.full((1, 8), c, dtype=F64), torch.ones(8, dtype=F64), eps)
    assert torch.allclose(y, torch.full((1, 8), c / math.sqrt(c * c + eps), dtype=F64), atol=1e-15)
    # a column weight [H, 1] is read as [H] (/root/reference/test/mlp_cuda_test.cpp:150-178)
    assert torch.equal(plain.rms_norm(x, w.reshape(24, 1), 1e-6), plain.rms_norm(x, w, 1e-6))
    # the inline oracle of /root/reference/test/mlp_cuda_test.cpp:28-53
    ss = (x * x).sum(-1, keepdim=True)
    assert torch.allclose(plain.rms_norm(x, w, 1e-6), x * (1.0 / torch.sqrt(ss / 24 + 1e-6)) * w, atol=1e-14)


# ----------------------------------------------------------------------------- rope
def rope_input():
    # the tensor of /root/reference/test/rope_test.cpp:82-93: values ((i % 17) - 8) / 7, [batch 2, heads 2, seq 3, hd 4]
    vals = torch.tensor([((i % 17) - 8) / 7.0 for i in range(2 * 2 * 3 * 4)], dtype=F64)
    return vals.reshape(2, 2, 3, 4)


def test_rope_offsets_of_the_reference():
    # per-sample offsets {-1, 2} equal per-slice scalar offsets, theta 1e6 (/root/reference/test/rope_test.cpp:95-115)
    base = rope_input()
    theta = 1e6
    for b, off in enumerate([-1, 2]):
        x = base[b].permute(1, 0, 2)                      # [seq, heads, hd]
        pos = torch.arange(3) + off
        out = plain.rope(x, pos, theta)
        # hand-written pairs (k, k + hd/2) with the float32 frequency table
        inv = [1.0 / (theta ** (2.0 * k / 4)) for k in range(2)]
        for s in range(3):
            for h in range(2):
                for k in range(2):
                    ang = float(pos[s]) * inv[k]
                    x1, x2 = float(x[s, h, k]), float(x[s, h, k + 2])
                    assert abs(float(out[s, h, k]) - (x1 * math.cos(ang) - x2 * math.sin(ang))) < 1e-6
                    assert abs(float(out[s, h, k + 2]) - (x1 * math.sin(ang) + x2 * math.cos(ang))) < 1e-6


def test_rope_is_a_complex_multiplication():
    # The pair (x_k, x_{k+hd/2}) read as the complex number x_k + i x_{k+hd/2} is multiplied by exp(i pos inv_freq_k):
    # the library's complex product stands in for the two lines of /root/reference/src/ops.cpp:416-417.  A wrong
    # sign, a swapped sine and cosine or interleaved pairs fail this.
    g = torch.Generator().manual_seed(11)
    for hd, theta in ((8, 10000.0), (6, 1e6)):
        x = torch.randn(7, 3, hd, generator=g, dtype=F64)
        pos = torch.tensor([0, 1, 2, 5, 40, 41, 1000])
        half = hd // 2
        inv = torch.tensor([theta ** (-2.0 * k / hd) for k in range(half)], dtype=F64)
        z = torch.complex(x[..., :half], x[..., half:]) * torch.polar(torch.ones(7, half, dtype=F64), pos[:, None].double() * inv)[:, None, :]
        ref = torch.cat([z.real, z.imag], dim=-1)
        # the plain implementation makes its angles in float32 as the reference does: 1e-7 relative on an angle of 1000
        assert torch.allclose(plain.rope(x, pos, theta), ref, atol=2e-4)
        assert torch.allclose(plain.rope(x[:4], pos[:4], theta), ref[:4], atol=1e-6)


def test_rope_invariants():
    g = torch.Generator().manual_seed(1)
    q = torch.randn(6, 2, 8, generator=g, dtype=F64)
    k = torch.randn(6, 2, 8, generator=g, dtype=F64)
    pos = torch.arange(6)
    theta = 10000.0
    # position 0 is the identity
    assert torch.allclose(plain.rope(q, torch.zeros(6, dtype=torch.long), theta), q, atol=1e-15)
    # pairs (k, k + hd/2) keep their norm; interleaved pairs (2k, 2k+1) would not in general
    r = plain.rope(q, pos, theta)
    assert torch.allclose(r[..., :4] ** 2 + r[..., 4:] ** 2, q[..., :4] ** 2 + q[..., 4:] ** 2, atol=1e-12)
    inter = r[..., 0::2] ** 2 + r[..., 1::2] ** 2
    assert not torch.allclose(inter, q[..., 0::2] ** 2 + q[..., 1::2] ** 2, atol=1e-6)
    # <R_m q, R_n k> depends on m - n only (a wrong sign in one of the two lines breaks this)
    def dots(shift):
        rq, rk = plain.rope(q, pos + shift, theta), plain.rope(k, pos + shift, theta)
        return torch.einsum("ihd,jhd->hij", rq, rk)
    assert torch.allclose(dots(0), dots(5), atol=1e-5)       # float32 angles limit this
    # the rotation is by +angle: feature 0 of e_0 at position 1 becomes cos(1), feature hd/2 becomes +sin(1)
    e = torch.zeros(1, 1, 8, dtype=F64)
    e[0, 0, 0] = 1.0
    out = plain.rope(e, torch.tensor([1]), theta)
    assert abs(float(out[0, 0, 0]) - math.cos(1.0)) < 1e-7 and abs(float(out[0, 0, 4]) - math.sin(1.0)) < 1e-7
    # frequency table: 1 / theta^(2k/hd)
    inv = plain.rope_inv_freq(8, theta)
    assert torch.allclose(inv.double(), torch.tensor([theta ** (-2 * k / 8) for k in range(4)], dtype=F64), rtol=1e-6)


# ----------------------------------------------------------------------------- attention
def test_attention_reduces_to_library_routine():
    g = torch.Generator().manual_seed(2)
    s, nq, nkv, hd = 9, 6, 2, 8
    q = torch.randn(s, nq, hd, generator=g, dtype=F64)
    k = torch.randn(s, nkv, hd, generator=g, dtype=F64)
    v = torch.randn(s, nkv, hd, generator=g, dtype=F64)
    out = plain.attention(q, k, v, nq, nkv)
    kk = k.repeat_interleave(nq // nkv, dim=1)            # query head h reads kv head h // G
    vv = v.repeat_interleave(nq // nkv, dim=1)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True)
    assert torch.allclose(out, ref.transpose(0, 1), atol=1e-12)
    # the other plausible mapping (h % nkv) is different
    k_bad = torch.cat([k] * (nq // nkv), dim=1)
    v_bad = torch.cat([v] * (nq // nkv), dim=1)
    bad = F.scaled_dot_product_attention(q.transpose(0, 1), k_bad.transpose(0, 1), v_bad.transpose(0, 1), is_causal=True)
    assert not torch.allclose(out, bad.transpose(0, 1), atol=1e-3)
    # nkv == nq is plain multi-head attention; one head too
    out1 = plain.attention(q[:, :1], k[:, :1], v[:, :1], 1, 1)
    ref1 = F.scaled_dot_product_attention(q[:, :1].transpose(0, 1), k[:, :1].transpose(0, 1), v[:, :1].transpose(0, 1), is_causal=True)
    assert torch.allclose(out1, ref1.transpose(0, 1), atol=1e-12)


def test_attention_special_cases():
    g = torch.Generator().manual_seed(3)
    q = torch.randn(5, 2, 4, generator=g, dtype=F64)
    k = torch.randn(5, 1, 4, generator=g, dtype=F64)
    v = torch.randn(5, 1, 4, generator=g, dtype=F64)
    out = plain.attention(q, k, v, 2, 1)
    assert torch.allclose(out[0], v[0].expand(2, 4), atol=1e-14)         # one visible key: the output is its value
    const = torch.ones(5, 1, 4, dtype=F64) * 0.7
    assert torch.allclose(plain.attention(q, k, const, 2, 1), torch.full((5, 2, 4), 0.7, dtype=F64), atol=1e-14)
    # window W: the query sees itself and W-1 keys before it
    w3 = plain.attention(q, k, v, 2, 1, window=3)
    assert torch.allclose(w3[:3], out[:3], atol=1e-14)                   # fewer than W keys: same as causal
    tail = plain.attention(q[2:], k[2:], v[2:], 2, 1)                    # keys 2..4 only
    assert torch.allclose(w3[4], tail[2], atol=1e-14)
    w1 = plain.attention(q, k, v, 2, 1, window=1)
    assert torch.allclose(w1, v.expand(5, 2, 4), atol=1e-14)


# ----------------------------------------------------------------------------- feed-forward
def test_swiglu():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(3, 8, generator=g, dtype=F64)
    w = {"p.up_proj.weight": torch.randn(16, 8, generator=g, dtype=F64),
         "p.gate_proj.weight": torch.randn(16, 8, generator=g, dtype=F64),
         "p.down_proj.weight": torch.randn(8, 16, generator=g, dtype=F64)}
    ref = F.linear(F.silu(F.linear(x, w["p.gate_proj.weight"])) * F.linear(x, w["p.up_proj.weight"]), w["p.down_proj.weight"])
    assert torch.allclose(plain.swiglu_mlp(x, w, "p."), ref, atol=1e-12)
    # the gate is the activated branch: swapping the two gives something else
    sw = dict(w)
    sw["p.up_proj.weight"], sw["p.gate_proj.weight"] = w["p.gate_proj.weight"], w["p.up_proj.weight"]
    assert not torch.allclose(plain.swiglu_mlp(x, sw, "p."), ref, atol=1e-3)
    # silu(0) = 0: a zero gate gives a zero output whatever up is
    z = dict(w)
    z["p.gate_proj.weight"] = torch.zeros(16, 8, dtype=F64)
    assert torch.equal(plain.swiglu_mlp(x, z, "p."), torch.zeros(3, 8, dtype=F64))


# ----------------------------------------------------------------------------- whole model
def test_whole_model_invariants(tiny_models):
    for name in ("A", "B", "C"):
        cfg, w = plain.read_model(tiny_models[name])
        g = torch.Generator().manual_seed(7)
        ids = torch.randint(0, cfg["vocab_size"], (30,), generator=g).tolist()
        logits = plain.forward_logits(cfg, w, ids)
        assert logits.shape == (30, cfg["vocab_size"])
        # causality: logits at a position do not change when later tokens change
        ids2 = ids[:20] + [(t + 1) % cfg["vocab_size"] for t in ids[20:]]
        assert torch.allclose(plain.forward_logits(cfg, w, ids2)[:20], logits[:20], atol=1e-12)
        # only distances count: shifting all positions changes nothing (up to float32 angles)
        shifted = plain.forward_logits(cfg, w, ids, first_position=3)
        assert torch.allclose(shifted, logits, atol=5e-5)
        # tied or not decides which matrix makes the logits
        if cfg["tie_word_embeddings"]:
            # a stray output matrix in the file is not used, and the logits are those of an untied model whose
            # output matrix is a copy of the embedding table
            stray = dict(w, **{"lm_head.weight": torch.ones_like(w["model.embed_tokens.weight"])})
            assert torch.equal(plain.forward_logits(cfg, stray, ids), logits)
            untied = dict(w, **{"lm_head.weight": w["model.embed_tokens.weight"].clone()})
            assert torch.equal(plain.forward_logits(dict(cfg, tie_word_embeddings=False), untied, ids), logits)
            # doubling the table doubles the logits (the norms undo the doubling of the residual stream up to eps)
            doubled = dict(w, **{"model.embed_tokens.weight": w["model.embed_tokens.weight"] * 2})
            assert not torch.allclose(plain.forward_logits(cfg, doubled, ids), logits, atol=1e-3)
        else:
            doubled = dict(w, **{"lm_head.weight": w["lm_head.weight"] * 2})
            assert torch.allclose(plain.forward_logits(cfg, doubled, ids), logits * 2, atol=1e-9)
            # the embedding table is not the output matrix: changing only the rows of tokens that are not in the
            # sequence changes nothing
            absent = [t for t in range(cfg["vocab_size"]) if t not in set(ids)]
            other = w["model.embed_tokens.weight"].clone()
            other[absent] += 1.0
            assert torch.equal(plain.forward_logits(cfg, dict(w, **{"model.embed_tokens.weight": other}), ids), logits)


def test_window_matters_in_config_c(tiny_models):
    cfg, w = plain.read_model(tiny_models["C"])
    g = torch.Generator().manual_seed(8)
    ids = torch.randint(0, cfg["vocab_size"], (60,), generator=g).tolist()
    with_window = plain.forward_logits(cfg, w, ids)
    no_window = plain.forward_logits(dict(cfg, use_sliding_window=False), w, ids)
    assert torch.allclose(with_window[:24], no_window[:24], atol=1e-12)       # window 24: the first 24 see everything
    assert not torch.allclose(with_window[40:], no_window[40:], atol=1e-4)


def test_norm_eps_and_theta_matter(tiny_models):
    cfg, w = plain.read_model(tiny_models["B"])
    ids = list(range(3, 40))
    base = plain.forward_logits(cfg, w, ids)
    assert not torch.allclose(plain.forward_logits(dict(cfg, rms_norm_eps=1e-2), w, ids), base, atol=1e-3)
    assert not torch.allclose(plain.forward_logits(dict(cfg, rope_theta=100.0), w, ids), base, atol=1e-4)


# ----------------------------------------------------------------------------- sampling
def test_sampling_distribution():
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(50, generator=g, dtype=F64) * 2
    # p^(1/T) renormalised is softmax(logits / T) (/root/reference/src/sampler.cpp:50-57)
    for t in (0.5, 0.8, 1.0, 1.7):
        d = plain.sampling_distribution(logits, t)
        assert torch.allclose(d, torch.softmax(logits / t, -1), atol=1e-12)
    d = plain.sampling_distribution(logits, 1.0, top_k=5)
    assert int((d > 0).sum()) == 5 and set(d.topk(5).indices.tolist()) == set(logits.topk(5).indices.tolist())
    assert abs(float(d.sum()) - 1) < 1e-12
    d = plain.sampling_distribution(logits, 1.0, top_p=0.6)
    p = torch.softmax(logits, -1)
    kept = (d > 0)
    assert float(p[kept].sum()) >= 0.6 and float(p[kept].sum() - p[kept].min()) < 0.6      # smallest such set
    assert plain.greedy(torch.tensor([1.0, 3.0, 3.0, 2.0])) == 1                             # first maximum wins
