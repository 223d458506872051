"""A plain, slow Qwen2 decoder written from the reference's formulas.

Whole sequences, no cache, one function per part, float64 on the CPU.  It shares
no code with the engine: it reads a model folder with its own few lines and knows
the tensor names itself.  Every function cites the place in /root/reference that
fixes its formula.  The reference was read, not run.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np
import torch

F64 = torch.float64


# ----------------------------------------------------------------------------- reading a model folder
def read_safetensors(path: str) -> dict[str, torch.Tensor]:
    """u64 header length, JSON header, raw data (/root/reference/src/models/loader.cpp:213-252,298-310)."""
    with open(path, "rb") as f:
        raw = f.read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8 : 8 + hlen])
    base = 8 + hlen
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        buf = raw[base + b : base + e]
        if info["dtype"] == "F32":
            a = torch.from_numpy(np.frombuffer(buf, dtype="<f4").copy())
        elif info["dtype"] == "BF16":
            u16 = np.frombuffer(buf, dtype="<u2").astype(np.uint32) << 16
            a = torch.from_numpy(u16.view(np.float32).copy())
        else:
            raise ValueError(info["dtype"])
        out[name] = a.reshape(info["shape"]).to(F64)
    return out


def read_model(model_dir: str, round_to_bf16: bool = False, device: str = "cpu"):
    """(config.json as a dict, {tensor name: float64 tensor}).  `device`: where the tensors are kept and the
    model is computed; the functions below are the same torch code on any device (large shapes take minutes on
    the CPU)."""
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = read_safetensors(os.path.join(model_dir, "model.safetensors"))
    if round_to_bf16:
        w = {k: v.to(torch.float32).to(torch.bfloat16).to(F64) for k, v in w.items()}
    if device != "cpu":
        w = {k: v.to(device) for k, v in w.items()}
    return cfg, w


# ----------------------------------------------------------------------------- parts
def linear(x, weight, bias=None):
    """y = x W^T + b, W is [out, in] (/root/reference/src/ops.cpp:101-118)."""
    y = x @ weight.transpose(-1, -2)
    return y if bias is None else y + bias


def rms_norm(x, weight, eps):
    """ss = sum x^2; inv = 1/sqrt(ss/H + eps); y = w * (x * inv)
    (/root/reference/src/models/norm.cpp:47-59; eps inside the square root at :54)."""
    mean_sq = (x * x).sum(-1, keepdim=True) / x.shape[-1]
    return weight.reshape(-1) * (x * (1.0 / torch.sqrt(mean_sq + eps)))


def rope_inv_freq(head_dim, theta):
    """inv_freq_k = 1 / theta^(2k/hd), k < hd/2, in float32 as the reference makes it
    (/root/reference/src/ops.cpp:170-175)."""
    k = torch.arange(head_dim // 2, dtype=torch.float32)
    freq = torch.pow(torch.tensor(theta, dtype=torch.float32), (2.0 * k) / float(head_dim))
    return (1.0 / freq).to(torch.float32)


def rope(x, positions, theta):
    """x [S, heads, hd]; pairs (k, k + hd/2); angle = float(pos) * inv_freq_k in float32;
    x1' = x1 cos - x2 sin, x2' = x1 sin + x2 cos (/root/reference/src/ops.cpp:404-420)."""
    hd = x.shape[-1]
    half = hd // 2
    inv = rope_inv_freq(hd, theta).to(x.device)
    ang = (positions.to(x.device, torch.float32)[:, None] * inv[None, :]).to(F64)   # float32 product, as the reference
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1)


def attention_scores_mask(seq_len, window=None):
    """Causal: key j is visible to query i iff j <= i (/root/reference/src/models/self_attn.cpp:75-100,
    CUDA key_limit /root/reference/src/cuda/ops/self_attn_detail.cuh:695-751).  With a window W
    (not in the reference) also j > i - W."""
    i = torch.arange(seq_len)[:, None]
    j = torch.arange(seq_len)[None, :]
    ok = j <= i
    if window:
        ok = ok & (j > i - window)
    return ok


def attention(q, k, v, n_heads, n_kv_heads, window=None):
    """q [S, nq, hd], k, v [S, nkv, hd].  Query head h reads kv head h // (nq/nkv)
    (/root/reference/src/cuda/ops/self_attn_detail.cuh:669); score = q.k / sqrt(hd); masked to -inf;
    softmax over keys; out = sum p v (/root/reference/src/models/self_attn.cpp:247-255)."""
    s, _, hd = q.shape
    group = n_heads // n_kv_heads
    ok = attention_scores_mask(s, window).to(q.device)
    out = torch.empty_like(q)
    for h in range(n_heads):
        kh = h // group
        scores = (q[:, h, :] @ k[:, kh, :].T) / math.sqrt(hd)
        scores = scores.masked_fill(~ok, float("-inf"))
        p = torch.softmax(scores, dim=-1)
        out[:, h, :] = p @ v[:, kh, :]
    return out


def self_attention_block(x, w, prefix, cfg, positions, window=None):
    """q,k,v projections with bias, split into heads (feature h*hd + d is head h,
    /root/reference/src/tensor.cpp:101-114), RoPE on q and k, attention, merge heads, o_proj
    (/root/reference/src/models/self_attn.cpp:225-259)."""
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = cfg.get("head_dim") or cfg["hidden_size"] // nq
    s = x.shape[0]
    q = linear(x, w[prefix + "q_proj.weight"], w.get(prefix + "q_proj.bias")).reshape(s, nq, hd)
    k = linear(x, w[prefix + "k_proj.weight"], w.get(prefix + "k_proj.bias")).reshape(s, nkv, hd)
    v = linear(x, w[prefix + "v_proj.weight"], w.get(prefix + "v_proj.bias")).reshape(s, nkv, hd)
    q = rope(q, positions, cfg["rope_theta"])
    k = rope(k, positions, cfg["rope_theta"])
    o = attention(q, k, v, nq, nkv, window).reshape(s, nq * hd)
    return linear(o, w[prefix + "o_proj.weight"])


def swiglu_mlp(x, w, prefix):
    """down( up(x) * silu(gate(x)) ), silu(g) = g / (1 + exp(-g))
    (/root/reference/src/models/mlp.cpp:41-49, /root/reference/src/cuda/ops/mlp.cu:158-161)."""
    u = linear(x, w[prefix + "up_proj.weight"])
    g = linear(x, w[prefix + "gate_proj.weight"])
    return linear(u * (g / (1.0 + torch.exp(-g))), w[prefix + "down_proj.weight"])


def layer_window(cfg, layer):
    if cfg.get("use_sliding_window") and layer >= cfg.get("max_window_layers", cfg["num_hidden_layers"]):
        return cfg["sliding_window"]
    return None


def forward_logits(cfg, w, token_ids, first_position=0, rows=None):
    """Logits [S, V] of one whole sequence: embedding gather, L pre-norm blocks
    (a = x + Attn(N1 x); y = a + MLP(N2 a), /root/reference/src/models/block.cpp:23-29), final norm,
    output projection with the embedding table when tied
    (/root/reference/src/models/gpt_model.cpp:310-333, /root/reference/src/models/embedding.cpp:54-81).
    `first_position` shifts all positions (for the invariance test only).  `rows`: only the logits at these
    places, [len(rows), V] (the reference computes all of them and reads one)."""
    table = w["model.embed_tokens.weight"]
    ids = torch.as_tensor(token_ids, dtype=torch.long, device=table.device)
    eps = cfg.get("rms_norm_eps", 1e-6)
    x = table[ids]
    positions = torch.arange(len(ids)) + first_position
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        xn = rms_norm(x, w[p + "input_layernorm.weight"], eps)
        x = x + self_attention_block(xn, w, p + "self_attn.", cfg, positions, layer_window(cfg, i))
        xn = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu_mlp(xn, w, p + "mlp.")
    if rows is not None:
        x = x[torch.as_tensor(list(rows), dtype=torch.long, device=x.device)]
    xn = rms_norm(x, w["model.norm.weight"], eps)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return linear(xn, head)


# ----------------------------------------------------------------------------- sampling
def greedy(logits):
    """First maximum wins (/root/reference/src/sampler.cpp:13-20)."""
    return int(torch.argmax(logits.to(F64)))


def sampling_distribution(logits, temperature, top_k=0, top_p=1.0):
    """The distribution the reference's sampler draws from (/root/reference/src/sampler.cpp:39-105):
    probabilities p = softmax(logits); p^(1/T); keep the k largest if 0 < k < V; then the smallest
    prefix (by descending p) whose normalised mass reaches top_p; renormalise."""
    p = torch.softmax(logits.to(F64), dim=-1)
    if abs(temperature - 1.0) > 1e-6:
        p = p.clamp_min(0) ** (1.0 / max(temperature, 1e-6))
    order = torch.argsort(p, descending=True, stable=True)
    ps = p[order]
    keep = len(ps)
    if 0 < top_k < keep:
        keep = top_k
    ps = ps[:keep]
    if 0.0 < top_p < 1.0:
        cum = torch.cumsum(ps / ps.sum(), dim=0)
        cutoff = int((cum >= top_p).nonzero()[0]) + 1 if bool((cum >= top_p).any()) else keep
        ps = ps[: max(1, cutoff)]
    out = torch.zeros_like(p)
    out[order[: len(ps)]] = ps / ps.sum()
    return out


def greedy_generate(cfg, w, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(greedy(forward_logits(cfg, w, ids)[-1]))
    return ids[len(prompt):]
