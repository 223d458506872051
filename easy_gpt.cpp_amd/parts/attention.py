"""Grouped-query softmax attention over the paged cache.

As the reference computes it (/root/reference/src/models/self_attn.cpp:217-260 and
the CUDA path /root/reference/src/cuda/ops/self_attn.cu:299-369,689-980):
q = x Wq^T + bq, k = x Wk^T + bk, v = x Wv^T + bv; features h*hd + d belong to head h
(/root/reference/src/tensor.cpp:101-114); queries and keys are rotated; keys and
values of the new tokens join the cache before attention so a prompt portion
attends to itself causally; query head h reads key/value head h // (nq/nkv)
(/root/reference/src/cuda/ops/self_attn_detail.cuh:669); score = q.k / sqrt(hd),
softmax in float32, output = sum_j p_j v_j; heads are concatenated and projected
by Wo (no bias in Qwen2, bias used if the tensor exists: src/models/linear.cpp:30-39).
"""
from __future__ import annotations

import math

import torch

from .. import kernels
from .base import CacheNeed, Mixer, PendingNorm, make_part, register_part
from .spec import ParamSpec, PartSpec


class GQAttention(Mixer):
    graph_safe = True
    takes_pending_norm = True

    def __init__(
        self,
        prefix: str,
        hidden_size: int,
        n_heads: int,
        n_kv_heads: int,
        head_dim: int,
        qkv_bias: bool,
        out_bias: bool,
        position: PartSpec,
        window: int | None = None,
        scale: float | None = None,
    ):
        if n_heads % n_kv_heads:
            raise ValueError(f"n_heads ({n_heads}) must be a multiple of n_kv_heads ({n_kv_heads})")
        if not 0 < int(head_dim) <= kernels.KernelBackend.max_head_dim:
            raise ValueError(f"head size {head_dim} is not supported by the attention kernels "
                             f"(1 to {kernels.KernelBackend.max_head_dim})")
        self.prefix = prefix
        self.hidden_size = int(hidden_size)
        self.n_heads = int(n_heads)
        self.n_kv_heads = int(n_kv_heads)
        self.head_dim = int(head_dim)
        self.qkv_bias = bool(qkv_bias)
        self.out_bias = bool(out_bias)
        self.window = int(window) if window else None
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.position = make_part("position_encoding", position, head_dim=self.head_dim)
        self.graph_safe = bool(getattr(self.position, "graph_safe", False))
        self.q_size = self.n_heads * self.head_dim
        self.kv_size = self.n_kv_heads * self.head_dim
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None

    # ------------------------------------------------------------------ declaration
    def cache_need(self):
        return CacheNeed.keys_and_values(self.n_kv_heads, self.head_dim, self.window)

    def param_specs(self):
        p, h = self.prefix, self.hidden_size
        specs = [
            ParamSpec(p + "q_proj.weight", (self.q_size, h)),
            ParamSpec(p + "k_proj.weight", (self.kv_size, h)),
            ParamSpec(p + "v_proj.weight", (self.kv_size, h)),
            ParamSpec(p + "o_proj.weight", (h, self.q_size)),
        ]
        if self.qkv_bias:
            specs += [
                ParamSpec(p + "q_proj.bias", (self.q_size,), role="bias"),
                ParamSpec(p + "k_proj.bias", (self.kv_size,), role="bias"),
                ParamSpec(p + "v_proj.bias", (self.kv_size,), role="bias"),
            ]
        if self.out_bias:
            specs.append(ParamSpec(p + "o_proj.bias", (h,), role="bias"))
        return specs + self.position.param_specs()

    def load(self, get, dtype, device):
        p = self.prefix
        # q, k and v stay separate tensors in the file; on the device their rows are one
        # matrix so that one product serves all three.
        w = torch.cat([get(p + n + "_proj.weight").to(dtype) for n in "qkv"], dim=0)
        self.w_qkv = w.to(device).contiguous()
        if self.qkv_bias:
            b = torch.cat([get(p + n + "_proj.bias").to(dtype) for n in "qkv"], dim=0)
            self.b_qkv = b.to(device).contiguous()
        self.w_o = self._to(get(p + "o_proj.weight"), "compute", dtype, device)
        if self.out_bias:
            self.b_o = self._to(get(p + "o_proj.bias"), "compute", dtype, device)
        self.position.load(get, dtype, device)

    # ------------------------------------------------------------------ computation
    def forward(self, x, ctx, cache, state=None):
        k = kernels.backend()
        width = self.q_size + 2 * self.kv_size
        rot = self.position.rotary(x.h.device if isinstance(x, PendingNorm) else x.device)
        # ---- q, k, v.  With few tokens the residual addition and the norm before this layer fold into the
        # product's staging of x; the rows' 1/rms factor is applied by the epilogue kernel below.
        scale_args = {}
        prod = None
        pending = x if isinstance(x, PendingNorm) else None
        if isinstance(x, PendingNorm):
            fused = None
            rms = x.rms()
            if rms is not None and rot is not None:
                fused = k.product_normed(x.h, x.delta, rms[0], self.w_qkv)
            if fused is not None:
                prod, row_ss, h_new = fused
                x.applied(h_new)
                scale_args = dict(row_ss=row_ss, hidden=self.hidden_size, eps=rms[1])
                dtype, device, t = self.w_qkv.dtype, h_new.device, h_new.shape[0]
            else:
                x = x.materialize()
        if prod is None:
            prod = k.product(x, self.w_qkv, unrounded=True)      # act [T, W], or float32 partial sums [S, T, W]
            dtype, device, t = x.dtype, x.device, x.shape[0]
        slots = cache.slots if cache.writes else None
        common = dict(
            k_cache=cache.k, v_cache=cache.v, nq=self.n_heads, nkv=self.n_kv_heads,
            hd=self.head_dim, page_size=cache.page_size,
        )
        attn = torch.empty((t, self.q_size), dtype=dtype, device=device)
        want_parts = self.b_o is None and t <= k.fused_rows
        # ---- single decoded tokens: bias, rotation, the store of the new key and value and the attention over
        # the cache in one kernel, straight from the product's partial sums
        parts = False
        cos_sin = self.position.table(ctx) if rot is not None else None
        if (prod.dim() == 3 and rot is not None and slots is not None and ctx.max_q_len == 1
                and ctx.rows_independent):
            parts = k.attention_decode_fused(
                prod, scale_args.get("row_ss"), scale_args.get("hidden", 0), scale_args.get("eps", 0.0), self.b_qkv,
                ctx.positions, rot[0], rot[1], slots, attn, cache.k, cache.v, cache.block_table, ctx.q_start, ctx.kv_len,
                self.n_heads, self.n_kv_heads, self.head_dim, cache.page_size, self.scale, self.window or 0,
                ctx.max_kv_len, combine=not want_parts, cos_sin=cos_sin)
        if parts is False:
            if cos_sin is not None:
                scale_args = dict(scale_args, cos_sin=cos_sin)
            parts = self._epilogue_and_attention(k, prod, t, width, dtype, device, rot, slots, common, scale_args, ctx,
                                                 cache, attn, want_parts)
        # the output projection: into the residual stream itself where that takes additions (then nothing is returned)
        residual = pending.residual() if pending is not None else None
        if parts is not None:
            out = k.product_attention(parts[0], parts[1], self.w_o, residual=residual)
            if out is not None:
                return None if out is residual else out
            k.combine_attention(parts[0], parts[1], attn)
        if self.b_o is None:
            out = k.product(attn, self.w_o, residual=residual)   # else the residual add that follows sums partial sums up
            return None if out is residual else out
        out = torch.empty((t, self.hidden_size), dtype=dtype, device=device)
        k.linear(attn, self.w_o, self.b_o, out)
        return out

    def _epilogue_and_attention(self, k, prod, t, width, dtype, device, rot, slots, common, scale_args, ctx, cache, attn,
                                want_parts):
        """Bias, position encoding and the store into the cache, then attention over the cache; returns what
        paged_attention returns (the parts of a split key range, or None when `attn` is written)."""
        qkv = prod if prod.dim() == 2 else torch.empty((t, width), dtype=dtype, device=device)
        if rot is not None:
            inv_freq, rotary_dim = rot
            k.qkv_rope_store(prod, self.b_qkv, ctx.positions, inv_freq, rotary_dim, slots, out=qkv, **common, **scale_args)
        else:
            # bias, then the position encoding's own transform, then the store
            if self.b_qkv is not None or prod.dim() == 3:
                k.qkv_rope_store(prod, self.b_qkv, ctx.positions, None, 0, None, out=qkv, **common)
            q_view = qkv[:, : self.q_size].view(t, self.n_heads, self.head_dim)
            k_view = qkv[:, self.q_size : self.q_size + self.kv_size].view(t, self.n_kv_heads, self.head_dim)
            self.position.apply(q_view, k_view, ctx.positions)
            if slots is not None:
                k.qkv_rope_store(qkv, None, ctx.positions, None, 0, slots, out=qkv, **common)
        # ---- attention over the cache.  If the kernel splits the keys, the output projection combines the parts.
        args = dict(
            nq=self.n_heads, nkv=self.n_kv_heads, hd=self.head_dim, page_size=cache.page_size,
            scale=self.scale, window=self.window or 0, max_q_len=ctx.max_q_len, max_kv_len=ctx.max_kv_len,
            singles=getattr(ctx, "single_token_requests", True),
        )
        if want_parts:
            args["combine"] = False
        return k.paged_attention(qkv, attn, cache.k, cache.v, cache.block_table, ctx.q_start, ctx.q_len, ctx.kv_len,
                                 **args)


register_part("mixer", "gq_attention", GQAttention)
