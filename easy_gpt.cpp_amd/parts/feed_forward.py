"""Dense gated feed-forward (SwiGLU).

As the reference computes it (/root/reference/src/models/mlp.cpp:41-49, CUDA form
/root/reference/src/cuda/ops/mlp.cu:152-162): u = x Wup^T, g = x Wgate^T,
y = (u * g / (1 + exp(-g))) Wdown^T; the gate is the activated branch; no biases.
The reference infers the inner width from the tensors
(/root/reference/src/models/model_param_validation.cpp:167-194); here it is a parameter.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import FeedForward, PendingNorm, register_part
from .spec import ParamSpec


class SwiGLU(FeedForward):
    graph_safe = True
    takes_pending_norm = True

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        if activation != "silu":
            raise ValueError(f"activation '{activation}' is not supported by the swiglu feed-forward")
        self.prefix = prefix
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.w_gate_up = self.w_down = None

    def param_specs(self):
        p, h, i = self.prefix, self.hidden_size, self.intermediate_size
        return [
            ParamSpec(p + "gate_proj.weight", (i, h)),
            ParamSpec(p + "up_proj.weight", (i, h)),
            ParamSpec(p + "down_proj.weight", (h, i)),
        ]

    def load(self, get, dtype, device):
        p = self.prefix
        w = torch.cat([get(p + "gate_proj.weight").to(dtype), get(p + "up_proj.weight").to(dtype)], dim=0)
        self.w_gate_up = w.to(device).contiguous()
        self.w_down = self._to(get(p + "down_proj.weight"), "compute", dtype, device)

    def forward(self, x, ctx=None):
        k = kernels.backend()
        # With few tokens: the norm folds into the first product's staging of x, and SwiGLU (with the rows'
        # 1/rms factor) into the second's.
        residual = None

        def down(act):
            out = k.product(act, self.w_down, residual=residual)     # else added to the residual stream by the next norm
            return None if out is residual else out

        if isinstance(x, PendingNorm):
            pending = x
            rms = x.rms()
            fused = None
            if rms is not None and self.intermediate_size % 8 == 0:
                fused = k.product_normed(x.h, x.delta, rms[0], self.w_gate_up)
            if fused is not None:
                gate_up, row_ss, h_new = fused
                x.applied(h_new)
                residual = pending.residual()
                out = k.product_swiglu(gate_up, row_ss, self.hidden_size, rms[1], self.w_down, residual=residual)
                if out is not None:
                    return None if out is residual else out
                # SwiGLU by itself; it applies the rows' pending 1/rms factor
                act = torch.empty((h_new.shape[0], self.intermediate_size), dtype=self.w_down.dtype, device=h_new.device)
                k.swiglu(gate_up, act, row_ss=row_ss, hidden=self.hidden_size, eps=rms[1])
                return down(act)
            x = x.materialize()
            residual = pending.residual()
        t = x.shape[0]
        act = k.gate_up_swiglu(x, self.w_gate_up)        # a few dozen tokens: product and activation in one kernel
        if act is not None:
            return down(act)
        gate_up = k.product(x, self.w_gate_up)           # act [T, 2I] or float32 partial sums [S, T, 2I]
        if gate_up.dim() == 3:
            out = k.product_swiglu(gate_up, None, self.hidden_size, 0.0, self.w_down, residual=residual)
            if out is not None:
                return None if out is residual else out
        act = torch.empty((t, self.intermediate_size), dtype=x.dtype, device=x.device)
        k.swiglu(gate_up, act)
        return down(act)


register_part("feed_forward", "swiglu", SwiGLU)
