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
from .base import FeedForward, register_part
from .spec import ParamSpec


class SwiGLU(FeedForward):
    graph_safe = True

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
        t = x.shape[0]
        gate_up = k.product(x, self.w_gate_up)           # act [T, 2I] or float32 partial sums [S, T, 2I]
        act = torch.empty((t, self.intermediate_size), dtype=x.dtype, device=x.device)
        k.swiglu(gate_up, act)
        return k.product(act, self.w_down)               # added to the residual stream by the next norm


register_part("feed_forward", "swiglu", SwiGLU)
