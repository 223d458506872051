"""RMSNorm, fused with the addition into the residual stream.

Formula as the reference computes it (/root/reference/src/models/norm.cpp:30-62,
CUDA form /root/reference/src/cuda/ops/self_attn_detail.cuh:385-418):
ss = sum_j x_j^2 in float32, inv = 1 / sqrt(ss / H + eps), y_j = x_j * inv * w_j.
The reference fixes eps = 1e-6 in code (norm.cpp:41); here it is a parameter.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import Norm, register_part
from .spec import ParamSpec


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, eps: float):
        self.prefix = prefix
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self.weight: torch.Tensor | None = None

    def param_specs(self):
        h = self.hidden_size
        return [ParamSpec(self.prefix + "weight", (h,), role="norm_scale", alt_shapes=((h, 1),))]

    def load(self, get, dtype, device):
        self.weight = self._to(get(self.prefix + "weight").reshape(self.hidden_size), "compute", dtype, device)

    def rms_params(self):
        return self.weight, self.eps

    def forward(self, h, delta):
        out = torch.empty(h.shape, dtype=self.weight.dtype, device=h.device)
        kernels.backend().add_rmsnorm(h, delta, self.weight, self.eps, out)
        return out

    def forward_rows(self, h, delta, rows):
        out = torch.empty((rows.shape[0], h.shape[1]), dtype=self.weight.dtype, device=h.device)
        kernels.backend().rows_add_rmsnorm(h, delta, rows, self.weight, self.eps, out)
        return out


register_part("norm", "rmsnorm", RMSNorm)
