"""Token embedding and the output projection.

Embedding: x[t, :] = E[id_t, :] (/root/reference/src/models/embedding.cpp:54-76; an
id outside [0, V) is an error there and here).  Output: logits = xn E^T with the
embedding table when tied (/root/reference/src/models/embedding.cpp:78-81,
src/models/gpt_model.cpp:328); the reference always ties; here `tied=False`
uses a separate `lm_head.weight` [V, H].  Logits come out in float32.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import Embedding, OutputHead, register_part
from .spec import ParamSpec


class TokenEmbedding(Embedding):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, vocab_size: int):
        self.prefix = prefix
        self.hidden_size = int(hidden_size)
        self.vocab_size = int(vocab_size)
        self.table: torch.Tensor | None = None

    def param_specs(self):
        return [ParamSpec(self.prefix + "weight", (self.vocab_size, self.hidden_size), role="embedding")]

    def load(self, get, dtype, device):
        self.table = self._to(get(self.prefix + "weight"), "compute", dtype, device)

    def output_matrix(self) -> torch.Tensor:
        return self.table

    def forward(self, ctx) -> torch.Tensor:
        k = kernels.backend()
        token_ids = ctx.token_ids
        out = torch.empty((token_ids.shape[0], self.hidden_size), device=token_ids.device,
                          dtype=k.residual_dtype(token_ids.shape[0], self.table.dtype))     # the residual stream
        k.embed(token_ids, self.table, out)
        return out


class LinearHead(OutputHead):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, vocab_size: int, tied: bool):
        self.prefix = prefix
        self.hidden_size = int(hidden_size)
        self.vocab_size = int(vocab_size)
        self.tied = bool(tied)
        self.weight: torch.Tensor | None = None

    def param_specs(self):
        if self.tied:
            return []
        return [ParamSpec(self.prefix + "weight", (self.vocab_size, self.hidden_size))]

    def load(self, get, dtype, device):
        if not self.tied:
            self.weight = self._to(get(self.prefix + "weight"), "compute", dtype, device)

    def tie(self, matrix: torch.Tensor) -> None:
        if tuple(matrix.shape) != (self.vocab_size, self.hidden_size):
            raise ValueError(f"a tied output head needs a [{self.vocab_size}, {self.hidden_size}] matrix, "
                             f"got {tuple(matrix.shape)}")
        self.weight = matrix

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty((x.shape[0], self.vocab_size), dtype=torch.float32, device=x.device)
        kernels.backend().linear(x, self.weight, None, out)
        return out


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("output_head", "linear_head", LinearHead)
