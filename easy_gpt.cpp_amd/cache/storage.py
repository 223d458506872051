"""Device memory behind the cache manager: key/value slabs per group and per-request state records."""
from __future__ import annotations

import torch

from ..parts.base import StateNeed


class KVStorage:
    """For each group, keys as [slabs, num_pages, n_kv_heads, page_size, head_dim] and values
    transposed within a page, [slabs, num_pages, n_kv_heads, head_dim, page_size].

    One head's part of a page is contiguous in both.  A key's features are contiguous (the
    score product sums over features); a feature's values over the page's tokens are
    contiguous (the output product sums over tokens): each is the order in which the matrix
    cores take their operands, so the attention kernels load them as they lie.  Pages are
    never cleared: a kernel reads only positions below a request's length."""

    def __init__(self, groups, slabs_per_group, num_pages, page_size: int, dtype: torch.dtype, device):
        self.page_size = page_size
        self.k: list[torch.Tensor] = []
        self.v: list[torch.Tensor] = []
        for need, n_slabs, pages in zip(groups, slabs_per_group, num_pages):
            k_shape = (n_slabs, pages, need.n_kv_heads, page_size, need.head_dim)
            v_shape = (n_slabs, pages, need.n_kv_heads, need.head_dim, page_size)
            self.k.append(torch.zeros(k_shape, dtype=dtype, device=device))
            self.v.append(torch.zeros(v_shape, dtype=dtype, device=device))

    def slab(self, group: int, index: int):
        return self.k[group][index], self.v[group][index]

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.k + self.v)


class StateStorage:
    """One record per request slot for every state id a model declares."""

    def __init__(self, needs: dict[int, StateNeed], max_requests: int, device):
        self.data = {
            sid: torch.zeros((max_requests, *need.shape), dtype=need.dtype, device=device)
            for sid, need in needs.items()
        }

    def reset(self, slot: int) -> None:
        for t in self.data.values():
            t[slot].zero_()
