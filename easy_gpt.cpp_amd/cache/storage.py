"""Device memory behind the cache manager: the paged tensors of every group and per-request state records."""
from __future__ import annotations

import torch

from ..parts.base import StateNeed


class PagedStorage:
    """The paged tensors of every cache group: for each group and each tensor its mixers declared
    (`CacheNeed.tensors`), one allocation [slabs, num_pages, *page_shape], a slab per cache id of the group.

    Attention declares keys [n_kv_heads, page_size, head_dim] and values [n_kv_heads, head_dim, page_size] per
    page.  One head's part of a page is contiguous in both.  A key's features are contiguous (the
    score product sums over features); a feature's values over the page's tokens are
    contiguous (the output product sums over tokens): each is the order in which the matrix
    cores take their operands, so the attention kernels load them as they lie.  Pages are
    never cleared: a kernel reads only positions below a request's length."""

    def __init__(self, groups, slabs_per_group, num_pages, page_size: int, dtype: torch.dtype, device):
        self.page_size = page_size
        self.tensors: list[dict[str, torch.Tensor]] = []
        for need, n_slabs, pages in zip(groups, slabs_per_group, num_pages):
            names = [t.name for t in need.tensors]
            if len(set(names)) != len(names):
                raise ValueError(f"a cache need names a tensor twice: {names}")
            self.tensors.append({
                t.name: torch.zeros((n_slabs, pages, *t.page_shape(page_size)),
                                    dtype=torch.float32 if t.dtype == "float32" else dtype, device=device)
                for t in need.tensors
            })

    def slab(self, group: int, index: int) -> dict[str, torch.Tensor]:
        return {name: t[index] for name, t in self.tensors[group].items()}

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for g in self.tensors for t in g.values())


class StateStorage:
    """One record per request slot for every state id a model declares, and one more that belongs to no
    request (`pad_slot`): rows that pad a step to its graph's size read and write that one."""

    def __init__(self, needs: dict[int, StateNeed], max_requests: int, device):
        self.pad_slot = max_requests
        self.data = {
            sid: torch.zeros((max_requests + 1, *need.shape), dtype=need.dtype, device=device)
            for sid, need in needs.items()
        }

    def reset(self, slot: int) -> None:
        for t in self.data.values():
            t[slot].zero_()
