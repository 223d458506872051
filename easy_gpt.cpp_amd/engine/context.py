"""What one step hands to the model: the flattened tokens of all requests and where their cache lies."""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..parts.base import CacheView, StateView


@dataclass
class GroupTables:
    block_table: torch.Tensor   # int32 [B, W], -1 where there is no page
    slots: torch.Tensor         # int32 [T], page * page_size + offset of each token of the step


@dataclass
class StepContext:
    """T tokens of B requests, request after request.

    token_ids, positions   int32 [T]; a token's position is the number of tokens before it in its request
    q_start, q_len         int32 [B]: where each request's tokens start in the flat arrays, and how many
    kv_len                 int32 [B]: tokens of the request in the cache once this step's are stored
    want_rows              int32 [R]: flat indices of the tokens whose logits are wanted, or None
    *_host                 the same numbers as Python lists, for parts that plan on the host
    rows_independent       False when several of the B "requests" are tokens of one request (a portion laid out as
                           single-token rows that share a block table): a row's keys and values must then be in the
                           cache before any row's attention reads it
    single_token_requests  False when no request of the step brings exactly one token: a kernel that takes those apart
                           from the portions of prompts need not run
    """

    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor
    positions: torch.Tensor
    q_start: torch.Tensor
    q_len: torch.Tensor
    kv_len: torch.Tensor
    want_rows: torch.Tensor | None
    max_q_len: int
    max_kv_len: int
    q_start_host: list[int]
    q_len_host: list[int]
    kv_len_host: list[int]
    state_slots: torch.Tensor
    state_slots_host: list[int]
    groups: list[GroupTables] = field(default_factory=list)
    page_size: int = 0
    kv_storage: object = None
    state_storage: object = None
    cache_location: dict = field(default_factory=dict)
    group_windows: list = field(default_factory=list)
    shared: dict = field(default_factory=dict)     # what parts of several layers compute once per step and share
    rows_independent: bool = True
    single_token_requests: bool = True     # False when the step is known to hold no request of exactly one token

    def cache_view(self, cache_id: int, writes: bool) -> CacheView:
        g, j = self.cache_location[cache_id]
        t = self.groups[g]
        return CacheView(self.kv_storage.slab(g, j), self.page_size, t.block_table, t.slots, self.group_windows[g], writes)

    def state_view(self, state_id: int) -> StateView:
        fresh = [kv == q for kv, q in zip(self.kv_len_host, self.q_len_host)]
        if "fresh_device" not in self.shared:            # a request is new when this step's tokens are all it holds
            self.shared["fresh_device"] = self.kv_len == self.q_len
        return StateView(self.state_storage.data[state_id], self.state_slots, self.state_slots_host, fresh,
                         self.shared["fresh_device"])
