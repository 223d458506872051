"""A model assembled from a ModelSpec: embedding, layers in their run order, final norm, output head.

The counterpart of the reference's GptModel::init_from_config / load_param /
forward_logits (/root/reference/src/models/gpt_model.cpp:132-153,310-333), without
its generation loop: this class only maps a step's tokens to logits at the wanted rows.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import kernels

from .base import BLOCKS, CacheNeed, StateNeed, make_part
from .spec import ModelSpec, ParamSpec


@dataclass(frozen=True)
class CacheGroup:
    """Cache slabs with the same needs; they share one page pool and one block table per request."""

    need: CacheNeed
    cache_ids: tuple[int, ...]


class Model:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        ctx = dict(hidden_size=spec.hidden_size)
        self.embedding = make_part("embedding", spec.embedding, vocab_size=spec.vocab_size, **ctx)
        self.layers = []
        for ls in spec.layers:
            if ls.block not in BLOCKS:
                raise KeyError(f"unknown block kind '{ls.block}' (registered: {', '.join(sorted(BLOCKS)) or 'none'})")
            mixer = make_part("mixer", ls.mixer, **ctx) if ls.mixer is not None else None
            ff = make_part("feed_forward", ls.feed_forward, **ctx) if ls.feed_forward is not None else None
            norms = {slot: make_part("norm", ns, **ctx) for slot, ns in ls.norms.items()}
            self.layers.append(BLOCKS[ls.block](mixer, ff, norms))
        self.final_norm = make_part("norm", spec.final_norm, **ctx)
        self.output_head = make_part("output_head", spec.output_head, vocab_size=spec.vocab_size, **ctx)
        self.dtype: torch.dtype | None = None
        self.device: torch.device | None = None
        self._plan_caches()
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in self.parts())

    # ------------------------------------------------------------------ cache and state plan
    def _plan_caches(self) -> None:
        needs: dict[int, CacheNeed] = {}
        writers: set[int] = set()
        self.state_needs: dict[int, StateNeed] = {}
        for i, run in enumerate(self.spec.run_order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"run order entry {i} names layer {run.layer}, the model has {len(self.layers)}")
            mixer = self.layers[run.layer].mixer
            if mixer is None:
                if run.cache is not None or run.state is not None:
                    raise ValueError(f"run order entry {i}: layer {run.layer} has no mixer, so neither cache nor state")
                continue
            need = mixer.cache_need()
            if need is None:
                if run.cache is not None:
                    raise ValueError(f"run order entry {i}: layer {run.layer}'s mixer has no paged cache")
            else:
                if run.cache is None:
                    raise ValueError(f"run order entry {i}: layer {run.layer}'s mixer needs a cache id")
                if run.cache in needs and needs[run.cache] != need:
                    raise ValueError(f"cache {run.cache} is shared by mixers with different needs")
                if run.writes_cache:
                    if run.cache in writers:
                        raise ValueError(f"cache {run.cache} is written by two run-order entries")
                    writers.add(run.cache)
                elif run.cache not in writers:
                    raise ValueError(f"run order entry {i} reads cache {run.cache} before any entry writes it")
                needs[run.cache] = need
            sneed = mixer.state_need()
            if sneed is not None:
                if run.state is None:
                    raise ValueError(f"run order entry {i}: layer {run.layer}'s mixer needs a state id")
                if run.state in self.state_needs:
                    raise ValueError(f"state {run.state} is used by two run-order entries")
                self.state_needs[run.state] = sneed
        by_need: dict[CacheNeed, list[int]] = {}
        for cid in sorted(needs):
            by_need.setdefault(needs[cid], []).append(cid)
        self.cache_groups = [CacheGroup(n, tuple(ids)) for n, ids in by_need.items()]
        self.cache_location: dict[int, tuple[int, int]] = {}
        for g, grp in enumerate(self.cache_groups):
            for j, cid in enumerate(grp.cache_ids):
                self.cache_location[cid] = (g, j)

    # ------------------------------------------------------------------ weights
    def parts(self):
        yield self.embedding
        for block in self.layers:
            yield from block.parts()
        yield self.final_norm
        yield self.output_head

    def param_specs(self) -> list[ParamSpec]:
        specs: list[ParamSpec] = []
        for p in self.parts():
            specs.extend(p.param_specs())
        names = [s.name for s in specs]
        if len(set(names)) != len(names):
            dup = sorted({n for n in names if names.count(n) > 1})
            raise ValueError(f"tensor names declared twice: {dup}")
        return specs

    def load(self, get, dtype: torch.dtype, device) -> None:
        """Take every declared tensor through `get(name)` (a checked weights source)."""
        device = resolve_device(device)
        for p in self.parts():
            p.load(get, dtype, device)
        if getattr(self.output_head, "tied", False):
            matrix = self.embedding.output_matrix()
            if matrix is None:
                raise ValueError(f"the output head is tied, but {type(self.embedding).__name__} has no matrix to share")
            self.output_head.tie(matrix)
        self.dtype, self.device = dtype, device

    # ------------------------------------------------------------------ one step
    def forward(self, ctx) -> torch.Tensor | None:
        """Run the step described by `ctx`; returns float32 logits [rows, V] or None if no row is wanted."""
        ctx.shared.clear()                           # per-step values that layers share are made anew every step
        with kernels.backend().pinned_stream():      # one look-up of the current stream for the whole pass
            return self._forward(ctx)

    def _forward(self, ctx) -> torch.Tensor | None:
        h = self.embedding.forward(ctx)
        delta = None
        for run in self.spec.run_order:
            block = self.layers[run.layer]
            cache = ctx.cache_view(run.cache, run.writes_cache) if run.cache is not None else None
            state = ctx.state_view(run.state) if run.state is not None else None
            h, delta = block.forward(h, delta, ctx, cache, state)
        if ctx.want_rows is None or ctx.want_rows.shape[0] == 0:
            return None
        x = self.final_norm.forward_rows(h, delta, ctx.want_rows)
        return self.output_head.forward(x)


def resolve_device(device) -> torch.device:
    """`device` as a torch.device with its index spelled out: "cuda" names the current GPU, and tensors made there
    report "cuda:<index>", which does not compare equal to the unindexed name."""
    device = torch.device(device)
    if device.type == "cuda" and device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    return device


def build_model(spec: ModelSpec) -> Model:
    return Model(spec)
