"""Interfaces of the parts a layer is made of, and the registries that name them.

A part gets its sizes and constants as constructor parameters, declares the
tensors it needs (`param_specs`), takes them (`load`) and computes (`forward`)
through the kernel backend.  It never learns which model it belongs to.

Shapes in the docstrings: T tokens of the step (all requests flattened), B
requests of the step, H the model width.  "act" is the engine's activation
dtype (bfloat16 or float32); the residual stream `h` is always float32.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable

import torch

from .spec import ParamSpec, PartSpec


# --------------------------------------------------------------------------- needs
@dataclass(frozen=True)
class PagedTensor:
    """One tensor of a paged cache: per token a block of `dims` numbers.  A page holds `page_size` tokens; its
    block has the shape of `dims` with the token's offset in the page put in as axis `token_axis`.
    dtype 'compute' is the engine's activation dtype, 'float32' stays."""

    name: str
    dims: tuple[int, ...]
    token_axis: int = 0
    dtype: str = "compute"

    def page_shape(self, page_size: int) -> tuple[int, ...]:
        if not 0 <= self.token_axis <= len(self.dims):
            raise ValueError(f"paged tensor '{self.name}': token_axis {self.token_axis} is outside its {len(self.dims)} dims")
        return (*self.dims[: self.token_axis], page_size, *self.dims[self.token_axis :])


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer asks of the paged cache: which tensors it keeps per token, and for how long.

    window None: every earlier token stays readable.  window W: a token reads only
    the last W tokens (itself included); pages wholly behind that are given back.
    Mixers with equal needs share a page pool and a block table per request.
    """

    tensors: tuple[PagedTensor, ...]
    window: int | None = None

    @classmethod
    def keys_and_values(cls, n_kv_heads: int, head_dim: int, window: int | None = None) -> "CacheNeed":
        """Attention's cache: keys [n_kv_heads, page_size, head_dim] per page (a key's features contiguous) and
        values [n_kv_heads, head_dim, page_size] (a feature's values over the page's tokens contiguous): each the
        order in which the matrix cores take their operands."""
        return cls((PagedTensor("k", (n_kv_heads, head_dim), 1), PagedTensor("v", (n_kv_heads, head_dim), 2)), window)


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size: one record of `shape` and `dtype` per live request."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


# --------------------------------------------------------------------------- views handed to a mixer
@dataclass
class CacheView:
    """One cache slab as a mixer sees it during a step.

    tensors      by the names of the mixer's `CacheNeed`: each [num_pages, *page_shape]; for attention
                 k [num_pages, n_kv_heads, page_size, head_dim] and v [num_pages, n_kv_heads, head_dim, page_size]
    block_table  int32 [B, W]: page ids of each request in order (-1 where a page was given back)
    slots        int32 [T]: page * page_size + offset where each token of the step is stored
    """

    tensors: dict[str, torch.Tensor]
    page_size: int
    block_table: torch.Tensor
    slots: torch.Tensor
    window: int | None
    writes: bool = True

    @property
    def k(self) -> torch.Tensor:
        return self.tensors["k"]

    @property
    def v(self) -> torch.Tensor:
        return self.tensors["v"]


@dataclass
class StateView:
    """Per-request state records: `data[slot]` belongs to the request that holds `slot`.

    data       [max_requests + 1, *shape]; the last record belongs to no request (rows that pad a step use it)
    slots      int32 [B] slot of each request of the step (device); slots_host the same on the host
    fresh      list[bool]: True where the request has no tokens before this step (state must start anew)
    fresh_device   the same as a bool tensor [B] on the device.  A mixer whose `forward` reads `slots` and
               `fresh_device` and neither host list is `graph_safe`: its decode steps replay from a graph, in
               which the host lists are those of the step that was captured.
    """

    data: torch.Tensor
    slots: torch.Tensor
    slots_host: list[int]
    fresh: list[bool]
    fresh_device: torch.Tensor | None = None


# --------------------------------------------------------------------------- part interfaces
class Part:
    """Common interface: parameters declared, loaded, then used.

    graph_safe: True if `forward` only launches device work whose arguments do not depend on host
    values other than the step's shapes (no reads of device data on the host, no host loops over
    requests).  Steps of models whose parts are all graph-safe can be captured into a device graph
    and replayed."""

    graph_safe = False

    def param_specs(self) -> list[ParamSpec]:
        return []

    def load(self, get: Callable[[str], torch.Tensor], dtype: torch.dtype, device: torch.device) -> None:
        """Take the tensors declared by `param_specs`; `get(name)` returns the stored (CPU) tensor."""

    @staticmethod
    def _to(t: torch.Tensor, spec_dtype: str, dtype: torch.dtype, device) -> torch.Tensor:
        if spec_dtype == "compute":
            t = t.to(dtype)
        return t.to(device).contiguous()


class Norm(Part):
    """forward(h, delta): h += delta (in place, skipped when delta is None; delta is act [T, H] or float32 partial
    sums [S, T, H]); returns norm(h) as act [T, H].  forward_rows does the same for selected rows without
    writing h back (used for the rows whose logits are wanted).  The stream h is float32 or 64-bit fixed point:
    a norm hands it to the backend (`add_rmsnorm`; or `residual_add` and `residual_values` for a norm that the
    backend has no kernel for) and never reads it by itself."""

    def rms_params(self) -> tuple[torch.Tensor, float] | None:
        """(weight, eps) if this norm is y = x / sqrt(mean(x^2) + eps) * weight, so that a part may fold it into its
        own first kernel; None for any other norm."""
        return None

    def forward(self, h: torch.Tensor, delta: torch.Tensor | None) -> torch.Tensor:
        raise NotImplementedError

    def forward_rows(self, h: torch.Tensor, delta: torch.Tensor | None, rows: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class PendingNorm:
    """x = norm(h + delta), not computed yet.

    A block hands this to a mixer or feed-forward that sets `takes_pending_norm`: such a part may fold the
    addition and the norm into its own first kernel (`rms()` gives it the norm's weight and eps when the
    norm is an RMSNorm) and must then call `applied(h_new)` with the updated residual stream; or it calls
    `materialize()` to get x as a tensor, as any other part would have been given.
    """

    def __init__(self, h: torch.Tensor, delta: torch.Tensor | None, norm: "Norm"):
        self.h, self.delta, self.norm = h, delta, norm
        self.h_after: torch.Tensor | None = None

    def rms(self):
        """(weight, eps) if the norm is y = x / rms(x) * weight, else None."""
        return self.norm.rms_params()

    def applied(self, h_new: torch.Tensor) -> None:
        self.h_after = h_new

    def residual(self) -> torch.Tensor | None:
        """The residual stream after the addition (known once `applied` or `materialize` was called), if it is of
        the kind that a part may add its own output into (64-bit fixed point, `kernels.residual_dtype`): the part
        passes it to the backend's product as `residual=` and returns None if the product went there."""
        h = self.h_after
        return h if h is not None and h.dtype == torch.int64 else None

    def materialize(self) -> torch.Tensor:
        x = self.norm.forward(self.h, self.delta)      # adds delta into h in place
        self.h_after = self.h
        return x


class PositionEncoding(Part):
    """How token positions enter a mixer.

    Either `rotary()` returns (inv_freq float32 [rotary_dim/2], rotary_dim) and the
    mixer's fused kernel rotates queries and keys itself, or it returns None and
    `apply(q, k, positions)` changes the [T, heads, head_dim] views in place.
    """

    def rotary(self, device) -> tuple[torch.Tensor, int] | None:
        return None

    def table(self, ctx) -> torch.Tensor | None:
        """For a rotary encoding: the step's cosines and sines float32 [T, rotary_dim / 2, 2], made once per step
        and shared by the layers (`ctx.shared`); None if there is no such table."""
        return None

    def apply(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor) -> None:
        raise NotImplementedError


class Mixer(Part):
    """Mixes information between the tokens of a request.

    forward(x, ctx, cache, state) -> act [T, H]; x is the normed input act [T, H];
    ctx is the engine's StepContext; cache a CacheView if `cache_need()` is not None;
    state a StateView if `state_need()` is not None.  A part that was given a PendingNorm may add its output
    into that norm's residual stream itself (`PendingNorm.residual()`) and then returns None.
    """

    takes_pending_norm = False     # True: forward may be given a PendingNorm instead of x

    def cache_need(self) -> CacheNeed | None:
        return None

    def state_need(self) -> StateNeed | None:
        return None

    def forward(self, x: torch.Tensor, ctx: Any, cache: CacheView | None, state: StateView | None) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """forward(x) -> act [T, H] for x act [T, H]; tokens are independent.  As a mixer, it may add its output into a
    PendingNorm's residual stream itself and return None."""

    takes_pending_norm = False

    def forward(self, x: torch.Tensor, ctx: Any) -> torch.Tensor:
        raise NotImplementedError


class Embedding(Part):
    """Turns a step's tokens into the residual stream.

    forward(ctx) -> [T, H] residual stream (of the type `kernels.residual_dtype` names for this many tokens).  It is
    handed the whole step context, so an embedding may use more than `ctx.token_ids` (int32 [T]): a learned vector
    per position would look up `ctx.positions`.  `output_matrix()` is the [V, H] matrix that an output head may tie
    itself to, or None if this embedding has none to share."""

    def output_matrix(self) -> torch.Tensor | None:
        return None

    def forward(self, ctx: Any) -> torch.Tensor:
        raise NotImplementedError


class OutputHead(Part):
    """forward(x) -> float32 logits [R, V] for the normed rows x act [R, H].  `tied` True: the head declares no
    matrix of its own and is given the embedding's (`tie`) after the weights are loaded."""

    tied = False

    def tie(self, matrix: torch.Tensor) -> None:
        raise NotImplementedError

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block:
    """Arrangement of one layer's parts around the residual stream.

    forward(h, delta, ctx, cache, state) -> (h', delta'): `h` [T, H] is the residual stream (float32, or
    64-bit fixed point in steps of few tokens: parts never look into it, they hand it to the backend) and
    `delta` the not-yet-added output of the previous layer (None for the first, or when that layer added it itself;
    act [T, H], or float32 partial sums [splits, T, H] of a split product: a norm's kernel adds either);
    h' is the residual stream after this layer's additions but one (it may be `h` updated in
    place, or a new tensor) and delta' this layer's not-yet-added output, so that the
    addition fuses with whatever norm comes next.
    """

    norm_slots: tuple[str, ...] = ()     # names of the norms this arrangement places
    uses_mixer = True
    uses_feed_forward = True

    def __init__(self, mixer: Mixer | None, feed_forward: FeedForward | None, norms: dict[str, Norm]):
        if set(norms) != set(self.norm_slots):
            raise ValueError(f"{type(self).__name__} places the norms {sorted(self.norm_slots)}, the layer gives {sorted(norms)}")
        if (mixer is not None) != self.uses_mixer or (feed_forward is not None) != self.uses_feed_forward:
            raise ValueError(f"{type(self).__name__} arranges {'a' if self.uses_mixer else 'no'} mixer and "
                             f"{'a' if self.uses_feed_forward else 'no'} feed-forward")
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = dict(norms)

    def parts(self) -> list[Part]:
        return [p for p in (*(self.norms[s] for s in self.norm_slots), self.mixer, self.feed_forward) if p is not None]

    def forward(self, h, delta, ctx, cache, state):
        raise NotImplementedError


# --------------------------------------------------------------------------- registries
MIXERS: dict[str, Callable[..., Mixer]] = {}
FEED_FORWARDS: dict[str, Callable[..., FeedForward]] = {}
NORMS: dict[str, Callable[..., Norm]] = {}
POSITION_ENCODINGS: dict[str, Callable[..., PositionEncoding]] = {}
BLOCKS: dict[str, Callable[..., Block]] = {}
EMBEDDINGS: dict[str, Callable[..., Part]] = {}
OUTPUT_HEADS: dict[str, Callable[..., Part]] = {}

_REGISTRIES = {
    "mixer": MIXERS,
    "feed_forward": FEED_FORWARDS,
    "norm": NORMS,
    "position_encoding": POSITION_ENCODINGS,
    "block": BLOCKS,
    "embedding": EMBEDDINGS,
    "output_head": OUTPUT_HEADS,
}


def register_part(family: str, kind: str, factory: Callable[..., Any], replace: bool = False) -> None:
    """Add a part under `kind` to one of the families: mixer, feed_forward, norm,
    position_encoding, block, embedding, output_head."""
    reg = _REGISTRIES[family]
    if kind in reg and not replace:
        raise ValueError(f"{family} '{kind}' is already registered")
    reg[kind] = factory


def make_part(family: str, spec: PartSpec, **context) -> Any:
    """Build the part `spec.kind` of `family` with `spec.params`, its name prefix and the
    sizes the surrounding model gives every part (`context`, e.g. hidden_size)."""
    reg = _REGISTRIES[family]
    if spec.kind not in reg:
        raise KeyError(f"unknown {family} kind '{spec.kind}' (registered: {', '.join(sorted(reg)) or 'none'})")
    return reg[spec.kind](prefix=spec.prefix, **context, **dict(spec.params))
