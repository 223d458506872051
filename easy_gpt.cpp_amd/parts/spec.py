"""Data that describes a model: which parts each layer has and in which order layers run.

A model is data before it is objects.  An architecture turns its typed
configuration into a `ModelSpec`; `parts.model.build_model` turns that into part
objects through the part registries.  Nothing in here knows any architecture.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping


@dataclass(frozen=True)
class ParamSpec:
    """One tensor of the weights file.

    role    how random weights draw it: 'matrix', 'embedding', 'bias' ~ N(0, 0.02);
            'norm_scale' ~ 1 + N(0, 0.02); 'int_table' uniform integers; or any role that was added
            with `weights.register_role` (a decay in (0, 1), a table of a special form, ...)
    dtype   'compute' (cast to the engine's dtype), 'float32' or 'int32' (kept as stored)
    alt_shapes  other shapes accepted on load (the reference accepts [H, 1] for a
            norm weight, /root/reference/src/models/model_param_validation.cpp:62-74)
    """

    name: str
    shape: tuple[int, ...]
    role: str = "matrix"
    dtype: str = "compute"
    alt_shapes: tuple[tuple[int, ...], ...] = ()


@dataclass(frozen=True)
class PartSpec:
    """A part chosen by `kind` from its registry, its parameters and the prefix of its tensor names."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)
    prefix: str = ""


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block arrangement with the parts it arranges.

    norms   the layer's norms by the slot names that the block arrangement declares (`Block.norm_slots`:
            'mixer' and 'feed_forward' for the pre-norm block; an arrangement with norms before and after each
            branch declares four, one with a single shared norm one)
    mixer, feed_forward   None where the arrangement has no such part (`Block.uses_mixer`, `uses_feed_forward`)
    """

    block: str
    mixer: PartSpec | None
    feed_forward: PartSpec | None
    norms: Mapping[str, PartSpec] = field(default_factory=dict)


@dataclass(frozen=True)
class RunSpec:
    """One entry of the run order.

    layer         index into ModelSpec.layers (a layer may be named more than once)
    cache         id of the cache slab its mixer reads; entries with the same id share keys
                  and values; None for a mixer without a paged cache
    writes_cache  False when the mixer only reads a slab that an earlier entry wrote
    state         id of the per-request state record of its mixer, None if it has none
    """

    layer: int
    cache: int | None = None
    writes_cache: bool = True
    state: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_position: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    run_order: tuple[RunSpec, ...]
    final_norm: PartSpec
    output_head: PartSpec
    ignorable_tensors: tuple[str, ...] = ()
    bos_token_id: int = -1
    eos_token_id: int = -1
