"""A model as data: which parts each layer is made of and in which order layers run.

An architecture module turns its typed configuration into a `ModelSpec`; nothing
below this file knows which architecture it serves.  Parts are named by registry
key (`kind`) and carry their sizes and constants in `params`, so two layers of one
model may use different mixers or feed-forwards, the run order may name a layer
twice, and a run may read the cache another run writes.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping


@dataclass(frozen=True)
class PartSpec:
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One set of weights: a mixer and a feed-forward, each behind a norm."""

    block: str                 # arrangement of the parts, e.g. "pre_norm"
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    ffn_norm: PartSpec


@dataclass(frozen=True)
class Run:
    """One execution of a layer.

    `cache_of` names the run (index into `ModelSpec.order`) whose cache this run
    uses; None means its own.  A run that uses another run's cache only reads it.
    """

    layer: int
    cache_of: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    width: int
    vocab_size: int
    embedding: PartSpec
    positions: Mapping[str, PartSpec]     # shared position encodings, by name
    layers: tuple[LayerSpec, ...]
    order: tuple[Run, ...]
    final_norm: PartSpec
    head: PartSpec
    max_position: int
    eos_token_id: int | None = None       # the checkpoint's end-of-sequence token, if it names one

    def validate(self) -> None:
        if not self.order:
            raise ValueError("a model needs at least one run")
        for r, run in enumerate(self.order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"run {r} names layer {run.layer}, model has {len(self.layers)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < r:
                    raise ValueError(
                        f"run {r} reads the cache of run {run.cache_of}, which must come earlier")
                if self.order[run.cache_of].cache_of is not None:
                    raise ValueError(
                        f"run {r} reads the cache of run {run.cache_of}, which owns none")
