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


class LayerSpec:
    """One set of weights: the parts one block is put together from, by role.

    Which roles there are, which of them a layer may leave out and which registry serves
    each is the block kind's business (`Block.ROLES`).  The pre-norm block has `mixer`,
    `feed_forward`, `mixer_norm` and `ffn_norm`, which may also be given in that order;
    another block kind may name other roles (a norm behind the mixer, no feed-forward).
    """

    __slots__ = ("block", "parts")
    _ORDER = ("mixer", "feed_forward", "mixer_norm", "ffn_norm")

    def __init__(self, block: str, *in_order: PartSpec, **by_role: PartSpec | None) -> None:
        if len(in_order) > len(self._ORDER):
            raise TypeError(f"at most {len(self._ORDER)} parts can be given by position")
        parts = dict(zip(self._ORDER, in_order))
        for role, spec in by_role.items():
            if role in parts:
                raise TypeError(f"part '{role}' given twice")
            if spec is not None:
                parts[role] = spec
        object.__setattr__(self, "block", block)
        object.__setattr__(self, "parts", parts)

    def __setattr__(self, name, value):
        raise AttributeError("a LayerSpec is not changed after it is made")

    def __getattr__(self, role):
        try:
            return self.parts[role]
        except KeyError:
            raise AttributeError(f"this layer has no part '{role}'") from None

    def __eq__(self, other):
        return isinstance(other, LayerSpec) and (self.block, self.parts) == (other.block, other.parts)

    def __repr__(self):
        return f"LayerSpec({self.block!r}, " + ", ".join(f"{k}={v!r}" for k, v in self.parts.items()) + ")"


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
