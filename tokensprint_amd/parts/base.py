"""Interfaces of the parts a layer is put together from, and their registries.

A part is built from a `PartSpec` (its sizes and constants) and a `BuildContext`
(kernels, dtype, device, shared position encodings).  It declares the checkpoint
tensors it needs by full name, receives them once, and then only sees activations,
the step's batch description and, for a mixer, the cache of the run it executes.
No part knows which model it is in.

Registries map a `kind` string to a class, one registry per role:
`MIXERS`, `FEED_FORWARDS`, `NORMS`, `POSITIONS`, `BLOCKS`, `EMBEDDINGS`, `HEADS`.  A test
or a new architecture adds a part with `register(MIXERS, "my_kind")(MyClass)`.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable

import torch

# ------------------------------------------------------------------ declarations


@dataclass(frozen=True)
class TensorDecl:
    """A checkpoint tensor a part needs.

    role "matrix": used in a matrix product or as an embedding table; kept in the
    run dtype unless the file stores it in 32-bit.  role "vector": a small per-
    channel vector (norm weight); always held in float32, which is exact for
    bfloat16 values.  role "table": an integer table, held as int32.
    """

    shape: tuple[int, ...]
    role: str = "matrix"
    optional: bool = False      # may be absent from the file (e.g. a tied head's copy)


@dataclass(frozen=True)
class PagedKVNeed:
    """Keys and values per token, in pages.  window None = every earlier key."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class SlotStateNeed:
    """A fixed-size per-request state tensor (shape without the slot axis)."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class BuildContext:
    ops: Any                    # kernel provider (see tokensprint_amd.kernels)
    dtype: torch.dtype          # activation dtype: bfloat16 or float32
    device: torch.device
    width: int
    positions: dict[str, "PositionEncoding"] = field(default_factory=dict)


# ------------------------------------------------------------------ part roles


class Part:
    def __init__(self, spec_params: dict, ctx: BuildContext) -> None:
        self.params = dict(spec_params)
        self.ctx = ctx
        self.ops = ctx.ops

    def tensors(self) -> dict[str, TensorDecl]:
        """Checkpoint name -> declaration, for every tensor this part reads."""
        return {}

    def load(self, get: Callable[[str], torch.Tensor | None]) -> None:
        """Take the declared tensors (`get(name)`, None if optional and absent)."""

    #: False for a part that cannot run inside a captured graph (it synchronises with the
    #: host, or its work depends on values the host reads from the device).  A decode step
    #: of a model with such a part always runs eagerly.  A part that leaves this True must,
    #: in a decode step, use only the batch's device tensors: the host lists of a captured
    #: batch (`q_lens`, `starts`) are placeholders.
    capturable = True

    def held_tensors(self) -> list[torch.Tensor]:
        """Every tensor this part keeps on the device (weights taken in `load`, tables)."""
        out = []
        for value in vars(self).values():
            for t in value if isinstance(value, (list, tuple)) else (value,):
                if isinstance(t, torch.Tensor):
                    out.append(t)
        return out

    def step_read_tensors(self) -> list[torch.Tensor]:
        """The tensors a step reads whole, whatever its tokens are: what a decode step's
        memory traffic is counted from.  Default: everything held."""
        return self.held_tensors()


class Norm(Part):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """Normalised copy of x [T, width] in the activation dtype."""
        raise NotImplementedError

    def add_forward(self, resid: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        """resid += delta (float32, in place), then the norm of the new resid."""
        raise NotImplementedError


class PositionEncoding(Part):
    """Applied by a mixer to its queries and keys.

    `rotary_tables()` returns (cos, sin) float32 [max_position, dim/2] for the
    fused rotate-half kernel, or None; then the mixer calls `apply` instead.
    """

    def rotary_tables(self):
        return None

    def apply(self, q: torch.Tensor, k: torch.Tensor | None, positions: torch.Tensor) -> None:
        """Encode positions into q [T, nq, hd] and k [T, nkv, hd] in place."""
        raise NotImplementedError


class Mixer(Part):
    def cache_need(self) -> PagedKVNeed | SlotStateNeed | None:
        return None

    def forward(self, h: torch.Tensor, batch, cache, write_cache: bool) -> torch.Tensor:
        """h [T, width] -> [T, width].  `cache` is this run's cache view (or None)."""
        raise NotImplementedError

    def stream_hint(self, norm: Norm):
        """What this part lets the producer of the stream know about its first product
        behind `norm`, or None.  Whatever it returns comes back as `hint` to the part
        that runs before it; the kernel provider's fused forms define the one kind there
        is (tokensprint_amd.kernels.stream), and a part may ignore all of it."""
        return None

    def forward_from_stream(self, resid, delta, norm: Norm, batch, cache, write_cache: bool,
                            hint=None):
        """The same from the residual stream: adds `delta` (may be None) to `resid`,
        norms, mixes.  Returns (output, residual stream after the add).  A part overrides
        this to fuse the add and the norm into its first product.  `hint` is the
        `stream_hint` of whatever reads the stream next, or None; a part may ignore it."""
        h = norm.forward(resid) if delta is None else norm.add_forward(resid, delta)
        return self.forward(h, batch, cache, write_cache), resid


class FeedForward(Part):
    def forward(self, h: torch.Tensor, batch) -> torch.Tensor:
        raise NotImplementedError

    def stream_hint(self, norm: Norm):
        """See Mixer.stream_hint."""
        return None

    def forward_from_stream(self, resid, delta, norm: Norm, batch, hint=None):
        """See Mixer.forward_from_stream."""
        h = norm.forward(resid) if delta is None else norm.add_forward(resid, delta)
        return self.forward(h, batch), resid


class TokenEmbedding(Part):
    """The model's first part: token ids (int32 [T]) -> the residual stream, float32
    [T, width]."""

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class OutputHead(Part):
    """The model's last part: rows of the residual stream -> logits, float32 [R, vocab]."""

    def forward_from_stream(self, resid: torch.Tensor, delta, norm: Norm) -> torch.Tensor:
        """Logits of the rows of the stream (`resid` float32, `delta` the last sub-layer's
        output not yet added, or None) behind the model's final `norm`."""
        raise NotImplementedError


class Block:
    """Arrangement of one layer's parts around the residual stream.

    `ROLES` names the parts a layer of this kind is made of: role -> (registry, required).
    The model builds each part a `LayerSpec` gives from the role's registry and hands them
    over by role; they become attributes of the block (a role the layer leaves out is
    None).

    The stream travels as (resid, delta): resid is float32 [T, width]; delta is
    the last sub-layer's output not yet added (None at the very start), so the
    add can be fused into the next norm.  Where the part that reads the stream next
    gives a `stream_hint`, the part before it may hand on, instead of a delta, whatever
    that hint's protocol defines; only that reader ever sees it.
    """

    ROLES: dict[str, tuple[dict, bool]] = {}

    def __init__(self, parts: dict[str, Part], ctx: BuildContext) -> None:
        unknown = sorted(set(parts) - set(self.ROLES))
        missing = sorted(r for r, (_, required) in self.ROLES.items()
                         if required and parts.get(r) is None)
        if unknown or missing:
            raise ValueError(f"{type(self).__name__}: unknown parts {unknown}, missing parts "
                             f"{missing}; its roles are {sorted(self.ROLES)}")
        for role in self.ROLES:
            setattr(self, role, parts.get(role))
        self.ctx = ctx

    def parts(self) -> list[Part]:
        return [getattr(self, role) for role in self.ROLES if getattr(self, role) is not None]

    def cache_need(self):
        """What a run of this block keeps per request: its mixer's need, if it has one."""
        mixer = getattr(self, "mixer", None)
        return mixer.cache_need() if mixer is not None else None

    def entry_hint(self):
        """The `stream_hint` of the part of this block that reads the stream first."""
        return None

    def forward(self, resid, delta, batch, cache, write_cache: bool, next_hint=None):
        """`next_hint`: the `entry_hint` of the block that runs next, or None."""
        raise NotImplementedError


# ------------------------------------------------------------------ registries

MIXERS: dict[str, type] = {}
FEED_FORWARDS: dict[str, type] = {}
NORMS: dict[str, type] = {}
POSITIONS: dict[str, type] = {}
BLOCKS: dict[str, type] = {}
EMBEDDINGS: dict[str, type] = {}
HEADS: dict[str, type] = {}


def register(registry: dict[str, type], kind: str, *, replace: bool = False):
    def deco(cls):
        if kind in registry and not replace:
            raise ValueError(f"part kind '{kind}' already registered")
        registry[kind] = cls
        return cls
    return deco


def build_part(registry: dict[str, type], spec, ctx: BuildContext):
    if spec.kind not in registry:
        raise ValueError(f"unknown part kind '{spec.kind}'; registered: {sorted(registry)}")
    return registry[spec.kind](dict(spec.params), ctx)
