"""What travels between the product that ends a sub-layer and the norm and product that
follow it, when a kernel provider fuses the residual add and the norm into the two."""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class NormHint:
    """What the producer of a sub-layer's output may be told about its consumer: the
    RMSNorm (weight, eps) the residual stream goes through next, and the first product
    after it (its weight; `silu_mul` as in the provider's `norm_linear`)."""

    norm_weight: torch.Tensor
    eps: float
    weight: torch.Tensor
    silu_mul: bool = False


@dataclass(frozen=True)
class PreparedRows:
    """A sub-layer's output already added into the residual stream, and the stream handed
    on prepared for the RMSNorm of `hint`: `rows` [M, K] = stream * norm weight (bfloat16,
    not yet divided by the row's root mean square) and `sumsq` [slices, M], the
    rows' sums of squares in slices of 16 or fewer columns.  Stands where the stream's `delta` does,
    and only the provider's `norm_linear` with the hinted norm and weight takes it."""

    rows: torch.Tensor
    sumsq: torch.Tensor
    hint: NormHint
