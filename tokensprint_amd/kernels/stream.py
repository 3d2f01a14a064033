"""What travels between the product that ends a sub-layer and the norm and product that
follow it, when a kernel provider fuses the residual add and the norm into the two, and
the optional mixins through which parts take part in that.  The part interfaces
(tokensprint_amd.parts.base) know none of this: a part that uses neither mixin works
between parts that do."""

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
    not yet divided by the row's root mean square) and `sumsq`, the rows' sums of squares
    in `slices` slices of columns, laid out as the producing kernel and its counterpart
    agree ([M, slices rounded up to four] from the kernels for few rows, [slices, M] from
    the tiled product's).  Stands where the stream's `delta` does, and only the provider's
    `norm_linear` with the hinted norm and weight takes it."""

    rows: torch.Tensor
    sumsq: torch.Tensor
    slices: int
    hint: NormHint


class UnmergedRows:
    """What `attend(defer_merge=True)` may return in place of a tensor: a decode step's
    attention output whose key splits have not been merged yet.  It is deliberately no
    tensor.  The provider's `linear_into_stream` takes it and lets the product's kernel do
    the merge; its other calls that take activation rows (`linear`, `norm_linear`, ...)
    merge first; `merged()` gives the tensor to anyone else; and anything that treats it
    as a tensor fails loudly instead of reading rows that are not there yet.  `view` gives
    the same pending rows another logical shape."""

    def __init__(self, pending, shape):
        self._pending, self.shape = pending, torch.Size(shape)

    @property
    def dtype(self):
        return self._pending.out.dtype

    @property
    def device(self):
        return self._pending.out.device

    @property
    def is_merged(self) -> bool:
        return self._pending.done

    def view(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list, torch.Size)):
            shape = tuple(shape[0])
        if torch.Size(shape).numel() != self.shape.numel():
            raise ValueError(f"cannot view rows of shape {tuple(self.shape)} as {tuple(shape)}")
        return UnmergedRows(self._pending, shape)

    def merged(self) -> torch.Tensor:
        """The attention output as a tensor; runs the merge if nothing has yet."""
        self._pending.merge()
        return self._pending.out.view(self.shape)


def fused_rmsnorm_of(norm):
    """(weight, eps) if `norm` says it is a plain RMSNorm that a kernel may fuse into the
    product after it (it has a `fused_rmsnorm()` that returns them), else None."""
    probe = getattr(norm, "fused_rmsnorm", None)
    return probe() if callable(probe) else None


class StreamProducts:
    """Mixin for a part (with `.ops` and `.ctx`) whose first product may take the residual
    add and RMSNorm before it, and whose last product may add itself into the stream."""

    def first_product_hint(self, norm, weight: torch.Tensor, silu_mul: bool = False):
        """For `stream_hint`: the hint, if `norm` can be fused and the provider has the
        kernels, else None."""
        fused = fused_rmsnorm_of(norm)
        if fused is None or not hasattr(self.ops, "linear_into_stream"):
            return None
        return NormHint(fused[0], fused[1], weight, silu_mul)

    def last_product(self, x: torch.Tensor, weight: torch.Tensor, resid: torch.Tensor, hint):
        """The product that ends a sub-layer: x W^T as the stream's next delta, or, where
        `hint` (a NormHint) says what follows and the provider can, added into `resid` at
        once and handed on as PreparedRows (which stand in delta's place)."""
        if isinstance(hint, NormHint):
            prepared = self.ops.linear_into_stream(x, weight, resid, hint)
            if prepared is not None:
                return prepared
        return self.ops.linear(x, weight, self.ctx.dtype)
