"""Dense SwiGLU feed-forward: down(silu(gate(h)) * up(h)), no bias
(engine/nn/layers.py:61-66).  Gate and up run as one product over row-concatenated
weights, with the activation applied as the product is written where the kernel
can, and by a separate kernel over both halves otherwise."""

from __future__ import annotations

import torch

from tokensprint_amd.kernels.stream import StreamProducts, fused_rmsnorm_of
from tokensprint_amd.parts.base import FEED_FORWARDS, FeedForward, TensorDecl, register


@register(FEED_FORWARDS, "swiglu")
class SwiGLU(StreamProducts, FeedForward):
    """params: prefix, inner_dim."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.prefix = params["prefix"]
        self.inner = int(params["inner_dim"])
        self.w_gate_up = self.w_down = None

    def tensors(self):
        H, I, pre = self.ctx.width, self.inner, self.prefix
        return {pre + "gate_proj.weight": TensorDecl((I, H)),
                pre + "up_proj.weight": TensorDecl((I, H)),
                pre + "down_proj.weight": TensorDecl((H, I))}

    def load(self, get):
        pre = self.prefix
        g, u = get(pre + "gate_proj.weight"), get(pre + "up_proj.weight")
        if g.dtype != u.dtype:
            raise ValueError(f"{pre}: gate and up weights are stored in different dtypes")
        self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        self.w_down = get(pre + "down_proj.weight")

    def stream_hint(self, norm):
        return self.first_product_hint(norm, self.w_gate_up, silu_mul=True)

    def forward_from_stream(self, resid, delta, norm, batch, hint=None):
        fused = fused_rmsnorm_of(norm)
        if fused is None:
            return super().forward_from_stream(resid, delta, norm, batch)
        act, resid = self.ops.norm_linear(resid, delta, fused[0], fused[1], self.w_gate_up,
                                          self.ctx.dtype, silu_mul=True)
        return self.last_product(act, self.w_down, resid, hint), resid

    def forward(self, h, batch):
        act = self.ops.linear_silu_mul(h, self.w_gate_up, self.ctx.dtype)
        return self.ops.linear(act, self.w_down, self.ctx.dtype)
