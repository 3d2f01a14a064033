"""RMSNorm.  Formula of engine/kernels/triton/rmsnorm.py:19-42 (float32 sum of
squares, rstd = rsqrt(sum/dim + eps), x*rstd*w, one rounding at the store)."""

from __future__ import annotations

from tokensprint_amd.parts.base import NORMS, Norm, TensorDecl, register


@register(NORMS, "rmsnorm")
class RMSNorm(Norm):
    """params: dim, eps, weight (checkpoint name)."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.dim = int(params["dim"])
        self.eps = float(params["eps"])
        self.weight_name = params["weight"]
        self.weight = None

    def tensors(self):
        return {self.weight_name: TensorDecl((self.dim,), role="vector")}

    def load(self, get):
        self.weight = get(self.weight_name)

    def fused_rmsnorm(self):
        return self.weight, self.eps

    def forward(self, x):
        return self.ops.rmsnorm(x, self.weight, self.eps, self.ctx.dtype)

    def add_forward(self, resid, delta):
        return self.ops.add_rmsnorm(resid, delta, self.weight, self.eps, self.ctx.dtype)
