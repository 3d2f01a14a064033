"""Pre-norm arrangement: x = x + mixer(norm(x)); x = x + ffn(norm(x))
(engine/nn/layers.py:111-121).  Each residual add is fused into the following norm."""

from __future__ import annotations

from tokensprint_amd.parts.base import BLOCKS, Block, register


@register(BLOCKS, "pre_norm")
class PreNormBlock(Block):
    def forward(self, resid, delta, batch, cache, write_cache):
        h = self.mixer_norm.forward(resid) if delta is None \
            else self.mixer_norm.add_forward(resid, delta)
        a = self.mixer.forward(h, batch, cache, write_cache)
        h = self.ffn_norm.add_forward(resid, a)
        f = self.feed_forward.forward(h, batch)
        return resid, f
