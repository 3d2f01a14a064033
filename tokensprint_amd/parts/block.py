"""Pre-norm arrangement: x = x + mixer(norm(x)); x = x + ffn(norm(x))
(engine/nn/layers.py:111-121).  Each residual add is fused into the following norm."""

from __future__ import annotations

from tokensprint_amd.parts.base import BLOCKS, Block, register


@register(BLOCKS, "pre_norm")
class PreNormBlock(Block):
    def entry_hint(self):
        return self.mixer.stream_hint(self.mixer_norm)

    def forward(self, resid, delta, batch, cache, write_cache, next_hint=None):
        a, resid = self.mixer.forward_from_stream(
            resid, delta, self.mixer_norm, batch, cache, write_cache,
            hint=self.feed_forward.stream_hint(self.ffn_norm))
        f, resid = self.feed_forward.forward_from_stream(resid, a, self.ffn_norm, batch,
                                                         hint=next_hint)
        return resid, f
