"""Pre-norm arrangement: x = x + mixer(norm(x)); x = x + ffn(norm(x))
(engine/nn/layers.py:111-121).  Each residual add is fused into the following norm.
A layer may leave out one of the two sub-layers (its part and its norm together)."""

from __future__ import annotations

from tokensprint_amd.parts.base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block, register


@register(BLOCKS, "pre_norm")
class PreNormBlock(Block):
    ROLES = {"mixer_norm": (NORMS, False), "mixer": (MIXERS, False),
             "ffn_norm": (NORMS, False), "feed_forward": (FEED_FORWARDS, False)}

    def __init__(self, parts, ctx):
        super().__init__(parts, ctx)
        if (self.mixer is None) != (self.mixer_norm is None) or \
                (self.feed_forward is None) != (self.ffn_norm is None):
            raise ValueError("pre_norm: a sub-layer and its norm come together")
        if self.mixer is None and self.feed_forward is None:
            raise ValueError("pre_norm: a layer needs a mixer or a feed-forward")

    def entry_hint(self):
        if self.mixer is not None:
            return self.mixer.stream_hint(self.mixer_norm)
        return self.feed_forward.stream_hint(self.ffn_norm)

    def forward(self, resid, delta, batch, cache, write_cache, next_hint=None):
        if self.mixer is not None:
            hint = self.feed_forward.stream_hint(self.ffn_norm) \
                if self.feed_forward is not None else next_hint
            delta, resid = self.mixer.forward_from_stream(
                resid, delta, self.mixer_norm, batch, cache, write_cache, hint=hint)
        if self.feed_forward is not None:
            delta, resid = self.feed_forward.forward_from_stream(
                resid, delta, self.ffn_norm, batch, hint=next_hint)
        return resid, delta
