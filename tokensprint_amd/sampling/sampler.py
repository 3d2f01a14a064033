"""Greedy and temperature sampling.

The reference samples with logits/T -> softmax -> divide by Exp(1) noise -> argmax
(engine/generation/sampler.py:10-16), which draws token i with probability
softmax(logits/T)[i]; its noise comes from the global generator, so a token depends on
the order of the batch.  Here the same draw is argmax(logits/T - log E) and the noise
of a (request, token index, vocabulary index) comes from a counter hash, so a request's
tokens do not change with batching, portions or recomputation after preemption.
Temperature 0 is greedy argmax, which the reference refuses (config.py:14-15).
"""

from __future__ import annotations

import torch

_MASK = (1 << 64) - 1


def mix64(z: int) -> int:
    """The 64-bit finaliser the sampling kernel uses, on Python integers."""
    z &= _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def noise_key(engine_seed: int, request_seed: int, request_ordinal: int, token_index: int) -> int:
    """Key of one draw: which engine, which request, which of its tokens."""
    k = mix64(engine_seed + 0x9E3779B97F4A7C15)
    k = mix64(k ^ mix64(request_seed + 0x632BE59BD9B4E019))
    k = mix64(k ^ mix64(request_ordinal + 0x85157AF5))
    return mix64(k ^ mix64(token_index + 0x2545F4914F6CDD1D))


def _signed(k: int) -> int:
    return k - (1 << 64) if k >= (1 << 63) else k


class Sampler:
    def __init__(self, ops, device, engine_seed: int = 0) -> None:
        self.ops, self.device, self.engine_seed = ops, device, engine_seed

    def inputs(self, requests, token_indices=None):
        """(temperatures, keys) as host lists, one per request: what the sampling kernel
        takes.  A greedy request has temperature 0 and needs no key.  `token_indices`:
        which completion token each request draws, if not its next one."""
        if token_indices is None:
            token_indices = [r.num_completion_tokens for r in requests]
        temps = [r.temperature if r.temperature > 1e-10 else 0.0 for r in requests]
        keys = [_signed(noise_key(self.engine_seed, r.seed, r.ordinal, k))
                if t > 0.0 else 0 for r, t, k in zip(requests, temps, token_indices)]
        return temps, keys

    def __call__(self, logits: torch.Tensor, requests) -> list[int]:
        """One token per row of logits; `requests[r]` has .temperature, .seed, .ordinal
        and .num_completion_tokens (the index of the token being drawn)."""
        if logits.shape[0] != len(requests):
            raise ValueError("one request per row of logits")
        if not requests:
            return []
        if all(r.temperature <= 1e-10 for r in requests):
            return self.ops.argmax(logits).tolist()
        temps = torch.tensor([r.temperature for r in requests], dtype=torch.float32)
        keys = torch.tensor(
            [_signed(noise_key(self.engine_seed, r.seed, r.ordinal, r.num_completion_tokens))
             for r in requests], dtype=torch.int64)
        return self.ops.sample(logits, temps.to(self.device), keys.to(self.device)).tolist()
