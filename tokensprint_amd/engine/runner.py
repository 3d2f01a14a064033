"""The step function: a batch of (request, its next tokens) -> logits at wanted places.

Counterpart of the reference's ModelRunner.run / run_model
(engine/generation/model_runner.py:183-201), with sampling taken out so that the
caller (scheduler loop, trace replay) decides what to do with the logits.  A step
runs only the tokens it is given, as one flat batch, against the cache earlier steps
left; portions of prompts and single decoded tokens may be mixed and cut anywhere.
"""

from __future__ import annotations

import torch

from tokensprint_amd.cache import CacheManager, CacheStorage, page_bytes
from tokensprint_amd.engine.batch import BatchBuilder, StepBatch, StepEntry
from tokensprint_amd.models.model import Model


class ModelRunner:
    def __init__(self, model: Model, *, page_size: int, num_pages: int, num_slots: int,
                 cache_dtype: torch.dtype | None = None) -> None:
        self.model = model
        self.device = model.ctx.device
        self.dtype = model.ctx.dtype
        needs = model.cache_needs()
        self.storage = CacheStorage(needs, page_size, num_pages, num_slots,
                                    cache_dtype or self.dtype, self.device)
        self.manager = CacheManager(self.storage.groups, page_size, num_pages, num_slots)
        self.builder = BatchBuilder(self.device, len(self.storage.groups),
                                    vocab_size=model.spec.vocab_size,
                                    max_position=model.spec.max_position)
        self.page_size = page_size

    @staticmethod
    def pages_that_fit(model: Model, page_size: int, free_bytes: int,
                       cache_dtype: torch.dtype) -> int:
        """Page ids affordable in `free_bytes` (every group gets that many pages);
        the arithmetic of engine/generation/model_runner.py:400-411."""
        from tokensprint_amd.cache.storage import group_runs
        groups, _ = group_runs(model.cache_needs())
        per_page = page_bytes(groups, page_size, cache_dtype)
        return int(free_bytes // max(per_page, 1))

    def build(self, entries: list[StepEntry], table_width=None) -> StepBatch:
        return self.builder.build(entries, table_width)

    @torch.inference_mode()
    def run(self, batch: StepBatch) -> torch.Tensor:
        return self.model.forward(batch, self.storage.views)

    def step(self, entries: list[StepEntry]) -> torch.Tensor:
        """Logits float32 [sum(len(e.want)), vocab], in the order of entries and want."""
        return self.run(self.build(entries))
