"""The step function: a batch of (request, its next tokens) -> logits at wanted places.

Counterpart of the reference's ModelRunner.run / run_model
(engine/generation/model_runner.py:183-201), with sampling taken out so that the
caller (scheduler loop, trace replay) decides what to do with the logits.  A step
runs only the tokens it is given, as one flat batch, against the cache earlier steps
left; portions of prompts and single decoded tokens may be mixed and cut anywhere.
"""

from __future__ import annotations

import time

import torch

from tokensprint_amd.cache import CacheManager, CacheStorage, page_bytes
from tokensprint_amd.engine.batch import BatchBuilder, StaticDecodeBatch, StepBatch, StepEntry
from tokensprint_amd.models.model import Model


class ModelRunner:
    def __init__(self, model: Model, *, page_size: int, num_pages: int, num_slots: int,
                 cache_dtype: torch.dtype | None = None, graph_max_len: int | None = None,
                 graph_max_batch: int = 256) -> None:
        """`graph_max_len`: the longest request a captured decode graph must serve (its
        block tables are that wide); None means every step runs eagerly."""
        self.model = model
        self.device = model.ctx.device
        self.dtype = model.ctx.dtype
        needs = model.cache_needs()
        self.storage = CacheStorage(needs, page_size, num_pages, num_slots,
                                    cache_dtype or self.dtype, self.device)
        self.manager = CacheManager(self.storage.groups, page_size, num_pages, num_slots,
                                    state_runs=self.storage.state_runs)
        self.builder = BatchBuilder(self.device, len(self.storage.groups),
                                    vocab_size=model.spec.vocab_size,
                                    max_position=model.spec.max_position)
        self.page_size = page_size
        self.num_slots = num_slots
        self.graph_max_len = graph_max_len
        self.graphs: dict[int, tuple] = {}      # bucket -> (graph, static batch, logits, tokens)
        self._graph_pool = None                 # one memory pool for every captured bucket
        self._last_drawn = 0                    # entries of the last captured step
        # a part that cannot be captured (it says so) keeps every step eager
        capture = bool(graph_max_len) and self.device.type == "cuda" and model.all_capturable()
        top = min(graph_max_batch, num_slots)
        self.buckets = sorted({b for b in [1, 2, 4, 8] + list(range(16, top + 1, 16)) + [top]
                               if b <= top}) if capture else []
        self._graph_widths = [-(-graph_max_len // page_size)] * len(self.storage.groups) \
            if capture else []
        # where every captured step leaves its drawn tokens, lane by lane, and where a
        # step launched before the host has seen them takes its tokens from
        self._drawn = torch.zeros(self.buckets[-1], dtype=torch.int32, device=self.device) \
            if self.buckets else None

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
        bucket = self._graph_bucket(entries)
        if bucket is not None:
            return self._replay(bucket, entries)[0]
        return self.run(self.build(entries))

    # ------------------------------------------------------------ captured decode steps
    # The reference captures model.decode for decode-only batches per batch-size bucket
    # and runs head and sampler eagerly (engine/generation/model_runner.py:203-390);
    # here the captured region also holds the head, and buckets are captured at first use.
    def _graph_bucket(self, entries):
        if not self.buckets or len(entries) > self.buckets[-1]:
            return None
        for e in entries:
            if len(e.tokens) != 1 or e.want != [0] or e.start + 1 > self.graph_max_len:
                return None
            # a cache extended beyond what the captured block tables can name (a caller
            # may reserve ahead) is served eagerly
            if any(len(t) > w for t, w in zip(e.cache.tables, self._graph_widths)):
                return None
        return next(b for b in self.buckets if b >= len(entries))

    def fits_captured(self, entries) -> bool:
        """True if `decode_and_sample` would serve these entries from a captured graph."""
        return self._graph_bucket(entries) is not None

    def _capture(self, bucket: int):
        static = StaticDecodeBatch(self.device, bucket, self._graph_widths,
                                   idle_slot=self.storage.idle_slot)
        static.batch.max_ctx_len = self.graph_max_len
        static.fill([])
        torch.cuda.synchronize(self.device)
        side = torch.cuda.Stream(self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        ops = self.model.ctx.ops
        timed_plans = getattr(ops, "timed_plans", lambda on: False)
        before = timed_plans(True)             # this step's shapes stay for the rest of the run
        try:
            with torch.cuda.stream(side):      # loads kernels, fills the batch's launch plans
                ops.take_tokens(static.batch.token_ids, static.token_sources, self._drawn)
                self.run(static.batch)
        finally:
            timed_plans(before)
        torch.cuda.current_stream(self.device).wait_stream(side)
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            # lanes whose token the step before drew and the host has not seen yet
            ops.take_tokens(static.batch.token_ids, static.token_sources, self._drawn)
            logits = self.run(static.batch)
            # the draw is part of the captured step: rows with temperature 0 are greedy
            tokens = ops.sample(logits, static.temperatures, static.keys,
                                out=self._drawn[:bucket])
        if self._graph_pool is None:
            self._graph_pool = graph.pool()
        self.graphs[bucket] = (graph, static, logits, tokens)
        return self.graphs[bucket]

    def capture_all(self) -> None:
        """Capture every decode bucket now, the largest first so that the smaller ones fit
        into the memory it took (engine/generation/model_runner.py:334,373-379 captures in
        that order for that reason).  Without this a bucket is captured at its first use."""
        self._reset_provider()
        self._choose_large_weight_rows()
        for bucket in reversed(self.buckets):
            if bucket not in self.graphs:
                self._capture(bucket)

    def _reset_provider(self) -> None:
        """What the kernel provider keeps between calls, back to its start (a provider
        without such state has no `reset_scratch`)."""
        reset = getattr(self.model.ctx.ops, "reset_scratch", None)
        if reset is not None:
            reset()

    def _choose_large_weight_rows(self) -> None:
        """Where the kernel provider has a choice to offer for the products of few rows
        with large weights (its own kernels or the vendor library's), take the one whose
        captured decode step of the smallest bucket replays faster; the default stays
        unless another is 3 % ahead.  The default's step is captured first: running it is
        how the provider meets the shapes, and if the default stays it is that bucket's
        graph."""
        ops = self.model.ctx.ops
        offers = getattr(ops, "large_weight_choices", None)
        if offers is None or not self.buckets or self.graphs:
            return
        bucket = self.buckets[0]

        def seconds(graph):
            for _ in range(3):
                graph.replay()
            torch.cuda.synchronize(self.device)
            start = time.perf_counter()
            for _ in range(10):
                graph.replay()
            torch.cuda.synchronize(self.device)
            return time.perf_counter() - start

        kept = self._capture(bucket)
        choices = offers()
        if len(choices) < 2:
            return
        best, best_seconds = choices[0], 0.97 * seconds(kept[0])
        for rows in choices[1:]:
            ops.try_large_weight_rows(rows)
            trial = self._capture(bucket)
            took = seconds(trial[0])
            if took < best_seconds:
                best, best_seconds, kept = rows, took, trial
        ops.keep_large_weight_rows(best)
        self.graphs[bucket] = kept

    def dummy_step(self, num_tokens: int, num_entries: int) -> int:
        """Run one step of `num_tokens` zero tokens in `num_entries` requests (fewer of
        either if the pool or the slots do not hold as many), each asking for its last
        token's logits, and give everything back: loads the kernels, lets the library
        choose its algorithms and shows what such a step costs in memory.  Returns the
        tokens it ran."""
        manager = self.manager
        if manager.live:
            raise RuntimeError("a dummy step needs an engine without live requests")
        n = max(1, min(num_entries, manager.slots.num_free, num_tokens))
        pool = min(p.num_free for p in manager.pools) if manager.pools else num_tokens
        longest = self.model.spec.max_position
        per = max(1, min(num_tokens // n, longest, (pool // n) * self.page_size))
        if manager.pools and pool < n:
            n, per = max(1, pool), min(self.page_size, longest)
        entries = []
        for i in range(n):
            rc = manager.admit(("dummy", i))
            manager.extend(rc, per)
            entries.append(StepEntry(rc, [0] * per, 0, [per - 1]))
        try:
            self._reset_provider()
            self.run(self.build(entries))
            if self.device.type == "cuda":
                torch.cuda.synchronize(self.device)
        finally:
            for e in entries:
                manager.free(e.cache)
        return n * per

    def decode_and_sample(self, entries: list[StepEntry], temperatures, keys, sources=None):
        """One decode step with the draw inside the captured graph: token ids (int32 device
        tensor, one per entry), or None if the step does not fit a captured graph.
        `temperatures` and `keys` are host sequences, one per entry.  The result is a
        view of the buffer every captured step draws into: read it (or enqueue its copy)
        before the next captured step.  `sources[i] >= 0` makes entry i's token the one
        the captured step before this one drew in that lane, so that a step can be
        launched before the host has seen the last one's tokens."""
        bucket = self._graph_bucket(entries)
        if bucket is None:
            return None
        if sources is not None and any(s >= self._last_drawn for s in sources):
            raise ValueError("a source lane beyond the entries of the step before")
        return self._replay(bucket, entries, temperatures, keys, sources)[1][:len(entries)]

    def _replay(self, bucket: int, entries: list[StepEntry], temperatures=None, keys=None,
                sources=None):
        graph, static, logits, tokens = self.graphs.get(bucket) or self._capture(bucket)
        vocab = self.model.spec.vocab_size
        for e in entries:
            if not 0 <= e.tokens[0] < vocab:
                raise ValueError(f"token id {e.tokens[0]} outside [0, {vocab})")
            if e.start + 1 > e.cache.num_tokens:
                raise ValueError(f"request {e.cache.request_id!r}: position {e.start} is not "
                                 "covered by its cache")
        static.fill(entries, temperatures, keys, sources)
        graph.replay()
        self._last_drawn = len(entries)
        return logits[:len(entries)], tokens
