"""Python entry point: LLMEngine(model, config, tokenizer).generate(prompts, params).

Surface of the reference's engine/generation/llm_engine.py:18-114: `add_request`,
`step` (schedule -> run -> postprocess), `generate` (enqueue all, loop until the
scheduler is empty, completions in request order), `is_finished`.  The tokenizer is
optional: prompts given as token-id lists need none.
"""

from __future__ import annotations

import logging
import time

import torch

from tokensprint_amd.config.engine_config import Config, SamplingParams
from tokensprint_amd.engine.batch import StepEntry
from tokensprint_amd.engine.request import Request, RequestStatus
from tokensprint_amd.engine.runner import ModelRunner
from tokensprint_amd.engine.scheduler import Scheduler
from tokensprint_amd.models.model import Model
from tokensprint_amd.sampling.sampler import Sampler

log = logging.getLogger(__name__)


class _Flight:
    """A step that has been launched.  `tokens` are its drawn tokens if the host has them
    already; otherwise they arrive in `host` once `event` has passed."""
    __slots__ = ("reqs", "sampled_index", "tokens", "host", "event", "positions",
                 "draw_index", "ahead")

    def __init__(self, reqs, sampled_index, tokens=None, host=None, event=None,
                 positions=None, draw_index=None, ahead=False):
        self.reqs, self.sampled_index, self.tokens = reqs, sampled_index, tokens
        self.host, self.event = host, event
        self.positions = positions      # per request: position of the token this step computes
        self.draw_index = draw_index    # per request: index of the completion token it draws
        self.ahead = ahead              # launched before the step before it was seen


class LLMEngine:
    def __init__(self, model: Model, config: Config, tokenizer=None) -> None:
        self.model, self.config, self.tokenizer = model, config, tokenizer
        if model.ctx.dtype != config.dtype:
            raise ValueError(f"model runs in {model.ctx.dtype}, config asks for {config.dtype}")
        page = config.kvcache_block_size
        on_gpu = model.ctx.device.type == "cuda"
        graph_len = None if config.enforce_eager or not on_gpu else config.max_model_len
        if hasattr(model.ctx.ops, "fold_merge"):
            model.ctx.ops.fold_merge = bool(config.fold_merge)
        # the shapes that the warm-up meets (the largest step, the captured decode steps)
        # are the ones the run is made of: their library plans are worth timing
        timed_plans = getattr(model.ctx.ops, "timed_plans", lambda on: False)
        before = timed_plans(config.warmup and on_gpu)
        try:
            self._set_up(model, config, page, on_gpu, graph_len)
        finally:
            timed_plans(before)

    def _set_up(self, model, config, page, on_gpu, graph_len) -> None:
        num_pages = config.num_kvcache_blocks
        if num_pages < 0:
            num_pages = self._pages_from_free_memory(model, config, graph_len)
            config.num_kvcache_blocks = num_pages
        self.runner = ModelRunner(
            model, page_size=page, num_pages=num_pages, num_slots=config.max_num_seqs,
            graph_max_len=graph_len)
        if config.enable_prefix_caching:
            self.runner.manager.enable_prefix_cache()
        if config.warmup and on_gpu:
            # before the first request: kernels loaded, the library's choices made, every
            # decode bucket captured (engine/generation/model_runner.py:28-35 warms up and
            # captures in its constructor)
            self.runner.dummy_step(*self.largest_step(config))
            self.runner.capture_all()
        self.scheduler = Scheduler(
            self.runner.manager, max_num_batched_tokens=config.max_num_batched_tokens,
            max_num_seqs=config.max_num_seqs, max_model_len=config.max_model_len,
            eos=config.eos, chunked_prefill=config.chunked_prefill)
        self.sampler = Sampler(model.ctx.ops, model.ctx.device, config.seed)
        self._next_ordinal = 0
        self.requests: dict[int, Request] = {}
        # decode steps in flight: the launched step whose tokens have not been read, and
        # two pinned buffers that take turns receiving a step's tokens
        self._flight: _Flight | None = None
        self._landing = []
        if self.runner.buckets:
            self._landing = [(torch.empty(self.runner.buckets[-1], dtype=torch.int32,
                                          pin_memory=True), torch.cuda.Event())
                             for _ in range(2)]
        self._turn = 0
        self.num_steps_ahead = 0        # steps launched before the step before them was seen

    @staticmethod
    def largest_step(config: Config) -> tuple[int, int]:
        """(tokens, requests) of the largest step the scheduler can put together: the
        token budget, or, when prefill is not chunked, a recomputed request of
        max_model_len - 1 tokens alone; as many requests as may be live, since each can
        ask for a row of logits."""
        tokens = config.max_num_batched_tokens
        if not config.chunked_prefill:
            tokens = max(tokens, config.max_model_len - 1)
        fewest = -(-tokens // (config.max_model_len - 1))
        return tokens, max(fewest, min(config.max_num_seqs, tokens))

    @staticmethod
    def measure_step_memory(model: Model, config: Config, graph_len) -> int:
        """Device bytes the engine needs beside weights and cache: the peak of its largest
        step plus what the captured decode graphs keep, measured on a throw-away cache
        just large enough for that step (the reference measures its dummy forward's peak
        the same way, engine/generation/model_runner.py:288-308,392-398)."""
        import gc
        device = model.ctx.device
        tokens, requests = LLMEngine.largest_step(config)
        page = config.kvcache_block_size
        torch.cuda.synchronize(device)
        torch.cuda.empty_cache()
        probe = ModelRunner(model, page_size=page, num_pages=-(-tokens // page) + requests,
                            num_slots=config.max_num_seqs, graph_max_len=graph_len)
        torch.cuda.synchronize(device)
        before = torch.cuda.memory_reserved(device)
        torch.cuda.reset_peak_memory_stats(device)
        probe.dummy_step(tokens, requests)
        step_peak = torch.cuda.max_memory_reserved(device) - before
        torch.cuda.empty_cache()
        before = torch.cuda.memory_reserved(device)
        probe.capture_all()
        torch.cuda.synchronize(device)
        torch.cuda.empty_cache()
        graphs = torch.cuda.memory_reserved(device) - before
        del probe
        gc.collect()
        torch.cuda.empty_cache()
        log.info("largest step (%d tokens, %d requests) peaks at %.1f MiB; captured graphs "
                 "keep %.1f MiB", tokens, requests, step_peak / 2**20, graphs / 2**20)
        return max(step_peak, 0) + max(graphs, 0)

    @staticmethod
    def _pages_from_free_memory(model: Model, config: Config, graph_len=None) -> int:
        """free * utilization minus the measured needs of the steps, in pages
        (engine/generation/model_runner.py:392-411)."""
        device = model.ctx.device
        if device.type != "cuda":
            raise ValueError("num_kvcache_blocks must be given when there is no GPU to size from")
        steps = LLMEngine.measure_step_memory(model, config, graph_len)
        free, _ = torch.cuda.mem_get_info(device)
        available = free * config.gpu_memory_utilization - steps
        pages = ModelRunner.pages_that_fit(model, config.kvcache_block_size, int(available),
                                           config.dtype)
        # no request can use more than max_model_len tokens
        cap = config.max_num_seqs * (-(-config.max_model_len // config.kvcache_block_size) + 1)
        pages = min(pages, cap)
        if pages < 1:
            raise RuntimeError("Insufficient GPU memory for the key/value cache: "
                               f"available={int(available)} bytes after {steps} bytes for the "
                               "steps themselves")
        log.info("key/value cache: %d pages of %d tokens", pages, config.kvcache_block_size)
        return pages

    # ------------------------------------------------------------ requests
    def _tokenize_prompt(self, prompt: str) -> list[int]:
        if self.tokenizer is None:
            raise ValueError("a text prompt needs a tokenizer; pass token ids instead")
        token_ids = self.tokenizer.encode(prompt, add_special_tokens=True)
        if not isinstance(token_ids, list):
            raise TypeError(f"the tokenizer's encode gave {type(token_ids).__name__}, "
                            "a list of token ids is needed")
        return token_ids

    def is_finished(self) -> bool:
        return self.scheduler.is_finished() and self._flight is None

    def add_request(self, prompt: str | list[int], sampling_params: SamplingParams) -> int:
        if isinstance(prompt, str):
            prompt = self._tokenize_prompt(prompt)
        vocab = self.model.spec.vocab_size
        if any(not 0 <= t < vocab for t in prompt):
            raise ValueError(f"prompt holds a token id outside [0, {vocab})")
        req = Request(self._next_ordinal, prompt, sampling_params)
        self.scheduler.add_request(req)
        self._next_ordinal += 1
        self.requests[req.ordinal] = req
        return req.ordinal

    # ------------------------------------------------------------ one step
    def step(self):
        """Finish one step: the one in flight, or a newly scheduled one.  While a captured
        decode step runs and the coming step is known without its tokens (nobody can be
        admitted, the same requests go on decoding), that step is launched first, taking
        its tokens on the device from the draw before it, so the GPU does not wait for the
        host's bookkeeping between decode steps."""
        flight = self._flight or self._launch(self.scheduler.schedule())
        self._flight = None
        if flight.event is not None and self.config.decode_ahead:
            try:
                self._flight = self._launch_ahead(flight)
            except BaseException:
                self._give_back_pages_taken_ahead(flight)
                raise
        try:
            return self._finish(flight)
        except BaseException:
            # the step that was launched ahead dies with the one it follows: nobody will
            # read its tokens, and the pages it took go back
            if self._flight is not None:
                self._give_back_pages_taken_ahead(flight)
                self._flight = None
            raise

    def _give_back_pages_taken_ahead(self, prev: _Flight) -> None:
        """After a failure around a step launched ahead of `prev`: every request of `prev`
        that still runs holds exactly the pages of the tokens it has and the one `prev`
        computes, as if nothing had been launched ahead."""
        manager = self.runner.manager
        for req, pos in zip(prev.reqs, prev.positions or []):
            if req.status is RequestStatus.RUNNING and req.cache is not None:
                manager.shrink(req.cache, pos + 1)

    def _land(self, drawn: torch.Tensor):
        """Enqueue the copy of a captured step's tokens to the host."""
        host, event = self._landing[self._turn]
        self._turn ^= 1
        host[:drawn.shape[0]].copy_(drawn, non_blocking=True)
        event.record()
        return host, event

    def _launch(self, reqs) -> _Flight:
        entries, sampled_index = [], []
        for i, req in enumerate(reqs):
            lo, hi = req.num_cached_tokens, req.num_cached_tokens + req.num_new_tokens
            last = hi == len(req)
            if last:
                sampled_index.append(i)
            entries.append(StepEntry(req.cache, req.token_ids[lo:hi], lo,
                                     [req.num_new_tokens - 1] if last else []))
        if len(sampled_index) == len(reqs):
            # every entry ends in a draw: a decode step may run, draw included, as one graph
            temps, keys = self.sampler.inputs(reqs)
            drawn = self.runner.decode_and_sample(entries, temps, keys)
            if drawn is not None:
                host, event = self._land(drawn)
                return _Flight(reqs, sampled_index, host=host, event=event,
                               positions=[e.start for e in entries],
                               draw_index=[r.num_completion_tokens for r in reqs])
        logits = self.runner.step(entries)
        tokens = self.sampler(logits, [reqs[i] for i in sampled_index])
        return _Flight(reqs, sampled_index, tokens=tokens)

    def _launch_ahead(self, prev: _Flight) -> _Flight | None:
        """The decode step after `prev`, launched before prev's tokens are known: the
        requests of prev that go on whatever prev draws, except an end of sequence, whose
        lane then computes one token that is thrown away.  None if the coming step is the
        scheduler's to decide (somebody may be admitted, pages run short) or no captured
        graph serves it."""
        sch, manager = self.scheduler, self.runner.manager
        if sch.may_admit():
            return None
        reqs, sources, positions, draw_index = [], [], [], []
        for lane, (req, pos, k) in enumerate(zip(prev.reqs, prev.positions, prev.draw_index)):
            if req.status is not RequestStatus.RUNNING:
                continue                 # ended at a step the host has seen since
            if k + 1 >= req.max_tokens or pos + 2 >= self.config.max_model_len:
                if sch.waiting:
                    return None          # its end makes room: the scheduler's step
                continue                 # ends with the token on its way, whatever it is
            reqs.append(req)
            sources.append(lane)
            positions.append(pos + 1)
            draw_index.append(k + 1)
        if not reqs:
            return None
        entries = [StepEntry(r.cache, [0], p, [0]) for r, p in zip(reqs, positions)]
        if not self.runner.fits_captured(entries):
            return None
        if not manager.can_extend_all([(r.cache, p + 1) for r, p in zip(reqs, positions)]):
            return None                  # the scheduler preempts, with everything seen
        for r, p in zip(reqs, positions):
            manager.extend(r.cache, p + 1)
        temps, keys = self.sampler.inputs(reqs, draw_index)
        drawn = self.runner.decode_and_sample(entries, temps, keys, sources)
        if drawn is None:
            raise RuntimeError("a decode step that fitted a captured graph no longer does")
        host, event = self._land(drawn)
        self.num_steps_ahead += 1
        return _Flight(reqs, list(range(len(reqs))), host=host, event=event,
                       positions=positions, draw_index=draw_index, ahead=True)

    def _finish(self, flight: _Flight):
        reqs, sampled_index, token_ids = flight.reqs, flight.sampled_index, flight.tokens
        if token_ids is None:
            flight.event.synchronize()
            token_ids = flight.host[:len(reqs)].tolist()
        if flight.ahead:
            # a request that ended with the token before this step's: its lane's token is
            # dropped (its pages went back when it ended; what this step wrote there was
            # written before anything their next owner runs)
            keep = [i for i, r in enumerate(reqs) if r.status is RequestStatus.RUNNING]
            reqs = [reqs[i] for i in keep]
            token_ids = [token_ids[i] for i in keep]
            sampled_index = list(range(len(reqs)))
            for r in reqs:
                r.num_new_tokens = 1
        self.scheduler.postprocess(reqs, token_ids, sampled_index)
        outputs = [(r.ordinal, r.completion_token_ids) for r in reqs if r.is_finished]
        num_total_tokens = sum(len(r) for r in reqs if r.is_finished)
        for r in reqs:
            if r.is_finished:
                self.requests.pop(r.ordinal, None)
        return outputs, num_total_tokens

    def generate(self, prompts, sampling_params, use_tqdm: bool = True) -> list[list[int]]:
        if not isinstance(sampling_params, list):
            sampling_params = [sampling_params] * len(prompts)
        if len(sampling_params) != len(prompts):
            raise ValueError(f"{len(prompts)} prompts but {len(sampling_params)} sampling "
                             "parameters: give one for all, or a list of equal length")
        pbar = None
        if use_tqdm:
            from tqdm.auto import tqdm
            pbar = tqdm(total=len(prompts), desc="Generating", dynamic_ncols=True)
        ordinals = [self.add_request(p, sp) for p, sp in zip(prompts, sampling_params)]
        outputs: dict[int, list[int]] = {}
        total, t0 = 0, time.perf_counter()
        while not self.is_finished():
            finished, n = self.step()
            total += n
            for ordinal, token_ids in finished:
                outputs[ordinal] = token_ids
                if pbar is not None:
                    pbar.update(1)
            if pbar is not None:
                rate = total / max(time.perf_counter() - t0, 1e-9)
                pbar.set_postfix({"total_throughput": f"{int(rate)}tok/s"})
        if pbar is not None:
            pbar.close()
        return [outputs[o] for o in ordinals]
