"""Continuous batching with chunked prefill and preemption by recomputation.

The policy is the reference's (engine/generation/scheduler.py:55-214): per step a token
budget; running requests first (one decode token, or the next portion of a prompt), and
when a running request cannot get the pages it needs, requests are preempted from the
tail of the running list: their pages go back, they return to the FRONT of the waiting
queue and are later prefilled again over prompt and generated tokens; waiting requests
are admitted in arrival order only in a step without preemption.

Decided here where the reference crashes or leaves it open
(tests/test_scheduler_policy_xfail.py of the reference):
  * a lone running request that cannot grow raises `OutOfPages`, naming the request,
    instead of the generic "empty schedule";
  * a request that could never run (more pages than the pool has for prompt plus one
    token; without chunked prefill, a prompt above the token budget) is refused when it
    is added;
  * a request that recomputation has made longer than the budget still runs, alone, in
    a step of its own when prefill is not chunked.
"""

from __future__ import annotations

import logging
from collections import deque

from tokensprint_amd.cache.pages import CacheManager, OutOfPages
from tokensprint_amd.engine.request import Request, RequestStatus

log = logging.getLogger(__name__)


class Scheduler:
    def __init__(self, manager: CacheManager, *, max_num_batched_tokens: int,
                 max_num_seqs: int, max_model_len: int, eos: int = -1,
                 chunked_prefill: bool = False) -> None:
        self.manager = manager
        self.enable_chunked = chunked_prefill
        self.max_model_len = max_model_len
        self.max_num_seqs = min(max_num_seqs, manager.slots.num_slots)
        self.max_num_batched_tokens = max_num_batched_tokens
        self.eos = eos
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []
        self.num_preemptions = 0
        self.num_prefix_hit_tokens = 0

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    # ------------------------------------------------------------ admission
    def add_request(self, req: Request) -> None:
        if len(req) > self.max_model_len - 1:
            raise ValueError(
                f"a request of {len(req)} tokens is too long: with max_model_len="
                f"{self.max_model_len} at most {self.max_model_len - 1} fit before the first "
                "generated token")
        need = -(-(len(req) + 1) // self.manager.page_size)
        full = [pool.num_pages for g, pool in zip(self.manager.groups, self.manager.pools)
                if g.window is None]
        if full and need > min(full):
            raise ValueError(
                f"request of {len(req)} tokens needs {need} pages, the pool has {min(full)}")
        if not self.enable_chunked and len(req) > self.max_num_batched_tokens:
            raise ValueError(
                f"prompt of {len(req)} tokens exceeds max_num_batched_tokens="
                f"{self.max_num_batched_tokens} and chunked prefill is off")
        self.waiting.append(req)

    add_sequence = add_request

    def may_admit(self) -> bool:
        """True if the coming `schedule` could start a waiting request (pages permitting)."""
        return bool(self.waiting) and len(self.running) < self.max_num_seqs \
            and self.manager.slots.num_free > 0

    # ------------------------------------------------------------ one step
    def schedule(self) -> list[Request]:
        scheduled_running: list[Request] = []
        scheduled_new: list[Request] = []
        preempted: list[Request] = []
        budget = self.max_num_batched_tokens

        index = 0
        while index < len(self.running) and budget > 0:
            req = self.running[index]
            n = len(req) - req.num_cached_tokens
            if self.enable_chunked:
                n = min(n, budget)
            n = min(n, self.max_model_len - 1 - req.num_cached_tokens)
            if n <= 0:
                raise RuntimeError(f"request {req.ordinal}: nothing to run (n={n})")
            while not self.manager.can_extend(req.cache, req.num_cached_tokens + n):
                victim = self.running.pop()
                if victim is req and not scheduled_running and not self.running:
                    # nobody else holds pages: no preemption can help
                    self.running.append(victim)
                    raise OutOfPages(
                        f"request {req.ordinal} alone needs "
                        f"{self.manager.pages_needed(req.cache, req.num_cached_tokens + n)} "
                        f"more pages per group at {req.num_cached_tokens + n} tokens; "
                        f"free: {[p.num_free for p in self.manager.pools]}")
                self.preempt(victim)
                preempted.append(victim)
                if victim is req:
                    break
            if req.status != RequestStatus.RUNNING:
                break
            req.num_new_tokens = n
            self.manager.extend(req.cache, req.num_cached_tokens + n)
            scheduled_running.append(req)
            budget -= n
            index += 1

        if not preempted:
            while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs:
                req = self.waiting[0]
                if self.manager.slots.num_free == 0:
                    break
                # with the prefix cache on, the request starts behind its cached pages
                # (the reference's get_token_layout / allocate, scheduler.py:129-150)
                rc = self.manager.admit(req.ordinal, req.token_ids)
                cached = rc.num_tokens
                n = len(req) - cached
                if self.enable_chunked:
                    n = min(n, budget)
                # over budget: only a recomputed request, and only alone in its step
                fits_budget = n <= budget or (n > self.max_num_batched_tokens
                                              and not scheduled_running and not scheduled_new)
                if not fits_budget or not self.manager.can_extend(rc, cached + n):
                    self.manager.free(rc)
                    break
                self.num_prefix_hit_tokens += cached
                self.manager.extend(rc, cached + n)
                req.cache = rc
                req.num_cached_tokens, req.num_new_tokens = cached, n
                req.status = RequestStatus.RUNNING
                self.waiting.popleft()
                self.running.append(req)
                scheduled_new.append(req)
                budget -= n

        scheduled = scheduled_running + scheduled_new
        if not scheduled:
            if preempted:
                raise OutOfPages("every running request was preempted: the pool cannot hold "
                                 "a single request at its current length")
            raise OutOfPages(
                "nothing can be scheduled: the first waiting request needs more pages than "
                f"are free ({[p.num_free for p in self.manager.pools]}) and nothing is running")
        return scheduled

    def preempt(self, req: Request) -> None:
        req.status = RequestStatus.WAITING
        self.manager.free(req.cache)
        req.cache = None
        req.num_cached_tokens = req.num_new_tokens = 0
        req.num_preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(req)

    # ------------------------------------------------------------ after the step
    def postprocess(self, reqs: list[Request], token_ids: list[int],
                    sampled_index: list[int]) -> None:
        """`token_ids[i]` was drawn for `reqs[sampled_index[i]]`."""
        if len(token_ids) != len(sampled_index):
            raise ValueError(f"{len(token_ids)} drawn tokens for {len(sampled_index)} "
                             "requests that were to draw one")
        for req in reqs:
            req.num_cached_tokens += req.num_new_tokens
            req.num_new_tokens = 0
            # before a finished request's pages go back: they stay findable while free
            self.manager.register_full_pages(req.cache, req.token_ids, req.num_cached_tokens)
        for i, token in zip(sampled_index, token_ids):
            req = reqs[i]
            req.append_token(token)
            if ((not req.ignore_eos and token == self.eos)
                    or req.num_completion_tokens == req.max_tokens
                    or len(req) >= self.max_model_len):
                if len(req) >= self.max_model_len:
                    log.info("Request %s reached max_model_len %s.", req.ordinal,
                             self.max_model_len)
                req.status = RequestStatus.FINISHED
                self.manager.free(req.cache)
                req.cache = None
                req.num_cached_tokens = req.num_new_tokens = 0
                self.running.remove(req)
