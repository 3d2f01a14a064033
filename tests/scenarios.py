"""Small paged-cache scenarios for kernel tests: entries with scattered pages."""

from __future__ import annotations

import torch

from tokensprint_amd.cache import CacheManager, CacheStorage
from tokensprint_amd.engine.batch import BatchBuilder, StepEntry
from tokensprint_amd.parts.base import PagedKVNeed


def paged_scenario(device, dtype, *, nkv, hd, page_size, spans, window=None, seed=0,
                   num_pages=None, fill=True):
    """`spans`: list of (start, q_len): each entry has `start` cached positions and
    `q_len` new tokens.  Pages are handed out in a scrambled order so that logical and
    physical order differ.  Returns (batch, cache view, table, manager)."""
    g = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-(s + n) // page_size) for s, n in spans)
    num_pages = num_pages or total_pages + 3
    storage = CacheStorage([PagedKVNeed(nkv, hd, window)], page_size, num_pages,
                           len(spans), dtype, device)
    manager = CacheManager(storage.groups, page_size, num_pages, len(spans))
    # scramble the free list
    order = torch.randperm(num_pages, generator=g).tolist()
    manager.pools[0].free = type(manager.pools[0].free)((i, None) for i in order)
    entries = []
    # interleave allocation so that pages of different requests interleave too
    caches = [manager.admit(i) for i in range(len(spans))]
    grown = True
    step = 0
    while grown:
        grown = False
        step += page_size
        for rc, (s, n) in zip(caches, spans):
            target = min(s + n, step)
            if target > rc.num_tokens:
                # do not let the window release pages while building the scenario
                total = -(-target // page_size)
                while len(rc.tables[0]) < total:
                    rc.tables[0].append(manager.pools[0].take())
                rc.num_tokens = target
                grown = True
    for rc, (s, n) in zip(caches, spans):
        tokens = torch.randint(0, 100, (n,), generator=g).tolist()
        entries.append(StepEntry(rc, tokens, s, [n - 1]))
    batch = BatchBuilder(device, 1).build(entries)
    cache = storage.views[0]
    if fill:
        cache.k_pages.copy_(torch.randn(cache.k_pages.shape, generator=g).to(dtype))
        cache.v_pages.copy_(torch.randn(cache.v_pages.shape, generator=g).to(dtype))
    return batch, cache, batch.tables[0], manager
