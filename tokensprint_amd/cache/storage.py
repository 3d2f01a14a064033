"""Device memory behind the cache manager, and the grouping of runs.

The reference allocates per layer [2, num_blocks, P, nkv, hd]
(engine/generation/model_runner.py:420-437).  Here each group of runs has one
pair of tensors: keys [runs, num_pages, nkv, P, hd] and values, transposed inside a
page, [runs, num_pages, nkv, hd, P].  One key/value head's part of a page is contiguous
in both; keys are contiguous along the head size (the reduction of q.k) and values along
the positions (the reduction of p.v), which is what the matrix-core kernels read without
a transpose.  A run's view is `LayerCache`.
Per-request state of fixed size lives in [num_slots + 1, *shape] tensors, one per run
that asks for it; the last row (`idle_slot`) belongs to no request: the idle lanes of a
captured decode batch point there, so whatever a part writes for them lands nowhere.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from tokensprint_amd.cache.pages import GroupLayout
from tokensprint_amd.parts.base import PagedKVNeed, SlotStateNeed


def group_runs(needs) -> tuple[list[GroupLayout], dict[int, int]]:
    """Group the runs that own a paged cache by (kv heads, head size, window)."""
    keyed: dict[tuple, list[int]] = {}
    for r, need in enumerate(needs):
        if isinstance(need, PagedKVNeed):
            keyed.setdefault((need.num_kv_heads, need.head_dim, need.window), []).append(r)
    groups, group_of_run = [], {}
    for g, (key, runs) in enumerate(keyed.items()):
        groups.append(GroupLayout(key[0], key[1], key[2], tuple(runs)))
        for r in runs:
            group_of_run[r] = g
    return groups, group_of_run


def page_bytes(groups: list[GroupLayout], page_size: int, dtype: torch.dtype) -> int:
    """Bytes one page id costs summed over all groups (each group has its own pool)."""
    item = torch.empty((), dtype=dtype).element_size()
    return sum(len(g.runs) * 2 * g.num_kv_heads * page_size * g.head_dim * item for g in groups)


@dataclass
class LayerCache:
    """The cache of one run, as a mixer sees it."""

    group: int                     # index into the batch's block tables
    page_size: int
    num_pages: int
    k_pages: torch.Tensor | None   # [num_pages, nkv, P, hd]
    v_pages: torch.Tensor | None   # [num_pages, nkv, hd, P]
    state: torch.Tensor | None = None   # [num_slots + 1, *shape] for fixed-size state


class CacheStorage:
    def __init__(self, needs, page_size: int, num_pages, num_slots: int,
                 dtype: torch.dtype, device) -> None:
        self.groups, group_of_run = group_runs(needs)
        counts = [num_pages] * len(self.groups) if isinstance(num_pages, int) else list(num_pages)
        self.page_size, self.num_pages, self.num_slots = page_size, counts, num_slots
        self.k_tensors, self.v_tensors = [], []
        for g, n in zip(self.groups, counts):
            self.k_tensors.append(torch.zeros(
                len(g.runs), n, g.num_kv_heads, page_size, g.head_dim, dtype=dtype, device=device))
            self.v_tensors.append(torch.zeros(
                len(g.runs), n, g.num_kv_heads, g.head_dim, page_size, dtype=dtype, device=device))
        self.idle_slot = num_slots
        self.state_runs = tuple(r for r, need in enumerate(needs)
                                if isinstance(need, SlotStateNeed))
        self.views: list[LayerCache | None] = []
        for r, need in enumerate(needs):
            if isinstance(need, PagedKVNeed):
                g = group_of_run[r]
                i = self.groups[g].runs.index(r)
                self.views.append(LayerCache(g, page_size, counts[g], self.k_tensors[g][i],
                                             self.v_tensors[g][i]))
            elif isinstance(need, SlotStateNeed):
                state = torch.zeros(num_slots + 1, *need.shape, dtype=need.dtype, device=device)
                self.views.append(LayerCache(-1, page_size, 0, None, None, state))
            else:
                self.views.append(None)
