"""One step's batch: what every kernel needs to know about the tokens it is given.

The reference flattens a step into input_ids, positions, cu_seqlens_q/k,
slot_mapping, context_lens, block_tables and seq_need_compute_logits with one Python
loop per token (engine/generation/model_runner.py:101-168, 64-99).  Here the same
facts travel as one int32 buffer copied to the device once; the cache slot of a token
is computed inside the kernels from the block table, so there is no per-token host
loop for it.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from tokensprint_amd.cache.pages import RequestCache


@dataclass
class StepEntry:
    """A request's next tokens: positions [start, start+len(tokens)), and the
    offsets among these tokens whose logits are wanted."""

    cache: RequestCache
    tokens: list[int]
    start: int
    want: list[int] = field(default_factory=list)


@dataclass
class StepBatch:
    num_tokens: int
    num_entries: int
    num_logit_rows: int
    token_ids: torch.Tensor        # int32 [T]
    positions: torch.Tensor        # int32 [T]
    entry_of_token: torch.Tensor   # int32 [T]
    q_start: torch.Tensor          # int32 [B+1]  first flat token of each entry
    ctx_len: torch.Tensor          # int32 [B]    keys of the entry after this step
    slot_ids: torch.Tensor         # int32 [B]    state slot of each entry
    logit_rows: torch.Tensor       # int32 [R]    flat token index of each wanted row
    tables: list[torch.Tensor]     # per group int32 [B, width_g], -1 = no page
    # host copies for launch planning
    q_lens: list[int]
    starts: list[int]
    max_q_len: int
    max_ctx_len: int
    plans: dict = field(default_factory=dict)   # kernels cache per-step launch plans here
    all_rows_wanted: bool = False   # logit_rows is 0..T-1: picking the wanted rows is no work


def _align(n: int, a: int = 4) -> int:
    return -(-n // a) * a


def decode_layout(bucket: int, widths: list[int]):
    """Section offsets of a decode-only batch of `bucket` entries, one token each."""
    sizes = [bucket, bucket, bucket, bucket + 1, bucket, bucket, bucket] \
        + [bucket * w for w in widths] + [bucket, 2 * bucket, bucket]   # ... temperatures, keys,
    #                                                                 lanes to take tokens from
    offs, total = [], 0
    for n in sizes:
        offs.append(total)
        total += _align(n)
    return offs, total


class StaticDecodeBatch:
    """A decode batch of fixed size in fixed device memory, for a captured graph.

    `fill` rewrites the contents for the step's entries; lanes beyond them are idle:
    token 0 at position 0 with no pages, so they write nothing to the cache
    (as the reference pads with slot -1, engine/generation/model_runner.py:253-276),
    and with state slot `idle_slot`, which no request owns.
    """

    def __init__(self, device, bucket: int, widths: list[int], idle_slot: int = 0) -> None:
        self.bucket, self.widths, self.idle_slot = bucket, widths, idle_slot
        self.offs, total = decode_layout(bucket, widths)
        self.host = torch.empty(total, dtype=torch.int32, pin_memory=True)
        self.dev = torch.zeros(total, dtype=torch.int32, device=device)
        self.copied = torch.cuda.Event()
        o, B = self.offs, bucket
        d = self.dev
        self.batch = StepBatch(
            num_tokens=B, num_entries=B, num_logit_rows=B,
            token_ids=d[o[0]:o[0] + B], positions=d[o[1]:o[1] + B],
            entry_of_token=d[o[2]:o[2] + B], q_start=d[o[3]:o[3] + B + 1],
            ctx_len=d[o[4]:o[4] + B], slot_ids=d[o[5]:o[5] + B], logit_rows=d[o[6]:o[6] + B],
            tables=[d[o[7 + g]:o[7 + g] + B * w].view(B, w) for g, w in enumerate(widths)],
            q_lens=[1] * B, starts=[0] * B, max_q_len=1, max_ctx_len=0,
            all_rows_wanted=True)
        h = self.host.numpy()
        h[:] = 0
        h[o[2]:o[2] + B] = np.arange(B)
        h[o[3]:o[3] + B + 1] = np.arange(B + 1)
        h[o[6]:o[6] + B] = np.arange(B)
        for g, w in enumerate(widths):
            h[o[7 + g]:o[7 + g] + B * w] = -1
        # what each lane's block-table rows hold: (request cache, pages written) per group
        self._lane = [[(None, 0)] * len(widths) for _ in range(B)]
        G = len(widths)
        # sampling inputs ride in the same buffer: float32 temperatures, int64 noise keys
        self.temperatures = d[o[7 + G]:o[7 + G] + B].view(torch.float32)
        self.keys = d[o[8 + G]:o[8 + G] + 2 * B].view(torch.int64)
        self._h_temps = h[o[7 + G]:o[7 + G] + B].view(np.float32)
        self._h_keys = h[o[8 + G]:o[8 + G] + 2 * B].view(np.int64)
        # lane of the previous step's draw that holds this lane's token; -1: the token
        # given by the host
        self.token_sources = d[o[9 + G]:o[9 + G] + B]
        self._h_sources = h[o[9 + G]:o[9 + G] + B]
        self._h_sources[:] = -1

    def fill(self, entries, temperatures=None, keys=None, sources=None) -> None:
        """`sources[i]`: the lane of the step before whose drawn token is entry i's token
        (its `tokens[0]` is then a placeholder), or -1."""
        o, B, n = self.offs, self.bucket, len(entries)
        if n > B:
            raise ValueError(f"{n} entries for a static batch of {B} lanes")
        if sources is not None and len(sources) != n:
            raise ValueError("one source lane per entry")
        for e in entries:
            for t, w in zip(e.cache.tables, self.widths):
                if len(t) > w:
                    raise ValueError(
                        f"request {e.cache.request_id!r}: block table of {len(t)} pages "
                        f"is wider than the static batch's {w}")
        self.copied.synchronize()          # the last copy out of the pinned buffer is done
        h = self.host.numpy()
        h[o[0] + n:o[0] + B] = 0
        h[o[1] + n:o[1] + B] = 0
        h[o[4] + n:o[4] + B] = 1
        h[o[5] + n:o[5] + B] = self.idle_slot
        starts = [e.start for e in entries]
        h[o[0]:o[0] + n] = [e.tokens[0] for e in entries]
        h[o[1]:o[1] + n] = starts
        h[o[4]:o[4] + n] = np.asarray(starts, dtype=np.int32) + 1
        h[o[5]:o[5] + n] = [e.cache.slot for e in entries]
        for g, w in enumerate(self.widths):
            base = o[7 + g]
            for i in range(B):
                rid, have = self._lane[i][g]
                if i >= n:                               # idle lane: no pages
                    if have or rid is not None:
                        h[base + i * w:base + i * w + have] = -1
                        self._lane[i][g] = (None, 0)
                    continue
                rc = entries[i].cache
                t = rc.tables[g]
                # same request as last step and nothing given back: only new pages to add
                if rid is rc and have <= len(t) and rc.released[g] == 0:
                    if have < len(t):
                        h[base + i * w + have:base + i * w + len(t)] = t[have:]
                else:
                    h[base + i * w:base + i * w + max(have, len(t))] = -1
                    h[base + i * w:base + i * w + len(t)] = t
                self._lane[i][g] = (rc, len(t))
        self._h_sources[:] = -1
        if sources is not None:
            self._h_sources[:n] = sources
        self._h_temps[:] = 0.0
        self._h_keys[:] = 0
        if temperatures is not None:
            self._h_temps[:n] = temperatures
            self._h_keys[:n] = keys
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()


class BatchBuilder:
    """Packs a step's description into one pinned buffer and one device copy."""

    def __init__(self, device, num_groups: int, vocab_size: int | None = None,
                 max_position: int | None = None) -> None:
        self.device = torch.device(device)
        self.num_groups = num_groups
        self.vocab_size = vocab_size
        self.max_position = max_position
        self._pinned = None
        self._copied = None

    def _host_buffer(self, n: int) -> torch.Tensor:
        if self.device.type != "cuda":
            return torch.empty(n, dtype=torch.int32)
        if self._pinned is None or self._pinned.numel() < n:
            self._pinned = torch.empty(max(n, 1 << 16), dtype=torch.int32, pin_memory=True)
            self._copied = torch.cuda.Event()
        else:
            self._copied.synchronize()     # the last copy out of the pinned buffer is done
        return self._pinned[:n]

    def build(self, entries: list[StepEntry], table_width: list[int] | None = None) -> StepBatch:
        if not entries:
            raise ValueError("a step needs at least one entry")
        B = len(entries)
        q_lens = [len(e.tokens) for e in entries]
        starts = [e.start for e in entries]
        if min(q_lens) < 1:
            raise ValueError("every entry of a step brings at least one token")
        T = sum(q_lens)
        for e, n in zip(entries, q_lens):
            if e.start < 0 or e.start + n > e.cache.num_tokens:
                raise ValueError(
                    f"request {e.cache.request_id!r}: tokens at [{e.start}, {e.start + n}) "
                    f"but its cache covers {e.cache.num_tokens} positions")
            if self.max_position is not None and e.start + n > self.max_position:
                raise ValueError(
                    f"request {e.cache.request_id!r}: position {e.start + n - 1} is beyond "
                    f"the model's {self.max_position} positions")
            if any(not 0 <= w < n for w in e.want):
                raise ValueError(f"request {e.cache.request_id!r}: wanted offsets {e.want} "
                                 f"outside its {n} tokens")
        R = sum(len(e.want) for e in entries)
        widths = []
        for g in range(self.num_groups):
            w = max(len(e.cache.tables[g]) for e in entries)
            if table_width is not None:
                if w > table_width[g]:
                    raise ValueError("block table wider than the fixed width")
                w = table_width[g]
            widths.append(max(w, 1))

        # layout of the one buffer (every section 16-byte aligned)
        sizes = [T, T, T, B + 1, B, B, max(R, 1)] + [B * w for w in widths]
        offs, total = [], 0
        for s in sizes:
            offs.append(total)
            total += _align(s)
        host = self._host_buffer(total)
        buf = host.numpy()

        ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries])
        if ids.min() < 0 or (self.vocab_size is not None and ids.max() >= self.vocab_size):
            raise ValueError(f"token id outside [0, {self.vocab_size})")
        buf[offs[0]:offs[0] + T] = ids
        qs = np.zeros(B + 1, dtype=np.int64)
        np.cumsum(q_lens, out=qs[1:])
        buf[offs[1]:offs[1] + T] = np.concatenate(
            [np.arange(s, s + n) for s, n in zip(starts, q_lens)])
        buf[offs[2]:offs[2] + T] = np.repeat(np.arange(B), q_lens)
        buf[offs[3]:offs[3] + B + 1] = qs
        buf[offs[4]:offs[4] + B] = [s + n for s, n in zip(starts, q_lens)]
        buf[offs[5]:offs[5] + B] = [e.cache.slot for e in entries]
        rows = [int(qs[i]) + w for i, e in enumerate(entries) for w in e.want]
        buf[offs[6]:offs[6] + R] = rows
        for g, w in enumerate(widths):
            tab = np.full((B, w), -1, dtype=np.int32)
            for i, e in enumerate(entries):
                t = e.cache.tables[g]
                tab[i, :len(t)] = t
            buf[offs[7 + g]:offs[7 + g] + B * w] = tab.reshape(-1)

        if self.device.type == "cuda":
            dev = host.to(self.device, non_blocking=True)
            self._copied.record()
        else:
            dev = host.clone()

        def sec(i, n):
            return dev[offs[i]:offs[i] + n]

        return StepBatch(
            num_tokens=T, num_entries=B, num_logit_rows=R,
            token_ids=sec(0, T), positions=sec(1, T), entry_of_token=sec(2, T),
            q_start=sec(3, B + 1), ctx_len=sec(4, B), slot_ids=sec(5, B),
            logit_rows=sec(6, R),
            tables=[sec(7 + g, B * w).view(B, w) for g, w in enumerate(widths)],
            q_lens=q_lens, starts=starts, max_q_len=max(q_lens),
            max_ctx_len=max(s + n for s, n in zip(starts, q_lens)),
            all_rows_wanted=R == T and all(e.want == list(range(len(e.tokens)))
                                           for e in entries),
        )
