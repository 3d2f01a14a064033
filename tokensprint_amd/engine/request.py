"""Host state of one request (the reference's Sequence, engine/sequence.py:31-251)."""

from __future__ import annotations

from enum import Enum, auto

from tokensprint_amd.cache.pages import RequestCache
from tokensprint_amd.config.engine_config import SamplingParams


class RequestStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED = auto()


class Request:
    def __init__(self, ordinal: int, token_ids: list[int],
                 sampling_params: SamplingParams | None = None) -> None:
        if not token_ids:
            raise ValueError("token_ids must be non-empty.")
        sp = sampling_params or SamplingParams()
        self.ordinal = ordinal                 # order of arrival; also the request's id
        self.token_ids = list(token_ids)       # prompt plus completion
        self.num_prompt_tokens = len(token_ids)
        self.num_cached_tokens = 0             # tokens whose keys/values are in the cache
        self.num_new_tokens = 0                # tokens scheduled for the coming step
        self.temperature = sp.temperature
        self.max_tokens = sp.max_tokens
        self.ignore_eos = sp.ignore_eos
        self.seed = sp.seed
        self.status = RequestStatus.WAITING
        self.cache: RequestCache | None = None
        self.num_preemptions = 0

    def __len__(self) -> int:
        return len(self.token_ids)

    @property
    def seq_id(self) -> int:
        return self.ordinal

    @property
    def is_finished(self) -> bool:
        return self.status == RequestStatus.FINISHED

    @property
    def num_completion_tokens(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def completion_token_ids(self) -> list[int]:
        return self.token_ids[self.num_prompt_tokens:]

    @property
    def block_table(self) -> list[int]:
        """Pages of the first cache group (empty when the request holds nothing)."""
        return self.cache.tables[0] if self.cache is not None and self.cache.tables else []

    def append_token(self, token_id: int) -> None:
        self.token_ids.append(int(token_id))
