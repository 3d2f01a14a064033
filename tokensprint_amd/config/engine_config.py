"""Engine knobs and per-request sampling parameters.

Names and meanings follow the reference's engine/generation/config.py:7-55.  Two
deliberate differences: temperature 0 means greedy argmax (the reference raises,
config.py:14-15), and the page size is free (the reference's multiple-of-256 rule,
config.py:38-42, only serves its external attention library).
"""

from __future__ import annotations

import os
from dataclasses import dataclass

import torch


@dataclass
class SamplingParams:
    temperature: float = 1.0
    max_tokens: int = 64
    ignore_eos: bool = False
    seed: int = 0

    def __post_init__(self) -> None:
        if self.temperature < 0.0:
            raise ValueError(f"temperature must be >= 0, got {self.temperature}")
        if self.max_tokens < 1:
            raise ValueError(f"max_tokens must be >= 1, got {self.max_tokens}")

    @property
    def greedy(self) -> bool:
        return self.temperature <= 1e-10


@dataclass
class Config:
    model: str
    max_num_batched_tokens: int = 16384
    max_num_seqs: int = 512
    max_model_len: int = 4096
    gpu_memory_utilization: float = 0.9
    enforce_eager: bool = False
    eos: int = -1
    kvcache_block_size: int = 16
    num_kvcache_blocks: int = -1          # -1: sized from free device memory
    chunked_prefill: bool = False
    dtype: torch.dtype = torch.bfloat16
    seed: int = 0
    enable_prefix_caching: bool = False   # share cached full pages between equal prefixes
    warmup: bool = True                   # largest dummy step and graph capture at construction
    decode_ahead: bool = True             # launch a decode step before the last one's tokens are read
    fold_merge: bool = True               # a decode step's attention merges its key splits itself
                                          # (False: a merge kernel of its own after it)

    def __post_init__(self) -> None:
        if not os.path.isdir(self.model):
            raise FileNotFoundError(f"Model directory does not exist: {self.model}")
        if self.kvcache_block_size < 1:
            raise ValueError(f"kvcache_block_size must be >= 1, got {self.kvcache_block_size}")
        if self.max_num_batched_tokens < 1 or self.max_num_seqs < 1 or self.max_model_len < 2:
            raise ValueError("max_num_batched_tokens, max_num_seqs must be >= 1 and "
                             "max_model_len >= 2")
        if self.dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype must be torch.bfloat16 or torch.float32, got {self.dtype}")
        if not 0.0 < self.gpu_memory_utilization <= 1.0:
            raise ValueError("gpu_memory_utilization must be in (0, 1]")
