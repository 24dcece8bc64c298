"""Per-request state: token ids, KV block table and block arithmetic.

Mirrors the bookkeeping of nanovllm/engine/sequence.py (block_size 256 class attribute,
``num_cached_tokens`` for prefix hits, ``last_block_num_tokens``).  There is no pickling:
the reference serialises sequences for its tensor-parallel worker processes only.
"""
from __future__ import annotations

import enum
import itertools
from typing import List

from .sampling_params import SamplingParams


PENDING_TOKEN = -1          # stands in token_ids for a token that is sampled but not yet read back


class SequenceStatus(enum.Enum):
    WAITING = enum.auto()
    RUNNING = enum.auto()
    FINISHED = enum.auto()


class Sequence:
    block_size = 256
    _ids = itertools.count()

    def __init__(self, token_ids: List[int], sampling_params: SamplingParams = SamplingParams()):
        assert len(token_ids) > 0, "empty prompt"
        self.seq_id = next(Sequence._ids)
        self.status = SequenceStatus.WAITING
        self.token_ids = list(token_ids)
        self.num_prompt_tokens = len(self.token_ids)
        self.num_cached_tokens = 0                 # leading tokens whose KV is already in the cache
        self.block_table: List[int] = []
        self.temperature = sampling_params.temperature
        self.max_tokens = sampling_params.max_tokens
        self.ignore_eos = sampling_params.ignore_eos

    def __len__(self) -> int:
        return len(self.token_ids)

    def __getitem__(self, key):
        return self.token_ids[key]

    @property
    def num_tokens(self) -> int:
        return len(self.token_ids)

    @property
    def last_token(self) -> int:
        return self.token_ids[-1]

    @property
    def is_finished(self) -> bool:
        return self.status is SequenceStatus.FINISHED

    @property
    def num_completion_tokens(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def prompt_token_ids(self) -> List[int]:
        return self.token_ids[: self.num_prompt_tokens]

    @property
    def completion_token_ids(self) -> List[int]:
        return self.token_ids[self.num_prompt_tokens:]

    @property
    def num_cached_blocks(self) -> int:
        return self.num_cached_tokens // self.block_size

    @property
    def num_blocks(self) -> int:
        return -(-len(self.token_ids) // self.block_size)

    @property
    def last_block_num_tokens(self) -> int:
        return len(self.token_ids) - (self.num_blocks - 1) * self.block_size

    def block(self, i: int) -> List[int]:
        assert 0 <= i < self.num_blocks
        return self.token_ids[i * self.block_size: (i + 1) * self.block_size]

    def append_token(self, token_id: int) -> None:
        self.token_ids.append(int(token_id))
