"""Prefill-first batching with preemption by recompute (policy of nanovllm/engine/scheduler.py).

``schedule`` admits waiting sequences while the token budget, the sequence budget and the
free KV blocks allow and returns them as one prefill batch; only when nothing can be
admitted does it return a decode batch of the running sequences, preempting from the back
of the queue when a sequence needs a block and none is free.
"""
from __future__ import annotations

from collections import deque
from typing import Deque, List, Tuple

from .block_manager import BlockManager
from .config import EngineConfig
from .sequence import Sequence, SequenceStatus


class Scheduler:

    def __init__(self, config: EngineConfig):
        self.max_num_seqs = config.max_num_seqs
        self.max_num_batched_tokens = config.max_num_batched_tokens
        self.eos = config.eos
        self.block_manager = BlockManager(config.num_kvcache_blocks, config.kvcache_block_size)
        self.waiting: Deque[Sequence] = deque()
        self.running: Deque[Sequence] = deque()

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    def add(self, seq: Sequence) -> None:
        self.waiting.append(seq)

    def schedule(self) -> Tuple[List[Sequence], bool]:
        batch: List[Sequence] = []
        tokens = 0
        while self.waiting and len(batch) < self.max_num_seqs:
            seq = self.waiting[0]
            if tokens + len(seq) > self.max_num_batched_tokens or not self.block_manager.can_allocate(seq):
                break
            self.block_manager.allocate(seq)
            tokens += len(seq) - seq.num_cached_tokens
            seq.status = SequenceStatus.RUNNING
            self.waiting.popleft()
            self.running.append(seq)
            batch.append(seq)
        if batch:
            return batch, True

        while self.running and len(batch) < self.max_num_seqs:
            seq = self.running.popleft()
            evicted_self = False
            while not self.block_manager.can_append(seq):
                if self.running:
                    self.preempt(self.running.pop())
                else:
                    self.preempt(seq)
                    evicted_self = True
                    break
            if not evicted_self:
                self.block_manager.may_append(seq)
                batch.append(seq)
        assert batch, "nothing schedulable: the KV cache is too small for a single sequence"
        self.running.extendleft(reversed(batch))
        return batch, False

    def preempt(self, seq: Sequence) -> None:
        seq.status = SequenceStatus.WAITING
        self.block_manager.deallocate(seq)
        self.waiting.appendleft(seq)

    def postprocess(self, seqs: List[Sequence], token_ids: List[int]) -> None:
        for seq, tok in zip(seqs, token_ids):
            seq.append_token(tok)
            hit_eos = (not seq.ignore_eos) and tok == self.eos
            if hit_eos or seq.num_completion_tokens == seq.max_tokens:
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                self.running.remove(seq)
