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
from .sequence import PENDING_TOKEN, Sequence, SequenceStatus


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

    # ---- running one step ahead of the sampled tokens ---------------------------------------------
    # ``postprocess`` needs the tokens of a step before the next one can be scheduled, which leaves
    # the GPU idle while the host reads them back and prepares the next batch.  ``advance`` +
    # ``commit`` split it in two: ``advance`` does everything that depends on lengths only (it
    # appends a PENDING_TOKEN and retires sequences that reach max_tokens), so that the next
    # decode step can be scheduled and launched at once; ``commit`` fills in the tokens when they
    # arrive, ends sequences that sampled eos (their one speculative step is dropped) and seals
    # the blocks those tokens completed.  With every step committed, the state equals what
    # ``postprocess`` leaves, except that blocks freed by an eos come back one step later.
    def advance(self, seqs: List[Sequence]) -> List[int]:
        """Returns the index in ``token_ids`` that the step's token of every sequence will take."""
        where = []
        for seq in seqs:
            where.append(len(seq))
            seq.append_token(PENDING_TOKEN)
            if seq.num_completion_tokens == seq.max_tokens:
                bs = self.block_manager.block_size
                if len(seq) >= 2 and seq.token_ids[-2] == PENDING_TOKEN and (len(seq) - 1) % bs == 0:
                    # the previous, uncommitted token completed a block: commit seals it from this copy
                    seq.late_seal = (len(seq) - 2, list(seq.block_table))
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                self.running.remove(seq)
        return where

    def commit(self, seqs: List[Sequence], where: List[int], token_ids: List[int]) -> List[Sequence]:
        """Returns the sequences whose last token this was."""
        done = []
        for seq, at, tok in zip(seqs, where, token_ids):
            if at >= len(seq):                     # dropped: the sequence ended on an earlier eos
                continue
            assert seq.token_ids[at] == PENDING_TOKEN
            seq.token_ids[at] = int(tok)
            hit_eos = (not seq.ignore_eos) and tok == self.eos
            late_seal = seq.__dict__.pop("late_seal", None) if seq.is_finished else None
            if late_seal is not None and late_seal[0] == at and not hit_eos:
                self.block_manager.seal(seq, at // self.block_manager.block_size, late_seal[1])
            if hit_eos and at + 1 < len(seq):
                del seq.token_ids[at + 1:]         # drop the step that ran past the eos
            if hit_eos and not seq.is_finished:
                if seq.status is SequenceStatus.RUNNING:
                    self.block_manager.deallocate(seq)
                    self.running.remove(seq)
                else:                              # preempted in the meantime: holds no blocks
                    self.waiting.remove(seq)
                seq.status = SequenceStatus.FINISHED
            if seq.is_finished:
                if at == len(seq) - 1:
                    done.append(seq)
            elif (at + 1) % self.block_manager.block_size == 0 and seq.block_table:
                self.block_manager.seal(seq, at // self.block_manager.block_size)
        return done
