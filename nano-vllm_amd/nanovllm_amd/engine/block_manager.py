"""Paged KV-cache allocator with a content-addressed prefix cache.

Same policy as nanovllm/engine/block_manager.py: a FIFO free list, per-block reference
counts, and a chained xxh64 over every FULL block of 256 token ids (the hash of block i
covers the hash of block i-1 followed by the block's ids as little-endian int64, as
``compute_hash`` does at :36-41) so that two prompts sharing a prefix share physical blocks.
Blocks keep their hash after they are freed: a later prompt can revive them as long as the
block has not been handed out again.
"""
from __future__ import annotations

from collections import deque
from typing import Deque, Dict, List, Optional, Set

import numpy as np
import xxhash

from .sequence import PENDING_TOKEN, Sequence

NO_HASH = -1


class _Block:
    __slots__ = ("block_id", "ref_count", "hash", "token_ids")

    def __init__(self, block_id: int):
        self.block_id = block_id
        self.ref_count = 0
        self.hash = NO_HASH
        self.token_ids: List[int] = []


class BlockManager:

    def __init__(self, num_blocks: int, block_size: int = 256):
        self.block_size = block_size
        self.blocks = [_Block(i) for i in range(num_blocks)]
        self.hash_to_block_id: Dict[int, int] = {}
        self.free_block_ids: Deque[int] = deque(range(num_blocks))
        self.used_block_ids: Set[int] = set()

    @staticmethod
    def compute_hash(token_ids: List[int], prefix: int = NO_HASH) -> int:
        h = xxhash.xxh64()
        if prefix != NO_HASH:
            h.update(int(prefix).to_bytes(8, "little"))
        h.update(np.asarray(token_ids, dtype=np.int64).tobytes())
        return h.intdigest()

    # ---- block bookkeeping ---------------------------------------------------------------
    def _take(self, block_id: int) -> _Block:
        blk = self.blocks[block_id]
        assert blk.ref_count == 0
        blk.ref_count = 1
        blk.hash = NO_HASH
        blk.token_ids = []
        self.free_block_ids.remove(block_id)
        self.used_block_ids.add(block_id)
        return blk

    def _release(self, block_id: int) -> None:
        assert self.blocks[block_id].ref_count == 0
        self.used_block_ids.remove(block_id)
        self.free_block_ids.append(block_id)

    # ---- prefill -------------------------------------------------------------------------
    def can_allocate(self, seq: Sequence) -> bool:
        return len(self.free_block_ids) >= seq.num_blocks

    def allocate(self, seq: Sequence) -> None:
        """Give ``seq`` a block table; leading blocks whose content hash is known are shared
        and counted in ``seq.num_cached_tokens``.  After the first miss every block is fresh."""
        assert not seq.block_table
        h = NO_HASH
        missed = False
        for i in range(seq.num_blocks):
            ids = seq.block(i)
            h = self.compute_hash(ids, h) if len(ids) == self.block_size else NO_HASH
            block_id = self.hash_to_block_id.get(h, -1)
            if block_id == -1 or self.blocks[block_id].token_ids != ids:
                missed = True
            if missed:
                blk = self._take(self.free_block_ids[0])
            else:
                seq.num_cached_tokens += self.block_size
                if block_id in self.used_block_ids:
                    blk = self.blocks[block_id]
                    blk.ref_count += 1
                else:                              # freed but never reused: revive it
                    blk = self._take(block_id)
            if h != NO_HASH:
                blk.hash = h
                blk.token_ids = ids
                self.hash_to_block_id[h] = blk.block_id
            seq.block_table.append(blk.block_id)

    def deallocate(self, seq: Sequence) -> None:
        for block_id in reversed(seq.block_table):
            blk = self.blocks[block_id]
            blk.ref_count -= 1
            if blk.ref_count == 0:
                self._release(block_id)
        seq.num_cached_tokens = 0
        seq.block_table.clear()

    # ---- decode --------------------------------------------------------------------------
    def can_append(self, seq: Sequence) -> bool:
        # a new block is needed exactly when the token about to be written opens one
        return len(self.free_block_ids) >= (1 if len(seq) % self.block_size == 1 else 0)

    def may_append(self, seq: Sequence) -> None:
        table = seq.block_table
        last = self.blocks[table[-1]]
        fill = len(seq) % self.block_size
        if fill == 1:                              # previous block just became full: open a new one
            assert last.hash != NO_HASH
            table.append(self._take(self.free_block_ids[0]).block_id)
        elif fill == 0:                            # block completed by the last token: seal it
            if seq.token_ids[-1] != PENDING_TOKEN:
                self.seal(seq, seq.num_blocks - 1)
        else:
            assert last.hash == NO_HASH

    def seal(self, seq: Sequence, index: int, table: Optional[List[int]] = None) -> None:
        """Register the content hash of the full block ``index`` of ``seq`` (no-op when it is
        sealed already).  ``may_append`` does this when the block fills up; when the step loop
        runs ahead of the sampled tokens the block's last id is not known at that moment, and the
        loop seals the block once the token has been read back (``table``: the block table the
        sequence had, if it has been deallocated since)."""
        table = seq.block_table if table is None else table
        blk = self.blocks[table[index]]
        if blk.hash != NO_HASH:
            return
        ids = seq.block(index)
        assert len(ids) == self.block_size and PENDING_TOKEN not in ids[-2:]
        prefix = self.blocks[table[index - 1]].hash if index > 0 else NO_HASH
        blk.hash = self.compute_hash(ids, prefix)
        blk.token_ids = ids
        self.hash_to_block_id[blk.hash] = blk.block_id
