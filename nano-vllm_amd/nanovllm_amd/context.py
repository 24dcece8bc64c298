"""Per-step side channel between the model runner and the attention layers.

Same contract as nanovllm/utils/context.py:5-27: a module-global record that the runner
replaces before each forward pass (``set_context``), the attention layers and the LM head
read (``get_context``) and the runner clears afterwards (``reset_context``).  Field names,
defaults and the positional order of ``set_context`` are the reference's
(nanovllm/engine/model_runner.py:160 passes eight positionals).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch


class DecodePlan:
    """Marks the decode-attention calls that share one work split: the layers of one decode
    step, which see the same ``context_lens`` and ``block_tables``.  The first call made with
    a plan derives the split, the later ones take it from the workspace.

    A runner may put a fresh plan on the context for every forward pass itself.  If it does not,
    the attention layer keeps one on the ``Context`` object it is handed: all layers of a forward
    pass see the same object, and the runner installs a new one for every step (``set_context``
    replaces the context wholesale, nanovllm/utils/context.py:21-23).  A plan made outside graph
    capture is never used inside one and vice versa (``capturing``): the reference warms a batch
    size up and captures it under one ``Context`` (nanovllm/engine/model_runner.py:229-237), and a
    captured layer must not rely on a split that only the warm-up run derived.
    """
    __slots__ = ("key", "capturing")

    def __init__(self, capturing: bool = False):
        self.key = None        # (workspace address, batch, heads, kv heads) of the call that built it
        self.capturing = capturing


@dataclass
class Context:
    """Tensors describing the batch being run.  Index tensors are int32 on the device.

    prefill: cu_seqlens_q/k ``[B+1]``, max_seqlen_q/k, slot_mapping ``[total_q]`` and, only
             when some sequence reads cached prefix blocks, block_tables ``[B, max_blocks]``.
    decode:  slot_mapping ``[B]``, context_lens ``[B]``, block_tables ``[B, max_blocks]``.
    """
    is_prefill: bool = False
    cu_seqlens_q: Optional[torch.Tensor] = None
    cu_seqlens_k: Optional[torch.Tensor] = None
    max_seqlen_q: int = 0
    max_seqlen_k: int = 0
    slot_mapping: Optional[torch.Tensor] = None
    context_lens: Optional[torch.Tensor] = None
    block_tables: Optional[torch.Tensor] = None
    decode_plan: Optional[DecodePlan] = None     # not in the reference: see DecodePlan


class _Holder:
    current = Context()


def get_context() -> Context:
    return _Holder.current


def set_context(is_prefill, cu_seqlens_q=None, cu_seqlens_k=None, max_seqlen_q=0, max_seqlen_k=0,
                slot_mapping=None, context_lens=None, block_tables=None, decode_plan=None) -> None:
    _Holder.current = Context(is_prefill, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                              slot_mapping, context_lens, block_tables, decode_plan)


def reset_context() -> None:
    _Holder.current = Context()
