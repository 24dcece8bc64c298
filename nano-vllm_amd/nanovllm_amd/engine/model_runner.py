"""Builds the per-step device tensors, owns the KV cache and the decode graphs, runs the model.

Single-GPU counterpart of nanovllm/engine/model_runner.py: ``prepare_prefill`` /
``prepare_decode`` reproduce the reference's input layouts (:126-179), ``allocate_kv_cache``
its cache layout ``[2, layers, num_blocks, 256, Hkv, Dh]`` (:100-117) and ``capture_graphs``
its static-buffer graph replay per batch-size bucket (:215-250).  Host tensors are built
with numpy into pinned staging buffers instead of Python lists.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np
import torch

from .. import _lib
from ..context import DecodePlan, get_context, reset_context, set_context
from ..sampler import Sampler
from .config import EngineConfig
from .model import Qwen3ForCausalLM
from .sequence import PENDING_TOKEN, Sequence


_capture_anchor: list = []       # see ModelRunner.__init__


@dataclass
class DecodeHandle:
    """A decode step that has been enqueued but whose tokens have not been read back."""
    seqs: List[Sequence]
    row_of: Dict[int, int]                # seq_id -> row of the step's batch
    tokens_dev: torch.Tensor              # int64 [len(seqs)], the sampler's output
    tokens_host: torch.Tensor             # pinned copy, valid once ``ready`` has completed
    ready: torch.cuda.Event

    def tokens(self) -> List[int]:
        self.ready.synchronize()
        return self.tokens_host[: len(self.seqs)].tolist()


def build_block_tables(seqs: List[Sequence]) -> np.ndarray:
    """``[len(seqs), widest table]`` int32, rows padded with -1 (model_runner.py:119-124)."""
    width = max(len(s.block_table) for s in seqs)
    table = np.full((len(seqs), width), -1, dtype=np.int32)
    for i, s in enumerate(seqs):
        table[i, : len(s.block_table)] = s.block_table
    return table


def build_prefill_inputs(seqs: List[Sequence], block_size: int) -> dict:
    """Host-side inputs of a prefill step (nanovllm/engine/model_runner.py:126-160).

    Only the uncached tail ``[num_cached_tokens, len)`` of every sequence is run: those are
    the input ids, positions and query lengths; key lengths are the full lengths.  The slot
    of position p is ``block_table[p // bs] * bs + p % bs``.  ``block_tables`` is present only
    when some sequence has cached tokens.
    """
    ids, pos, slots = [], [], []
    cu_q, cu_k = [0], [0]
    max_q = max_k = 0
    for s in seqs:
        n, cached = len(s), s.num_cached_tokens
        ids.append(np.asarray(s.token_ids[cached:], dtype=np.int64))
        p = np.arange(cached, n, dtype=np.int64)
        pos.append(p)
        cu_q.append(cu_q[-1] + n - cached)
        cu_k.append(cu_k[-1] + n)
        max_q, max_k = max(max_q, n - cached), max(max_k, n)
        if s.block_table:                                         # empty during warm-up
            table = np.asarray(s.block_table, dtype=np.int64)
            slots.append(table[p // block_size] * block_size + p % block_size)
    return dict(
        input_ids=np.concatenate(ids), positions=np.concatenate(pos),
        cu_seqlens_q=np.asarray(cu_q, dtype=np.int32), cu_seqlens_k=np.asarray(cu_k, dtype=np.int32),
        max_seqlen_q=max_q, max_seqlen_k=max_k,
        slot_mapping=(np.concatenate(slots) if slots else np.empty(0, np.int64)).astype(np.int32),
        block_tables=build_block_tables(seqs) if cu_k[-1] > cu_q[-1] else None)


def build_decode_inputs(seqs: List[Sequence], block_size: int) -> dict:
    """Host-side inputs of a decode step (nanovllm/engine/model_runner.py:162-179): the last
    token of every sequence at position len-1, written to the last block of its table."""
    n = len(seqs)
    ids = np.fromiter((s.token_ids[-1] for s in seqs), dtype=np.int64, count=n)
    lens = np.fromiter((len(s.token_ids) for s in seqs), dtype=np.int64, count=n)
    last_blk = np.fromiter((s.block_table[-1] for s in seqs), dtype=np.int64, count=n)
    return dict(input_ids=ids, positions=lens - 1, context_lens=lens.astype(np.int32),
                slot_mapping=(last_blk * block_size + (lens - 1) % block_size).astype(np.int32),
                block_tables=build_block_tables(seqs))


class ModelRunner:

    def __init__(self, config: EngineConfig, device: str = "cuda:0"):
        self.config = config
        self.cfg = config.hf_config
        self.block_size = config.kvcache_block_size
        self.enforce_eager = config.enforce_eager
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        prev = torch.get_default_dtype()
        torch.set_default_dtype(torch.bfloat16)
        try:
            with torch.device(self.device):
                self.model = Qwen3ForCausalLM(self.cfg, config.max_model_len, self.device, config.seed)
        finally:
            torch.set_default_dtype(prev)
        self.model.eval()
        self.sampler = Sampler(seed=config.seed)
        self.max_table_width = -(-config.max_model_len // self.block_size)
        self.graphs = {}
        self.graph_bs: List[int] = []
        self.bucket_rows = [0, 0]                        # decode rows used / rows replayed (bucket padding), since start
        self.kv_tokens_attended = 0                      # sum of context lengths over all decode steps, since start
        self.decode_step_events = None                   # a list: (start, end) HIP events of every decode step are appended
        self.graph_segments = 4                          # consecutive graphs per decode step (see capture_graphs)
        self._graph_keepalive = []
        if not self.enforce_eager and not torch.is_inference_mode_enabled() and not _capture_anchor:
            # torch allocates the default generator's graph bookkeeping tensors when the first live graph
            # registers and updates them in place at every later capture: allocated under inference mode
            # (where the decode graphs are captured) they would make every capture outside it fail for
            # as long as those graphs live.  One small graph captured here and kept for the life of the
            # process pins them as ordinary tensors.
            probe, one = torch.cuda.CUDAGraph(), torch.ones(1, device=self.device)
            with torch.cuda.graph(probe):
                one = one + 1
            _capture_anchor.append((probe, one))
        with torch.inference_mode():
            self.warmup_model()
            self.allocate_kv_cache()
            if not self.enforce_eager:
                self.capture_graphs()

    # ---- set-up ------------------------------------------------------------------------------
    def warmup_model(self) -> None:
        """One prefill of the largest admissible batch, cache not yet allocated: the attention
        layers skip the scatter and run packed (non-paged) prefill, which is also what sizes the
        activation peak used to carve the KV cache out of free memory."""
        torch.cuda.empty_cache()
        torch.cuda.reset_peak_memory_stats()
        cfg = self.config
        num_seqs = max(1, min(cfg.max_num_batched_tokens // cfg.max_model_len, cfg.max_num_seqs))
        seqs = [Sequence([0] * cfg.max_model_len) for _ in range(num_seqs)]
        self.run(seqs, True)
        torch.cuda.empty_cache()

    def allocate_kv_cache(self) -> None:
        cfg, m = self.config, self.cfg
        block_bytes = 2 * m.num_hidden_layers * self.block_size * m.num_key_value_heads * m.head_dim * 2
        if cfg.num_kvcache_blocks <= 0:
            free, total = torch.cuda.mem_get_info()
            stats = torch.cuda.memory_stats()
            peak, current = stats["allocated_bytes.all.peak"], stats["allocated_bytes.all.current"]
            budget = int(total * cfg.gpu_memory_utilization) - (total - free) - peak + current
            cfg.num_kvcache_blocks = budget // block_bytes
        assert cfg.num_kvcache_blocks > 0, "no memory left for the KV cache"
        self.kv_cache = torch.empty(2, m.num_hidden_layers, cfg.num_kvcache_blocks, self.block_size,
                                    m.num_key_value_heads, m.head_dim, dtype=torch.bfloat16, device=self.device)
        layer_id = 0
        for module in self.model.modules():
            if hasattr(module, "k_cache") and hasattr(module, "v_cache"):
                module.k_cache = self.kv_cache[0, layer_id]
                module.v_cache = self.kv_cache[1, layer_id]
                layer_id += 1
        assert layer_id == m.num_hidden_layers

    # ---- host -> device inputs -----------------------------------------------------------------
    def _to_device(self, array: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
        t = torch.from_numpy(np.ascontiguousarray(array)).to(dtype)
        return t.pin_memory().to(self.device, non_blocking=True)

    def prepare_block_tables(self, seqs: List[Sequence]) -> torch.Tensor:
        return self._to_device(build_block_tables(seqs), torch.int32)

    def _init_prefill_staging(self) -> None:
        """Pinned host buffers (two, used in turn) and one device buffer for everything a prefill step
        needs on the device: the step's arrays are packed one after the other and cross PCIe in a
        single kernel (the reference issues one pinned copy per tensor, nanovllm/engine/
        model_runner.py:155-159,184)."""
        cfg = self.config
        tokens, seqs = cfg.max_num_batched_tokens, cfg.max_num_seqs
        total = tokens * (8 + 8 + 4) + 2 * (seqs + 1) * 4 + seqs * self.max_table_width * 4 + seqs * 4 + 8 * 256
        self._pf_host = [torch.zeros(total, dtype=torch.uint8).pin_memory() for _ in range(2)]
        self._pf_dev = torch.zeros(total, dtype=torch.uint8, device=self.device)
        self._pf_turn = 0

    def _stage_prefill(self, fields):
        """``fields``: list of (numpy array, torch dtype).  Packs them (256-byte aligned) into a pinned
        buffer, copies the used part to the device with one kernel and returns device views."""
        if not hasattr(self, "_pf_host"):
            self._init_prefill_staging()
        self._pf_turn ^= 1
        host = self._pf_host[self._pf_turn].numpy()
        at, views = 0, []
        for array, dtype in fields:
            if array is None:
                views.append(None)
                continue
            raw = np.ascontiguousarray(array).view(np.uint8).reshape(-1)
            if at + raw.size > host.size:
                raise RuntimeError("prefill step exceeds max_num_batched_tokens / max_num_seqs")
            host[at: at + raw.size] = raw
            views.append(self._pf_dev[at: at + raw.size].view(dtype).view(array.shape))
            at += (raw.size + 255) // 256 * 256
        rc = _lib.load().nva_stage_decode_inputs(self._pf_dev.data_ptr(), self._pf_host[self._pf_turn].data_ptr(), at,
                                                 0, 0, 0, None, 0, torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "nva_stage_decode_inputs")
        return views

    def prepare_prefill(self, seqs: List[Sequence]):
        h = build_prefill_inputs(seqs, self.block_size)
        ids, pos, cu_q, cu_k, slots, tables, self._pf_temperatures = self._stage_prefill([
            (h["input_ids"], torch.int64), (h["positions"], torch.int64), (h["cu_seqlens_q"], torch.int32),
            (h["cu_seqlens_k"], torch.int32), (h["slot_mapping"], torch.int32), (h["block_tables"], torch.int32),
            (np.fromiter((s.temperature for s in seqs), dtype=np.float32, count=len(seqs)), torch.float32)])
        set_context(True, cu_q, cu_k, h["max_seqlen_q"], h["max_seqlen_k"], slots, None, tables)
        return ids, pos

    def prepare_decode(self, seqs: List[Sequence]):
        h = build_decode_inputs(seqs, self.block_size)
        set_context(False, slot_mapping=self._to_device(h["slot_mapping"], torch.int32),
                    context_lens=self._to_device(h["context_lens"], torch.int32),
                    block_tables=self._to_device(h["block_tables"], torch.int32), decode_plan=DecodePlan())
        return self._to_device(h["input_ids"], torch.int64), self._to_device(h["positions"], torch.int64)

    def prepare_sample(self, seqs: List[Sequence]) -> torch.Tensor:
        return self._to_device(np.fromiter((s.temperature for s in seqs), dtype=np.float32, count=len(seqs)),
                               torch.float32)

    # ---- execution -----------------------------------------------------------------------------
    def _init_decode_staging(self, max_bs: int) -> None:
        """Pinned host buffers and one device buffer holding every per-step decode input; the
        graph's static tensors are typed views into the device buffer, so a decode step needs a
        single host-to-device transfer (the reference issues one copy per tensor plus one device copy
        per graph variable, nanovllm/engine/model_runner.py:162-179,197-203).  There are two host
        buffers, used in turn: with steps launched ahead of the previous step's tokens the copy
        of one step may still be queued while the host fills in the next."""
        fields = [("input_ids", np.int64, (max_bs,)), ("positions", np.int64, (max_bs,)),
                  ("slot_mapping", np.int32, (max_bs,)), ("context_lens", np.int32, (max_bs,)),
                  ("temperatures", np.float32, (max_bs,)), ("token_src", np.int32, (max_bs,)),
                  ("block_tables", np.int32, (max_bs, self.max_table_width))]
        offsets, total = {}, 0
        for name, dt, shape in fields:
            nbytes = int(np.prod(shape)) * np.dtype(dt).itemsize
            offsets[name] = (total, nbytes, dt, shape)
            total += (nbytes + 255) // 256 * 256
        # zero-filled: rows past the batch are replayed too (bucket padding) and must hold valid ids / positions
        self._stage_host = [torch.zeros(total, dtype=torch.uint8).pin_memory() for _ in range(2)]
        self._stage_dev = torch.zeros(total, dtype=torch.uint8, device=self.device)
        self._tokens_host = [torch.zeros(max_bs, dtype=torch.int64).pin_memory() for _ in range(2)]
        self._stage_turn = 0
        tdt = {np.int64: torch.int64, np.int32: torch.int32, np.float32: torch.float32}
        self._stage_np, self.graph_vars = [{}, {}], {}
        self._stage_offsets = {name: off for name, (off, _, _, _) in offsets.items()}
        for name, (off, nbytes, dt, shape) in offsets.items():
            for k in range(2):
                self._stage_np[k][name] = self._stage_host[k].numpy()[off: off + nbytes].view(dt).reshape(shape)
            self.graph_vars[name] = self._stage_dev[off: off + nbytes].view(tdt[dt]).view(shape)

    def _run_decode_graph(self, seqs: List[Sequence], prev: Optional[DecodeHandle] = None) -> torch.Tensor:
        """Fill a staging buffer, copy it once, replay the bucket's graph; returns logits.  Rows
        whose last token is still pending take it on the device from ``prev``'s sampler output."""
        bs = len(seqs)
        bucket = next(x for x in self.graph_bs if x >= bs)
        self.bucket_rows[0] += bs                                 # rows that carry a sequence / rows replayed
        self.bucket_rows[1] += bucket
        h = build_decode_inputs(seqs, self.block_size)
        self.kv_tokens_attended += int(h["context_lens"].sum(dtype=np.int64))
        self._stage_turn ^= 1
        st = self._stage_np[self._stage_turn]
        pending = h["input_ids"] == PENDING_TOKEN
        n_pending = int(pending.sum())
        if n_pending:
            assert prev is not None, "a pending token needs the step that samples it"
            st["token_src"][:bs] = np.fromiter((prev.row_of[s.seq_id] if p else -1 for s, p in zip(seqs, pending)),
                                               dtype=np.int32, count=bs)
            h["input_ids"][pending] = 0
        st["input_ids"][:bs] = h["input_ids"]
        st["positions"][:bs] = h["positions"]
        st["slot_mapping"][:bs] = h["slot_mapping"]
        st["slot_mapping"][bs:bucket] = -1                        # padded rows store nothing ...
        st["context_lens"][:bs] = h["context_lens"]
        st["context_lens"][bs:bucket] = 0                         # ... and attend over nothing
        st["temperatures"][:bs] = np.fromiter((s.temperature for s in seqs), dtype=np.float32, count=bs)
        st["block_tables"][:bs, : h["block_tables"].shape[1]] = h["block_tables"]   # stale columns stay: never read
        # one kernel reads the pinned buffer and writes the device buffer; pending input ids come
        # from the previous step's sampler output on the way
        if not n_pending:
            st["token_src"][:bs] = -1
        ids_off, idx_off = self._stage_offsets["input_ids"], self._stage_offsets["token_src"]
        rc = _lib.load().nva_stage_decode_inputs(
            self._stage_dev.data_ptr(), self._stage_host[self._stage_turn].data_ptr(), self._stage_dev.numel(),
            ids_off, idx_off, bs, prev.tokens_dev.data_ptr() if n_pending else None,
            prev.tokens_dev.numel() if n_pending else 0, torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "nva_stage_decode_inputs")
        for graph in self.graphs[bucket]:                         # later segments are enqueued while the first runs
            graph.replay()
        reset_context()                                           # a decode step: the head must not gather by a prefill step's cu_seqlens_q
        return self.model.compute_logits(self.graph_vars["outputs"][:bs])

    def can_launch_ahead(self, num_seqs: int) -> bool:
        """Whether a decode batch of this size can be launched without waiting for its tokens."""
        return bool(self.graph_bs) and num_seqs <= self.graph_bs[-1]

    def launch_decode(self, seqs: List[Sequence], prev: Optional[DecodeHandle] = None) -> DecodeHandle:
        """Enqueue one decode step and its sampling; nothing is read back.  ``prev`` is the step
        launched before, if its tokens have not been committed to the sequences yet."""
        with torch.inference_mode():
            started = self._step_started()
            logits = self._run_decode_graph(seqs, prev)
            tokens_dev = self.sampler(logits, self.graph_vars["temperatures"][: len(seqs)])
            self._step_ended(started)
            tokens_host = self._tokens_host[self._stage_turn]
            tokens_host[: len(seqs)].copy_(tokens_dev, non_blocking=True)
            ready = torch.cuda.Event()
            ready.record()
        reset_context()
        return DecodeHandle(seqs, {s.seq_id: i for i, s in enumerate(seqs)}, tokens_dev, tokens_host, ready)

    @torch.inference_mode()
    def run_model(self, input_ids: torch.Tensor, positions: torch.Tensor, is_prefill: bool) -> torch.Tensor:
        if is_prefill:                                            # final norm on the last row of every sequence only
            return self.model.prefill_logits(input_ids, positions)
        return self.model.compute_logits(self.model(input_ids, positions))

    def _step_started(self):
        """Start event of a decode step when the caller asked for step timings (``decode_step_events``)."""
        if self.decode_step_events is None:
            return None
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        return ev

    def _step_ended(self, started) -> None:
        if started is not None:
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            self.decode_step_events.append((started, ev))

    def run(self, seqs: List[Sequence], is_prefill: bool) -> List[int]:
        with torch.inference_mode():
            started = None if is_prefill else self._step_started()
            if not is_prefill and self.graph_bs and len(seqs) <= self.graph_bs[-1]:
                logits = self._run_decode_graph(seqs)
                temperatures = self.graph_vars["temperatures"][: len(seqs)]
            else:
                if is_prefill:
                    input_ids, positions = self.prepare_prefill(seqs)
                    temperatures = self._pf_temperatures          # staged with the other prefill inputs
                else:
                    self.kv_tokens_attended += sum(len(s) for s in seqs)
                    input_ids, positions = self.prepare_decode(seqs)
                    temperatures = self.prepare_sample(seqs)
                logits = self.run_model(input_ids, positions, is_prefill)
            tokens_dev = self.sampler(logits, temperatures)
            self._step_ended(started)
            tokens = tokens_dev.tolist()                           # the one device->host sync per step
        reset_context()
        return tokens

    @torch.inference_mode()
    def capture_graphs(self) -> None:
        cfg = self.config
        max_bs = min(cfg.max_num_seqs, 512)
        self._init_decode_staging(max_bs)
        gv = self.graph_vars
        input_ids, positions, slot_mapping = gv["input_ids"], gv["positions"], gv["slot_mapping"]
        context_lens, block_tables = gv["context_lens"], gv["block_tables"]
        outputs = torch.zeros(max_bs, self.cfg.hidden_size, dtype=torch.bfloat16, device=self.device)
        step = cfg.graph_bucket_step                      # the reference captures 1, 2, 4, 8 and every 16th size (model_runner.py:227)
        self.graph_bs = [b for b in (1, 2, 4, 8) if b <= max_bs and b < step] + list(range(step, max_bs + 1, step))
        if self.graph_bs[-1] != max_bs:
            self.graph_bs.append(max_bs)
        # The layer stack of a bucket is captured as several consecutive graphs instead of one:
        # launching a graph costs the host about a microsecond per node before the first kernel
        # starts, and with segments only the first segment's launch is exposed -- the others are
        # enqueued while the GPU already runs.
        n_layers = len(self.model.layers)
        cuts = sorted({round(i * n_layers / self.graph_segments) for i in range(self.graph_segments + 1)})
        pool = None
        for bs in reversed(self.graph_bs):
            set_context(False, slot_mapping=slot_mapping[:bs], context_lens=context_lens[:bs],
                        block_tables=block_tables[:bs])
            outputs[:bs] = self.model(input_ids[:bs], positions[:bs])        # eager warm-up (sizes workspaces)
            # the captured layers share one work split of the decode kernel: the first layer derives
            # it at every replay, the others take it from the workspace
            get_context().decode_plan = DecodePlan(capturing=True)
            segments, hidden, residual = [], None, None
            for first, last in zip(cuts[:-1], cuts[1:]):
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, pool):
                    hidden, residual = self.model.forward_layers(input_ids[:bs], positions[:bs], hidden, residual,
                                                                 first, last)
                    if last == n_layers:
                        outputs[:bs] = self.model.finish(hidden, residual)
                if pool is None:
                    pool = graph.pool()
                segments.append((graph, hidden, residual))      # keep the boundary activations alive
            self.graphs[bs] = [g for g, _, _ in segments]
            self._graph_keepalive.append(segments)
            torch.cuda.synchronize()
            reset_context()
        self.graph_pool = pool
        self.graph_vars["outputs"] = outputs
