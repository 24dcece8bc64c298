"""Host-side engine logic: block manager / prefix cache, scheduler, step-input builders.
Pure Python + numpy, no GPU.  Reference behaviour: nanovllm/engine/{block_manager,scheduler,
sequence,model_runner}.py."""
import numpy as np
import pytest
import xxhash

from nanovllm_amd.engine import BlockManager, EngineConfig, SamplingParams, Scheduler, Sequence, SequenceStatus, qwen3_0_6b
from nanovllm_amd.engine.model_runner import build_decode_inputs, build_prefill_inputs

BS = 256


def _seq(n, start=0, **kw):
    return Sequence(list(range(start, start + n)), SamplingParams(**kw))


def test_sequence_block_arithmetic():
    s = _seq(600)
    assert (s.num_blocks, s.last_block_num_tokens, s.num_cached_blocks) == (3, 88, 0)
    assert s.block(2) == list(range(512, 600)) and len(s.block(0)) == 256
    s.append_token(7)
    assert (len(s), s.last_token, s.num_completion_tokens) == (601, 7, 1)
    assert _seq(512).num_blocks == 2 and _seq(512).last_block_num_tokens == 256 and _seq(513).num_blocks == 3


def test_block_hash_is_chained_xxh64_of_int64_ids():
    ids = list(range(256))
    h0 = BlockManager.compute_hash(ids)
    assert h0 == xxhash.xxh64(np.arange(256, dtype="<i8").tobytes()).intdigest()
    h1 = BlockManager.compute_hash(ids, h0)
    assert h1 == xxhash.xxh64(h0.to_bytes(8, "little") + np.arange(256, dtype="<i8").tobytes()).intdigest()
    assert h1 != h0 and BlockManager.compute_hash(ids, 5) != BlockManager.compute_hash(ids, 6)


def test_prefix_cache_shares_full_blocks_only():
    bm = BlockManager(16)
    a = _seq(600)
    bm.allocate(a)
    assert a.block_table == [0, 1, 2] and a.num_cached_tokens == 0
    b = Sequence(list(range(512)) + [9999] * 100)             # same first two blocks
    bm.allocate(b)
    assert b.block_table[:2] == [0, 1] and b.block_table[2] not in (0, 1, 2) and b.num_cached_tokens == 512
    assert bm.blocks[0].ref_count == 2 and bm.blocks[2].ref_count == 1
    c = Sequence([5] + list(range(1, 600)))                    # differs in block 0: nothing shared afterwards
    bm.allocate(c)
    assert c.num_cached_tokens == 0 and not set(c.block_table) & set(a.block_table)
    bm.deallocate(a)
    assert bm.blocks[0].ref_count == 1 and 2 in bm.free_block_ids and 0 not in bm.free_block_ids
    bm.deallocate(b)
    bm.deallocate(c)
    assert len(bm.free_block_ids) == 16 and not bm.used_block_ids
    d = _seq(300)                                              # freed blocks keep their hash: revived
    bm.allocate(d)
    assert d.block_table[0] == 0 and d.num_cached_tokens == 256


def test_fully_cached_prompt_has_empty_query_span():
    bm = BlockManager(8)
    a, b = _seq(512), _seq(512)
    bm.allocate(a)
    bm.allocate(b)
    assert b.num_cached_tokens == 512 and b.block_table == a.block_table
    h = build_prefill_inputs([a, b], BS)
    assert h["cu_seqlens_q"].tolist() == [0, 512, 512] and h["cu_seqlens_k"].tolist() == [0, 512, 1024]
    assert h["block_tables"] is not None and h["slot_mapping"].size == 512


def test_may_append_opens_and_seals_blocks():
    bm = BlockManager(4)
    s = _seq(255)
    bm.allocate(s)
    assert s.block_table == [0] and bm.blocks[0].hash == -1
    s.append_token(1)                                           # 256 tokens: block full -> sealed
    bm.may_append(s)
    assert bm.blocks[0].hash == BlockManager.compute_hash(s.block(0)) and s.block_table == [0]
    s.append_token(2)                                           # 257: needs a block
    assert bm.can_append(s)
    bm.may_append(s)
    assert s.block_table == [0, 1]
    bm2 = BlockManager(1)
    t = _seq(256)
    bm2.allocate(t)
    t.append_token(3)
    assert not bm2.can_append(t)


@pytest.mark.parametrize("lens,cached_blocks", [([5, 300, 256], [0, 0, 0]), ([700, 260], [2, 1])])
def test_prefill_inputs_match_per_position_formula(lens, cached_blocks):
    rng = np.random.default_rng(0)
    seqs, free = [], list(rng.permutation(64))
    for n, cb in zip(lens, cached_blocks):
        s = Sequence(list(rng.integers(0, 1000, n)))
        s.block_table = [int(free.pop()) for _ in range(s.num_blocks)]
        s.num_cached_tokens = cb * BS
        seqs.append(s)
    h = build_prefill_inputs(seqs, BS)
    ids, pos, slots = [], [], []
    for s in seqs:                                              # brute force, one position at a time
        for p in range(s.num_cached_tokens, len(s)):
            ids.append(s.token_ids[p])
            pos.append(p)
            slots.append(s.block_table[p // BS] * BS + p % BS)
    assert h["input_ids"].tolist() == ids and h["positions"].tolist() == pos and h["slot_mapping"].tolist() == slots
    assert h["cu_seqlens_q"].tolist() == np.cumsum([0] + [len(s) - s.num_cached_tokens for s in seqs]).tolist()
    assert h["cu_seqlens_k"].tolist() == np.cumsum([0] + lens).tolist()
    assert h["max_seqlen_q"] == max(len(s) - s.num_cached_tokens for s in seqs) and h["max_seqlen_k"] == max(lens)
    if any(cached_blocks):
        bt = h["block_tables"]
        assert bt.dtype == np.int32 and bt.shape == (len(seqs), max(s.num_blocks for s in seqs))
        for i, s in enumerate(seqs):
            assert bt[i, : s.num_blocks].tolist() == s.block_table and (bt[i, s.num_blocks:] == -1).all()
    else:
        assert h["block_tables"] is None


def test_decode_inputs_match_per_position_formula():
    seqs = []
    for n, table in [(1, [7]), (256, [3]), (257, [3, 9]), (1000, [1, 2, 4, 8])]:
        s = Sequence(list(range(n)))
        s.block_table = table
        seqs.append(s)
    h = build_decode_inputs(seqs, BS)
    assert h["input_ids"].tolist() == [0, 255, 256, 999]
    assert h["positions"].tolist() == [0, 255, 256, 999] and h["context_lens"].tolist() == [1, 256, 257, 1000]
    assert h["slot_mapping"].tolist() == [7 * 256, 3 * 256 + 255, 9 * 256, 8 * 256 + 999 % 256]
    assert h["block_tables"].tolist() == [[7, -1, -1, -1], [3, -1, -1, -1], [3, 9, -1, -1], [1, 2, 4, 8]]


def _config(**kw):
    return EngineConfig(qwen3_0_6b(), **kw)


def test_scheduler_prefill_first_then_decode_and_finish():
    sch = Scheduler(_config(num_kvcache_blocks=16, max_num_batched_tokens=4096, max_model_len=4096))
    a, b = _seq(300, max_tokens=2, ignore_eos=True), _seq(3000, 5000, max_tokens=1, ignore_eos=True)
    c = _seq(1000, 9000, max_tokens=3, ignore_eos=True)
    for s in (a, b, c):
        sch.add(s)
    batch, is_prefill = sch.schedule()
    assert is_prefill and batch == [a, b]                       # c would exceed the 4096-token budget
    sch.postprocess(batch, [1, 2])
    assert b.is_finished and not a.is_finished and not b.block_table
    batch, is_prefill = sch.schedule()
    assert is_prefill and batch == [c]                          # waiting work is admitted before decoding
    sch.postprocess(batch, [3])
    batch, is_prefill = sch.schedule()
    assert not is_prefill and batch == [a, c]
    sch.postprocess(batch, [4, 5])
    assert a.is_finished and a.completion_token_ids == [1, 4]
    batch, _ = sch.schedule()
    sch.postprocess(batch, [6])
    assert c.is_finished and sch.is_finished() and len(sch.block_manager.free_block_ids) == 16


def test_scheduler_eos_and_preemption_by_recompute():
    sch = Scheduler(_config(num_kvcache_blocks=2, eos=42))
    a, b = _seq(256, max_tokens=8), _seq(256, 1000, max_tokens=8)
    sch.add(a)
    sch.add(b)
    batch, is_prefill = sch.schedule()
    assert is_prefill and batch == [a, b]
    sch.postprocess(batch, [1, 2])                              # both now need a second block; none is free
    batch, is_prefill = sch.schedule()
    assert not is_prefill and batch == [a]                      # b was preempted to make room
    assert b.status is SequenceStatus.WAITING and not b.block_table and sch.waiting[0] is b
    sch.postprocess(batch, [42])                                # eos ends a
    assert a.is_finished and a.completion_token_ids == [1, 42]
    batch, is_prefill = sch.schedule()
    assert is_prefill and batch == [b] and len(b) == 257        # recomputed from its full history


def test_engine_config_checks():
    with pytest.raises(AssertionError):
        _config(kvcache_block_size=128)
    with pytest.raises(AssertionError):
        _config(max_num_batched_tokens=1024, max_model_len=4096)
    with pytest.raises(AssertionError):
        SamplingParams(temperature=1e-12)
    assert SamplingParams(temperature=0).temperature == 0
    assert _config(max_model_len=10 ** 6, max_num_batched_tokens=65536).max_model_len == 40960


# ---- decode steps launched one step ahead of their tokens --------------------------------------
class _FakeHandle:
    def __init__(self, seqs, toks):
        self.seqs, self._toks = seqs, toks
        self.row_of = {s.seq_id: i for i, s in enumerate(seqs)}

    def tokens(self):
        return self._toks


class _FakeRunner:
    """Stands in for the GPU: the token after a sequence of length n whose last token is t is a
    fixed function of (first prompt token, n, t), so that any mix-up of rows, positions or
    pending tokens changes the completions."""
    vocab = 50

    def __init__(self):
        self.launched_ahead = 0

    def _next(self, seq, last):
        return (seq.token_ids[0] * 31 + len(seq) * 7 + last * 13) % self.vocab

    def run(self, seqs, is_prefill):
        from nanovllm_amd.engine.sequence import PENDING_TOKEN
        assert all(PENDING_TOKEN not in s.token_ids for s in seqs)
        return [self._next(s, s.token_ids[-1]) for s in seqs]

    def can_launch_ahead(self, n):
        return True

    def launch_decode(self, seqs, prev=None):
        from nanovllm_amd.engine.sequence import PENDING_TOKEN
        toks = []
        for s in seqs:
            last = s.token_ids[-1]
            if last == PENDING_TOKEN:
                last = prev.tokens()[prev.row_of[s.seq_id]]
                self.launched_ahead += 1
            assert PENDING_TOKEN not in s.token_ids[:-1]
            toks.append(self._next(s, last))
        return _FakeHandle(list(seqs), toks)


def _fake_engine(lookahead, **kw):
    from nanovllm_amd.engine.llm import LLMEngine
    eng = LLMEngine.__new__(LLMEngine)
    eng.config = _config(**kw)
    eng.tokenizer = None
    eng.model_runner = _FakeRunner()
    eng.scheduler = Scheduler(eng.config)
    eng.lookahead = lookahead
    eng._inflight = None
    eng.stats = {k: 0 for k in ("prefill_steps", "decode_steps", "prefill_tokens", "decode_tokens", "prefill_s", "decode_s")}
    return eng


@pytest.mark.parametrize("eos,blocks", [(-1, 64), (7, 64), (-1, 9), (7, 9)])
def test_lookahead_loop_matches_the_synchronous_loop(eos, blocks):
    """Same completions with and without lookahead: plain, with sequences ending on eos (their
    speculative step is dropped), with a cache so small that sequences are preempted and
    recomputed, and both.  Lengths cross several block boundaries (sealing, new blocks)."""
    rng = np.random.default_rng(3)
    prompts = [[int(100 + i)] + rng.integers(0, 50, size=int(n)).tolist()
               for i, n in enumerate(rng.integers(200, 700, size=12))]
    params = [SamplingParams(max_tokens=int(m), ignore_eos=(eos < 0)) for m in rng.integers(1, 400, size=12)]
    results, engines = [], []
    for lookahead in (False, True):
        eng = _fake_engine(lookahead, num_kvcache_blocks=blocks, eos=eos, max_num_batched_tokens=4096, max_model_len=4096)
        results.append(eng.generate(prompts, params))
        engines.append(eng)
        bm = eng.scheduler.block_manager
        assert len(bm.free_block_ids) == blocks and not bm.used_block_ids and eng._inflight is None
    assert [r["token_ids"] for r in results[0]] == [r["token_ids"] for r in results[1]]
    assert engines[1].model_runner.launched_ahead > 0 and engines[0].model_runner.launched_ahead == 0
    for r, p in zip(results[1], params):
        ids = r["token_ids"]
        assert 1 <= len(ids) <= p.max_tokens and (len(ids) == p.max_tokens or ids[-1] == eos)
        assert eos < 0 or eos not in ids[:-1]
    if eos < 0 and blocks == 64:                                # no preemption, no eos: identical prefix-cache state
        a, b = (e.scheduler.block_manager for e in engines)
        assert a.hash_to_block_id == b.hash_to_block_id
        assert [blk.hash for blk in a.blocks] == [blk.hash for blk in b.blocks]


def test_commit_drops_the_step_that_ran_past_an_eos():
    sch = Scheduler(_config(num_kvcache_blocks=4, eos=42))
    a, b = _seq(10, max_tokens=8), _seq(10, 100, max_tokens=8)
    sch.add(a)
    sch.add(b)
    batch, _ = sch.schedule()
    sch.postprocess(batch, [1, 2])
    batch, _ = sch.schedule()
    w1 = sch.advance(batch)                                     # step t launched
    batch2, _ = sch.schedule()
    assert batch2 == [a, b]
    w2 = sch.advance(batch2)                                    # step t+1 launched before t's tokens are known
    assert len(a) == 13 and w1 == [11, 11] and w2 == [12, 12]
    done = sch.commit(batch, w1, [42, 5])                       # a sampled eos at step t
    assert done == [a] and a.completion_token_ids == [1, 42] and a.is_finished and not a.block_table
    assert list(sch.running) == [b]
    done = sch.commit(batch2, w2, [9, 6])                       # a's token of step t+1 is dropped
    assert done == [] and a.completion_token_ids == [1, 42] and b.completion_token_ids == [2, 5, 6]
