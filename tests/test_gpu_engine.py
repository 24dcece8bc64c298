"""End-to-end checks of the hot path inside a Qwen3-architecture stack on the GPU:
the engine's prefill / decode steps against the CPU oracle model, and the generate() loop
(prefix cache, preemption, graph replay) for the behaviour the reference's engine has."""
import pytest
import torch

from oracle import engine_cpu, glue
from nanovllm_amd.engine import EngineConfig, ModelConfig, SamplingParams, Sequence
from nanovllm_amd.engine.llm import LLM
from nanovllm_amd.context import reset_context
from nanovllm_amd.engine.model_runner import ModelRunner, build_decode_inputs, build_prefill_inputs

pytestmark = pytest.mark.gpu


def tiny_model(**kw):
    base = dict(vocab_size=2048, hidden_size=512, num_hidden_layers=3, num_attention_heads=4, num_key_value_heads=2,
                head_dim=128, intermediate_size=1024, max_position_embeddings=4096, name="tiny")
    base.update(kw)
    return ModelConfig(**base)


@pytest.fixture(scope="module")
def runner(dev):
    cfg = EngineConfig(tiny_model(), max_model_len=2048, max_num_batched_tokens=4096, num_kvcache_blocks=40,
                       enforce_eager=True)
    return ModelRunner(cfg)


def _rel_err(got, want):
    got, want = got.float().cpu(), want.float()
    return float((got - want).norm() / want.norm().clamp_min(1e-12))


def _steps_match_cpu_oracle_model(runner, tol, graph_decode=False, n_first=300, lens=(700, 290, 33)):
    """Prefill (with a prefix-cache hit in the batch), then two decode steps, teacher-forced:
    logits of the HIP path vs the CPU oracle on the same weights, and the KV cache rows written by
    the (fused) scatter against the rows the oracle's scatter wrote."""
    cfg = runner.cfg
    weights = {k: v.detach().cpu() for k, v in runner.model.state_dict().items()}
    rope = glue.build_rope_cache(cfg.head_dim, 2048, cfg.rope_theta)
    with torch.inference_mode():
        runner.kv_cache.zero_()
    kv_cpu = torch.zeros_like(runner.kv_cache, device="cpu")
    g = torch.Generator().manual_seed(0)
    errs = []

    def mk(n, table, cached=0, ids=None):
        s = Sequence(torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() if ids is None else ids)
        s.block_table, s.num_cached_tokens = table, cached
        return s

    first = mk(n_first, [5, 9])
    # first pass: fills blocks 5 and 9 (block 5 becomes a reusable full prefix block)
    second = [mk(lens[0], [1, 2, 3]),
              mk(lens[1], [5, 11], cached=256, ids=first.token_ids[:256] + [7] * (lens[1] - 256)), mk(lens[2], [20])]
    for seqs in ([first], second):
        h = build_prefill_inputs(seqs, 256)
        ids, pos = runner.prepare_prefill(seqs)
        with torch.inference_mode():
            logits = runner.run_model(ids, pos, True)            # final norm on the last rows only
            # the reference's order -- norm every row, then gather -- gives the same bits
            assert torch.equal(logits, runner.model.compute_logits(runner.model(ids, pos)))
        ctx = engine_cpu.context_from_host_inputs(h, True)
        hidden = engine_cpu.forward(weights, cfg, torch.from_numpy(h["input_ids"]), torch.from_numpy(h["positions"]),
                                    ctx, kv_cpu, rope, "fp32")
        want = engine_cpu.compute_logits(weights, cfg, hidden, ctx)
        assert logits.shape == want.shape == (len(seqs), cfg.vocab_size)
        reset_context()                                          # as ModelRunner.run does after every step
        errs.append(_rel_err(logits, want))
        assert errs[-1] < tol, errs
    assert (h["block_tables"] is not None)                       # the second batch went through the paged path
    seqs = seqs[:2] + [seqs[2]]
    for step in range(2):                                        # decode, same forced token on both sides
        for s in seqs:
            s.append_token(int(torch.randint(0, cfg.vocab_size, (1,), generator=g)))
            if len(s) % 256 == 1:
                s.block_table.append(30 + s.seq_id % 8)
        h = build_decode_inputs(seqs, 256)
        with torch.inference_mode():
            if graph_decode:                                     # replay of the captured bucket (3 rows in a bucket of 4)
                assert runner.graph_bs and not runner.enforce_eager
                logits = runner._run_decode_graph(seqs)
            else:
                ids, pos = runner.prepare_decode(seqs)
                logits = runner.model.compute_logits(runner.model(ids, pos))
        reset_context()
        ctx = engine_cpu.context_from_host_inputs(h, False)
        hidden = engine_cpu.forward(weights, cfg, torch.from_numpy(h["input_ids"]), torch.from_numpy(h["positions"]),
                                    ctx, kv_cpu, rope, "fp32")
        want = engine_cpu.compute_logits(weights, cfg, hidden, ctx)
        errs.append(_rel_err(logits, want))
        assert errs[-1] < tol, (step, errs)
    # both caches hold the same rows wherever anything was written (values agree to bf16 noise),
    # and the first layer's rows -- computed from identical inputs on both sides -- agree to the
    # glue kernels' one-ulp tolerance, V rows of the first layer bit for bit
    with torch.inference_mode():
        kv_gpu = runner.kv_cache.cpu()
    written = kv_cpu.float().abs().sum(dim=(-1, -2)) > 0
    assert torch.equal(written, kv_gpu.float().abs().sum(dim=(-1, -2)) > 0)
    assert _rel_err(kv_gpu, kv_cpu) < tol
    v0_gpu, v0_cpu = kv_gpu[1, 0].view(torch.int16), kv_cpu[1, 0].view(torch.int16)
    assert float((v0_gpu == v0_cpu).float().mean()) > 0.995      # same qkv GEMM inputs; bf16 GEMM rounding differs on few elements
    print("relative logit errors (prefill, prefill with prefix hit, decode, decode):", [round(e, 5) for e in errs])
    return errs


def test_model_steps_match_cpu_oracle_model(runner):
    _steps_match_cpu_oracle_model(runner, tol=3e-2)


def test_model_steps_at_qwen3_0_6b_geometry_match_cpu_oracle(dev):
    """The full Qwen3-0.6B architecture (28 layers, hidden 1024, 16 query / 8 kv heads of 128, MLP
    3072, tied 151,936-way LM head): one prefill with a prefix-cache hit and two graph-replayed
    decode steps against the fp32 CPU oracle model on the same weights."""
    from nanovllm_amd.engine import qwen3_0_6b
    cfg = EngineConfig(qwen3_0_6b(), max_model_len=2048, max_num_batched_tokens=2048, num_kvcache_blocks=40,
                       max_num_seqs=4, enforce_eager=False)
    runner = ModelRunner(cfg)
    assert runner.cfg.vocab_size == 151936 and len(runner.model.layers) == 28
    _steps_match_cpu_oracle_model(runner, tol=3e-2, graph_decode=True, n_first=280, lens=(300, 290, 33))


def test_model_steps_at_qwen3_8b_geometry_match_cpu_oracle(dev):
    """Two layers at the Qwen3-8B geometry (hidden 4096, 32 query / 8 kv heads of 128 -- GQA group
    4 --, MLP 12288, untied 151,936-way LM head), same procedure."""
    from nanovllm_amd.engine import qwen3_8b
    model = qwen3_8b()
    model.num_hidden_layers = 2
    cfg = EngineConfig(model, max_model_len=2048, max_num_batched_tokens=2048, num_kvcache_blocks=40,
                       max_num_seqs=4, enforce_eager=False)
    runner = ModelRunner(cfg)
    assert not runner.cfg.tie_word_embeddings and runner.cfg.num_attention_heads == 32
    _steps_match_cpu_oracle_model(runner, tol=3e-2, graph_decode=True, n_first=280, lens=(300, 290, 33))


def _requests(n, seed=0, lo=20, hi=600, out_lo=5, out_hi=40, vocab=2048, temperature=0.6):
    g = torch.Generator().manual_seed(seed)
    prompts = [torch.randint(0, vocab, (int(torch.randint(lo, hi + 1, (1,), generator=g)),), generator=g).tolist()
               for _ in range(n)]
    params = [SamplingParams(temperature=temperature, ignore_eos=True,
                             max_tokens=int(torch.randint(out_lo, out_hi + 1, (1,), generator=g))) for _ in range(n)]
    return prompts, params


@pytest.mark.parametrize("eager", [True, False])
def test_generate_returns_every_request_in_order(dev, eager):
    llm = LLM(tiny_model(), enforce_eager=eager, max_model_len=2048, max_num_batched_tokens=4096,
              num_kvcache_blocks=64, max_num_seqs=32)
    prompts, params = _requests(20)
    outs = llm.generate(prompts, params)
    assert len(outs) == 20
    for o, p in zip(outs, params):
        assert len(o["token_ids"]) == p.max_tokens and all(0 <= t < 2048 for t in o["token_ids"])
    assert llm.stats["decode_steps"] >= max(p.max_tokens for p in params) - 1
    assert len(llm.scheduler.block_manager.free_block_ids) == 64          # everything was released


def test_greedy_decode_is_reproducible_and_matches_eager(dev):
    """Temperature 0: graph replay and eager execution produce the same tokens for the first
    steps (later steps may drift by bf16 GEMM tie-breaks), and a rerun is bit-identical."""
    prompts, params = _requests(6, seed=3, out_lo=12, out_hi=12, temperature=0.0)
    runs = []
    for eager in (False, False, True):
        llm = LLM(tiny_model(), enforce_eager=eager, max_model_len=2048, max_num_batched_tokens=4096,
                  num_kvcache_blocks=32, max_num_seqs=8)
        runs.append([o["token_ids"] for o in llm.generate(prompts, params)])
    assert runs[0] == runs[1]
    assert [r[:2] for r in runs[0]] == [r[:2] for r in runs[2]]


def test_prefix_cache_hit_changes_nothing_but_the_work(dev):
    llm = LLM(tiny_model(), enforce_eager=True, max_model_len=2048, max_num_batched_tokens=4096,
              num_kvcache_blocks=32, max_num_seqs=8)
    g = torch.Generator().manual_seed(5)
    shared = torch.randint(0, 2048, (512,), generator=g).tolist()
    sp = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
    a = llm.generate([shared + [1, 2, 3]], sp)[0]["token_ids"]
    before = llm.stats["prefill_tokens"]
    seq_probe = Sequence(shared + [1, 2, 3])
    llm.scheduler.block_manager.allocate(seq_probe)                          # the two full blocks are still cached
    assert seq_probe.num_cached_tokens == 512
    llm.scheduler.block_manager.deallocate(seq_probe)
    sizes = []
    real = llm.model_runner.prepare_prefill

    def spy(seqs):
        ids, pos = real(seqs)
        sizes.append(ids.numel())
        return ids, pos
    llm.model_runner.prepare_prefill = spy
    b = llm.generate([shared + [1, 2, 3]], sp)[0]["token_ids"]               # served through the paged prefill path
    assert sizes == [3]                                                      # only the uncached tail was run
    assert llm.stats["prefill_tokens"] - before == 516                       # accounting counts full lengths
    assert a[:3] == b[:3]


def test_preemption_by_recompute_still_finishes(dev):
    llm = LLM(tiny_model(), enforce_eager=True, max_model_len=2048, max_num_batched_tokens=4096,
              num_kvcache_blocks=6, max_num_seqs=8)
    prompts, params = _requests(4, seed=7, lo=200, hi=250, out_lo=70, out_hi=90)
    outs = llm.generate(prompts, params)                                     # 4 x 2 blocks needed, 6 exist
    assert [len(o["token_ids"]) for o in outs] == [p.max_tokens for p in params]
    assert llm.stats["prefill_steps"] > 1


def test_lookahead_decode_produces_the_same_tokens(dev):
    """Greedy requests with staggered output lengths (the batch shrinks, rows move) and lengths
    that cross a block boundary: launching decode steps one step ahead of their tokens (ids
    handed over on the device) gives exactly the tokens of the synchronous loop.  Then with an
    eos token picked from that run, so that some requests end early and their speculative step is
    dropped."""
    prompts, params = _requests(12, seed=11, lo=200, hi=300, out_lo=3, out_hi=90, temperature=0.0)
    runs = {}
    for lookahead in (False, True):
        llm = LLM(tiny_model(), max_model_len=2048, max_num_batched_tokens=4096, num_kvcache_blocks=40, max_num_seqs=16,
                  decode_lookahead=lookahead)
        assert llm.lookahead == lookahead
        runs[lookahead] = [o["token_ids"] for o in llm.generate(prompts, params)]
        assert len(llm.scheduler.block_manager.free_block_ids) == 40
    assert runs[True] == runs[False]
    eos = runs[False][0][len(runs[False][0]) // 2]              # a token the first request emits mid-way
    for p in params:
        p.ignore_eos = False
    stopped = {}
    for lookahead in (False, True):
        llm = LLM(tiny_model(), max_model_len=2048, max_num_batched_tokens=4096, num_kvcache_blocks=40, max_num_seqs=16,
                  decode_lookahead=lookahead, eos=eos)
        stopped[lookahead] = [o["token_ids"] for o in llm.generate(prompts, params)]
    # batches differ between the runs once sequences end early (other GEMM shapes, bf16 tie-breaks),
    # so only the structure is compared: every request ends on its first eos or at max_tokens
    for run in stopped.values():
        for ids, p in zip(run, params):
            assert 1 <= len(ids) <= p.max_tokens and eos not in ids[:-1]
            assert ids[-1] == eos or len(ids) == p.max_tokens
        assert any(ids[-1] == eos and len(ids) < p.max_tokens for ids, p in zip(run, params))
    assert [r[:1] for r in stopped[True]] == [r[:1] for r in runs[True]]


def test_bench_request_mix_at_full_request_count(dev):
    """The 256 requests of the end-to-end benchmark (prompt lengths U[100,1024] over the whole
    vocabulary, temperature 0.6, ignore_eos) on the full Qwen3-0.6B architecture with hipGraph
    decode, output lengths divided by 8 to keep the run short: every request returns exactly
    ``max_tokens`` ids inside the vocabulary, every KV block is back on the free list afterwards,
    the bucket accounting adds up, and a second generate() on newly drawn ids of the same lengths
    gives the same counts."""
    import os
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    from nanovllm_amd.engine import qwen3_0_6b
    prompts, params = bench.e2e_workload()
    assert len(prompts) == 256 and min(map(len, prompts)) >= 100 and max(map(len, prompts)) <= 1024
    for p in params:
        p.max_tokens = max(1, p.max_tokens // 8)
    llm = LLM(qwen3_0_6b(), enforce_eager=False, max_model_len=4096, num_kvcache_blocks=2048)
    mr, bm = llm.model_runner, llm.scheduler.block_manager
    assert mr.graph_bs[-1] == 512 and 256 in mr.graph_bs
    for round_ in range(2):
        used0, replayed0 = mr.bucket_rows
        steps0 = llm.stats["decode_steps"]
        outs = llm.generate(bench.fresh_prompts(prompts, 100 + round_), params)
        assert len(outs) == 256
        for o, p in zip(outs, params):
            assert len(o["token_ids"]) == p.max_tokens
            assert all(0 <= t < 151936 for t in o["token_ids"])
        assert len(bm.free_block_ids) == 2048 and not bm.used_block_ids       # every block was released
        assert not llm.scheduler.running and not llm.scheduler.waiting
        used, replayed = mr.bucket_rows[0] - used0, mr.bucket_rows[1] - replayed0
        # every sampled token but the one the prefill step produces comes from one decode row
        # (a launched-ahead step may add rows for sequences that had just finished: none here, ignore_eos)
        assert used == sum(p.max_tokens - 1 for p in params), (used, sum(p.max_tokens - 1 for p in params))
        assert used <= replayed <= used + 15 * (llm.stats["decode_steps"] - steps0)      # padding below one bucket step per step
        assert llm.stats["decode_steps"] - steps0 >= max(p.max_tokens for p in params) - 1
    # different prompts, same temperature: the sampled tokens differ between the rounds
    assert outs[0]["token_ids"] != [0] * len(outs[0]["token_ids"])
