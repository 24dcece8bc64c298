#!/usr/bin/env python3
"""Benchmark of the MI355X attention hot path.  Prints ONE JSON line on stdout.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

A "step" is one pass of the selected workload over one batch of synthetic input that is
already resident in HBM.  Workloads (shapes are the five benchmark configurations):
    e2e       (default) generate() over 256 requests on a Qwen3-0.6B-architecture model (config 4)
    longctx   Qwen3-8B-architecture long-context decode stress, batch 128, ctx U[4096,16384]  (config 5)
    decode    paged decode attention, batch 64, 16/8 heads, ctx U[100,2048]       (config 2)
    scatter   store_kvcache, 4096 tokens into 512 blocks x 256 slots              (config 1)
    prefill   causal varlen prefill, 16 sequences, half with cached prefix        (config 3)
    sampler   temperature sampling over 256 x 151,936 logits (--noise: the replayable path with an Exp(1) tensor)
    rope-scatter  q/k norm + rotary + cache write in one kernel, 16,384 tokens (the scatter the engine runs)
    glue      residual add + RMSNorm (--glue add-rms-norm) or SiLU(gate) * up (--glue silu-mul), 16,384 rows (--tokens N)
    decode-e2e-shape / decode-longctx-shape / copy   profiling helpers: the decode attention of configs 4 / 5
              alone (one layer); a plain copy of known size
    read-probe    calibration: a bare streaming read at the sizes of the bandwidth-bound workloads
The line carries `roofline` (algorithmic bytes or flops of the dominant kernel per launch,
divided by its average duration measured with HIP events on the launch stream) and
`cpu_baseline` (the CPU oracle timed on this box's host cores on a bounded sample).  The default
(e2e) line also carries `extra`: the rooflines of the scatter, decode, prefill and sampler
configurations and of the long-context decode shape, each timed in isolation in the same run, and
one eager (no hipGraph) pass of the same workload, and `extra.attainable`: what a bare streaming read of the decode and
sampler workloads' bytes takes on this GPU.  Every timed e2e pass generates from prompts
the engine has not seen (fresh draw per pass), like the reference's bench.py:22-27.
The scatter workload is timed as one replayed hipGraph of its K launches (a Python call costs as much
as that 7 us kernel; the eager-loop figure is reported beside it).
Only one GPU is used; --gpus above 1 is refused.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "nano-vllm_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16


def _event_time_ms(fn_list, steps, warmup):
    """Run fn_list[i % len] for warmup + steps iterations; HIP-event time of the timed part."""
    import torch
    n = len(fn_list)
    for i in range(warmup):
        fn_list[i % n]()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        fn_list[(warmup + i) % n]()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop)


def _steady_time_ms(fn_list, steps, warmup, tol=0.02, max_blocks=10):
    """Blocks of `steps` launches, timed one after the other until two consecutive blocks agree within `tol`:
    a kernel bound by the matrix pipes runs ~20 % slower in the first milliseconds after the GPU was idle than
    once its clocks have settled (the same 56 launches: 83.9, 76.5, 71.7, 69.1 us each in four consecutive
    blocks), so the sustained rate is what the last block shows.  Returns (ms of the last block, ms of the
    first block, blocks run)."""
    first = prev = _event_time_ms(fn_list, steps, warmup)
    blocks = 1
    while blocks < max_blocks:
        cur = _event_time_ms(fn_list, steps, 0)
        blocks += 1
        settled = abs(cur - prev) <= tol * prev
        prev = cur
        if settled:
            break
    return prev, first, blocks


def _graph_time_ms(fn_list, steps, warmup):
    """The same launches captured into one hipGraph and replayed: per-launch time of short kernels
    without the host in the loop (a Python + ctypes call takes 5-10 us, as long as the scatter kernel
    itself, so the eager loop above measures the call rate for them; the decode step runs its kernels
    from a replayed graph in the reference as here).  Returns (graph ms, eager-loop ms) for `steps` launches."""
    import torch
    eager = _event_time_ms(fn_list, steps, warmup)
    n = len(fn_list)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for i in range(steps):
                fn_list[i % n]()
    torch.cuda.synchronize()
    for _ in range(2):
        graph.replay()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    graph.replay()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop), eager


def _cpu_cores():
    """Threads the CPU baseline really runs on (torch's intra-op pool, which follows OMP_NUM_THREADS),
    and what the host reports."""
    import torch
    return {"cores": torch.get_num_threads(), "host_cpu_count": os.cpu_count()}


def _median_cpu_seconds(fn, repeats=5, warm=1):
    for _ in range(warm):
        fn()
    times = []
    for _ in range(repeats):
        t = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t)
    return statistics.median(times)


# ----------------------------------------------------------------------------- workloads
def bench_decode(args, dev):
    """Config 2.  Timed the way an engine calls it: 28 launches (the layers of one decode step of
    Qwen3-0.6B) share one work split, each on the KV pool of its own "layer" (4 rotating 1 GiB
    pools, so the 256 MB Infinity Cache cannot serve re-reads).  `standalone_us_per_launch` is the
    same call without a shared split (every launch derives it)."""
    import torch
    from nanovllm_amd import synthetic
    pools = 4
    caches = []
    for p in range(pools):
        g = torch.Generator(device=dev).manual_seed(100 + p)
        caches.append(tuple(torch.randn((1024, 256, 8, 128), generator=g, device=dev, dtype=torch.float32)
                            .to(torch.bfloat16) for _ in range(2)))
    case = synthetic.decode_case(seed=0, cache=(None, None))      # context lengths only; the tables are drawn per pool
    ctx = case.context_lens
    roof = decode_shape_roofline(dev, caches, 1024, ctx, 16, "config 2: batch 64, ctx U[100,2048]", width=8, layers=28,
                                 steps=args.steps)
    alone = decode_shape_roofline(dev, caches, 1024, ctx, 16, "", width=8, layers=None, steps=args.steps)
    roof["standalone_us_per_launch"] = alone["us_per_launch"]
    result = {
        "metric": "paged decode attention, achieved HBM GB/s (config 2)",
        "value": roof["achieved"], "unit": "GB/s", "ms_per_step": round(roof["us_per_launch"] / 1e3, 5),
        "config": {"workload": "paged_decode_attn config2: batch 64, 16q/8kv heads, head_dim 128, block 256, "
                               "ctx U[100,2048], 4 rotating 1 GiB KV pools, 28 launches per work split",
                   "batch": 64, "kv_tokens_per_step": int(ctx.sum())},
        "roofline": roof,
    }

    def cpu():
        import oracle
        c = synthetic.decode_case(seed=0)
        sec = _median_cpu_seconds(lambda: oracle.paged_decode_attention(
            c.q, c.k_cache, c.v_cache, c.context_lens, c.block_tables, c.scale, "sdpa"), repeats=5)
        return {"value": round(c.algorithmic_bytes / sec / 1e9, 3), "unit": "GB/s", **_cpu_cores(),
                "kind": "port", "sample": "config 2 full batch (64 sequences), bf16 torch SDPA on gathered pages, "
                                          "median of 5", "seconds": round(sec, 4)}
    return result, cpu


def bench_scatter(args, dev):
    import torch
    import nanovllm_amd as nva
    from nanovllm_amd import synthetic
    pools = 4
    fns, alg, cases = [], [], []
    n_tokens = getattr(args, "tokens", None) or 4096
    contiguous = bool(getattr(args, "contiguous", False))
    for p in range(pools):
        c = synthetic.scatter_case(seed=p, n_tokens=n_tokens)
        if contiguous:                               # slots as a prefill produces them: runs of consecutive slots, block by block
            c.slot_mapping = torch.where(c.slot_mapping >= 0, c.slot_mapping.sort().values, c.slot_mapping)
        k, v, kc, vc, sm = (t.to(dev) for t in (c.key, c.value, c.k_cache, c.v_cache, c.slot_mapping))
        cases.append(c)
        alg.append(c.algorithmic_bytes)
        fns.append(lambda k=k, v=v, kc=kc, vc=vc, sm=sm: nva.store_kvcache(k, v, kc, vc, sm))
    ms, eager_ms = _graph_time_ms(fns, args.steps, args.warmup)
    per_step_ms = ms / args.steps
    gbps = alg[0] / (per_step_ms * 1e-3) / 1e9
    result = {
        "metric": "store_kvcache, achieved HBM GB/s (config 1)", "value": round(gbps, 1), "unit": "GB/s",
        "ms_per_step": round(per_step_ms, 5),
        "config": {"workload": "store_kvcache config1: %d tokens x 8 kv heads x 128, 512 blocks x 256 slots, "
                               "5%% skipped%s" % (n_tokens, ", slots in ascending order" if contiguous else ""), "tokens": n_tokens},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None, "kernel": "store_kvcache_kernel",
                     "algorithmic_bytes_per_launch": int(alg[0]), "timing": "hipGraph replay of %d launches" % args.steps,
                     "us_per_launch_eager_loop": round(eager_ms / args.steps * 1e3, 2)},
    }

    def cpu():
        import oracle
        c = cases[0]
        sec = _median_cpu_seconds(lambda: oracle.store_kvcache(c.key, c.value, c.k_cache, c.v_cache, c.slot_mapping),
                                  repeats=7)
        return {"value": round(alg[0] / sec / 1e9, 3), "unit": "GB/s", **_cpu_cores(),
                "kind": "port", "sample": "config 1 full size, torch index_copy_, median of 7",
                "seconds": round(sec, 5)}
    return result, cpu


def bench_prefill(args, dev):
    import torch
    import nanovllm_amd as nva
    from nanovllm_amd import synthetic
    uniform = getattr(args, "uniform", None)
    if uniform:
        # S packed sequences of L tokens each, no prefix cache: the matrix-bound end of the prefill kernel
        n_seq, seq_len = (int(x) for x in uniform.lower().split("x"))
        hq, hkv, d = 16, 8, 128
        g = torch.Generator(device=dev).manual_seed(3)
        q = torch.randn(n_seq * seq_len, hq, d, device=dev, generator=g).to(torch.bfloat16)
        k = torch.randn(n_seq * seq_len, hkv, d, device=dev, generator=g).to(torch.bfloat16)
        v = torch.randn(n_seq * seq_len, hkv, d, device=dev, generator=g).to(torch.bfloat16)
        cu = torch.arange(0, (n_seq + 1) * seq_len, seq_len, dtype=torch.int32, device=dev)
        fn = lambda: nva.varlen_prefill_attention(q, k, v, cu, cu, seq_len, seq_len, d ** -0.5)
        flops = n_seq * 4 * d * hq * (seq_len * (seq_len + 1) // 2)
        what = "varlen_prefill_attn: %d packed sequences of %d tokens, no prefix cache, 16q/8kv heads, head_dim 128" % (n_seq, seq_len)
        metric = "causal varlen prefill attention, achieved TFLOP/s (%d x %d tokens)" % (n_seq, seq_len)
        kernel, total_q, c = "prefill_attn_kernel<packed>", n_seq * seq_len, None
    else:
        c = synthetic.prefill_case(seed=0)
        q, k, v, kc, vc = (t.to(dev) for t in (c.q, c.k, c.v, c.k_cache, c.v_cache))
        cq, ck, sm, bt = (t.to(dev) for t in (c.cu_seqlens_q, c.cu_seqlens_k, c.slot_mapping, c.block_tables))
        nva.store_kvcache(k, v, kc, vc, sm)
        fn = lambda: nva.varlen_prefill_attention(q, kc, vc, cq, ck, c.max_seqlen_q, c.max_seqlen_k, c.scale,
                                                  block_table=bt)
        flops = c.algorithmic_flops
        what = ("varlen_prefill_attn config3: 16 sequences, Lq U[100,1024], half with 1-3 cached "
                "256-token prefix blocks, 16q/8kv heads, head_dim 128")
        metric = "causal varlen prefill attention with prefix cache, achieved TFLOP/s (config 3)"
        kernel, total_q = "prefill_attn_kernel<paged>", int(c.q.shape[0])
    ms, first_ms, blocks = _steady_time_ms([fn], args.steps, args.warmup)
    per_step_ms = ms / args.steps
    tflops = flops / (per_step_ms * 1e-3) / 1e12
    result = {
        "metric": metric,
        "value": round(tflops, 2), "unit": "TFLOP/s", "ms_per_step": round(per_step_ms, 5),
        "config": {"workload": what, "total_q": total_q},
        "roofline": {"bound": "mfma", "achieved": round(tflops, 2), "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": kernel, "algorithmic_flops_per_launch": int(flops),
                     "timing": "sustained: blocks of %d launches until two consecutive blocks agree within 2 %% (%d blocks run); "
                               "the first block after idle, clocks not yet settled, is reported beside it" % (args.steps, blocks),
                     "us_per_launch_first_block_after_idle": round(first_ms / args.steps * 1e3, 2)},
    }

    def cpu():
        import oracle
        if c is None:
            # one sequence cut to 2048 tokens: the full size would take the host minutes
            n = min(2048, q.shape[0])
            qc, kc_, vc_ = q[:n].cpu(), k[:n].cpu(), v[:n].cpu()
            one = torch.tensor([0, n], dtype=torch.int32)
            sec = _median_cpu_seconds(lambda: oracle.varlen_prefill_attention(qc, kc_, vc_, one, one, 128 ** -0.5, precision="sdpa"), repeats=3)
            fl = 4 * 128 * 16 * (n * (n + 1) // 2)
            return {"value": round(fl / sec / 1e12, 4), "unit": "TFLOP/s", **_cpu_cores(), "kind": "port",
                    "sample": "one sequence of %d tokens, bf16 torch SDPA with explicit lower-right mask, median of 3" % n,
                    "seconds": round(sec, 3)}
        ek, ev = c.k_cache.clone(), c.v_cache.clone()
        oracle.store_kvcache(c.k, c.v, ek, ev, c.slot_mapping)
        sec = _median_cpu_seconds(lambda: oracle.varlen_prefill_attention(
            c.q, None, None, c.cu_seqlens_q, c.cu_seqlens_k, c.scale, ek, ev, c.block_tables, "sdpa"), repeats=3)
        return {"value": round(flops / sec / 1e12, 4), "unit": "TFLOP/s", **_cpu_cores(),
                "kind": "port", "sample": "config 3 full batch, bf16 torch SDPA with explicit lower-right mask, "
                                          "median of 3", "seconds": round(sec, 3)}
    return result, cpu


def bench_sampler(args, dev):
    import torch
    import nanovllm_amd as nva
    batch, vocab = 256, 151936
    g = torch.Generator(device=dev).manual_seed(5)
    sets = []
    for p in range(4):
        logits = (torch.randn((batch, vocab), generator=g, device=dev) * 2).to(torch.bfloat16)
        sets.append(logits)
    temps = torch.full((batch,), 0.6, device=dev)
    with_noise = bool(getattr(args, "noise", False))
    # the engine's sampler call: records in the library's built-in scratch (nva_sample_static, no allocation);
    # `--workspace`: nva_sample with a workspace tensor allocated per call
    static = not bool(getattr(args, "workspace", False))
    if with_noise:                                   # the replayable path: an Exp(1) tensor per set of logits is read as well
        noises = [torch.empty((batch, vocab), device=dev).exponential_(1.0, generator=g) for _ in sets]
        mk = lambda st: [lambda l=l, n=n: nva.sample(l, temps, n, static_scratch=st) for l, n in zip(sets, noises)]
    else:
        mk = lambda st: [lambda l=l, i=i: nva.sample(l, temps, None, seed=1, offset=i, static_scratch=st) for i, l in enumerate(sets)]
    ms = _event_time_ms(mk(static), args.steps, args.warmup)
    per_step_ms = ms / args.steps
    other_us = _event_time_ms(mk(not static), args.steps, args.warmup) / args.steps * 1e3

    alg = batch * vocab * (6 if with_noise else 2)
    gbps = alg / (per_step_ms * 1e-3) / 1e9
    result = {
        "metric": "sampler (%s), achieved HBM GB/s" % ("noise tensor given" if with_noise else "in-kernel randomness"),
        "value": round(gbps, 1), "unit": "GB/s",
        "ms_per_step": round(per_step_ms, 5),
        "config": {"workload": "sampler: 256 rows x 151,936 bf16 logits, T=0.6, " +
                               ("Exp(1) noise tensor read (the reference's argmax(p / E))" if with_noise else
                                "in-kernel randomness (tree of inverse-CDF draws, Philox uniforms)"),
                   "batch": batch},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": ("sampler_chunk_kernel<2, true>" if with_noise else "sampler_chunk_kernel<4, false>") + " + sampler_row_kernel",
                     "algorithmic_bytes_per_launch": alg,
                     ("us_per_launch_with_workspace_tensor" if static else "us_per_launch_static_scratch"): round(other_us, 2)},
    }

    def cpu():
        import oracle
        l = sets[0][:64].cpu()
        t = temps[:64].cpu()
        noise = torch.empty(64, vocab).exponential_(1.0)
        sec = _median_cpu_seconds(lambda: oracle.sample(l, t, noise), repeats=5)
        return {"value": round(64 * vocab * 2 / sec / 1e9, 3), "unit": "GB/s", **_cpu_cores(),
                "kind": "port", "sample": "64 of the 256 rows, eager torch sampler with pre-drawn noise, "
                                          "median of 5", "seconds": round(sec, 4)}
    return result, cpu


def bench_glue(args, dev):
    """The elementwise steps either side of the attention, as the engine runs them between its GEMMs:
    residual add + RMSNorm and SiLU(gate) * up, Qwen3-0.6B widths, a prefill-sized batch of rows."""
    import torch
    from nanovllm_amd.engine import layers
    n, hidden, inter = (getattr(args, "tokens", None) or 16384), 1024, 3072
    which = getattr(args, "glue", None) or "add-rms-norm"
    g = torch.Generator(device=dev).manual_seed(2)
    fns = []
    if which == "add-rms-norm":
        w = torch.ones(hidden, dtype=torch.bfloat16, device=dev)
        for _ in range(3):
            x = torch.randn(n, hidden, device=dev, generator=g).to(torch.bfloat16)
            r = torch.randn(n, hidden, device=dev, generator=g).to(torch.bfloat16)
            fns.append(lambda x=x, r=r: layers.add_rms_norm(x, r, w, 1e-6))
        alg = n * hidden * 2 * 4 + hidden * 2            # x and the residual in, both results out
        kernel = "rms_norm_kernel<2, true, false>"
    elif which == "last-token-norm":
        # the final norm of a prefill step: 29 sequences in a batch of n rows; only their last rows feed the LM head
        w = torch.ones(hidden, dtype=torch.bfloat16, device=dev)
        batch = 29
        cu = torch.linspace(0, n, batch + 1).to(torch.int32).to(dev)
        full = bool(getattr(args, "grid_order", False))   # (--grid-order here: the reference's order -- norm every row, then gather)
        for _ in range(3):
            x = torch.randn(n, hidden, device=dev, generator=g).to(torch.bfloat16)
            r = torch.randn(n, hidden, device=dev, generator=g).to(torch.bfloat16)
            if full:
                fns.append(lambda x=x, r=r: layers.add_rms_norm(x, r, w, 1e-6)[0][(cu[1:] - 1).long()].contiguous())
            else:
                fns.append(lambda x=x, r=r: layers.gather_last_rms_norm(x, r, cu, w, 1e-6))
        alg = batch * hidden * 2 * 3 + hidden * 2 + (batch + 1) * 4     # the picked rows of x and the residual in, their norm out
        kernel = "rms_norm_kernel<2, true, false> over all rows + index kernels" if full else "rms_norm_kernel<2, true, true>"
    else:
        for _ in range(3):
            x = torch.randn(n, 2 * inter, device=dev, generator=g).to(torch.bfloat16)
            fns.append(lambda x=x: layers.silu_and_mul(x))
        alg = n * inter * 2 * 3                          # gate and up in, the product out
        kernel = "silu_and_mul_kernel"
    ms = _event_time_ms(fns, args.steps, args.warmup) / args.steps
    gbps = alg / (ms * 1e-3) / 1e9
    result = {"metric": "%s, achieved HBM GB/s" % which, "value": round(gbps, 1), "unit": "GB/s", "ms_per_step": round(ms, 5),
              "config": {"workload": "%s: %d rows, hidden 1024 / intermediate 3072 (Qwen3-0.6B), output allocated per call as in the engine" % (which, n),
                         "tokens": n},
              "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                           "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None, "kernel": kernel,
                           "algorithmic_bytes_per_launch": alg}}
    return result, (lambda: None)


def bench_rope_scatter(args, dev):
    """The scatter as the engine runs it: q/k norm + rotary embedding + cache write in one kernel
    (nva_qk_norm_rope with cache pointers), Qwen3-0.6B head geometry, a prefill-sized batch of tokens."""
    import torch
    from nanovllm_amd.engine import layers
    n, hq, hkv, d = (getattr(args, "tokens", None) or 16384), 16, 8, 128
    g = torch.Generator(device=dev).manual_seed(1)
    w = torch.ones(d, dtype=torch.bfloat16, device=dev)
    rope = layers.build_rope_cache(d, 4096, 1e6, dev)
    pos = torch.randint(0, 4096, (n,), device=dev)
    fns = []
    for p in range(3):
        qkv = torch.randn(n, (hq + 2 * hkv) * d, device=dev, generator=g).to(torch.bfloat16)
        kc = torch.zeros(512, 256, hkv, d, dtype=torch.bfloat16, device=dev)
        vc = torch.zeros_like(kc)
        sm = torch.randperm(131072, device=dev)[:n].to(torch.int32)
        fns.append(lambda qkv=qkv, kc=kc, vc=vc, sm=sm: layers.qk_norm_rope(qkv, pos, w, w, rope, hq, hkv, d, 1e-6,
                                                                            kv_store=(kc, vc, sm)))
    ms = _event_time_ms(fns, args.steps, args.warmup) / args.steps
    # per token: the qkv row in; q, k out; the K and V cache rows out; one rope table row, a position and a slot id in
    alg = n * ((hq + 2 * hkv) * d * 2 + (hq + hkv) * d * 2 + 2 * hkv * d * 2 + d * 4 + 8 + 4)
    gbps = alg / (ms * 1e-3) / 1e9
    result = {"metric": "q/k norm + rotary + KV-cache scatter in one kernel, achieved HBM GB/s", "value": round(gbps, 1),
              "unit": "GB/s", "ms_per_step": round(ms, 5),
              "config": {"workload": "nva_qk_norm_rope with cache pointers: %d tokens, 16q/8kv heads x 128, slots drawn from "
                                     "512 blocks x 256" % n, "tokens": n},
              "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                           "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None, "kernel": "qk_norm_rope_kernel",
                           "algorithmic_bytes_per_launch": alg}}
    return result, (lambda: None)


def e2e_workload(num_seqs=256, max_input_len=1024, max_output_len=1024, vocab=151936, seed=0):
    """The request mix of the reference's bench.py:9-18, ids uniform over the whole vocabulary."""
    import random
    from nanovllm_amd.engine import SamplingParams
    rng = random.Random(seed)
    prompts = [[rng.randint(0, vocab - 1) for _ in range(rng.randint(100, max_input_len))] for _ in range(num_seqs)]
    params = [SamplingParams(temperature=0.6, ignore_eos=True, max_tokens=rng.randint(100, max_output_len))
              for _ in range(num_seqs)]
    return prompts, params


TRAFFIC_PROFILE = "profiles/hbm_traffic_pmc__all_kernels.txt"


def measured_traffic(key):
    """HBM bytes per launch from the tracked summary of the two rocprofv3 --pmc passes (FETCH_SIZE, then
    WRITE_SIZE, each scaled by what the same counter reads for the plain copy of `--workload copy`):
    the line `traffic_bytes_per_launch[<key>] = <bytes>` of TRAFFIC_PROFILE; None when it is absent."""
    import re
    try:
        text = open(os.path.join(ROOT, TRAFFIC_PROFILE)).read()
    except OSError:
        return None
    m = re.search(r"traffic_bytes_per_launch\[%s\]\s*=\s*([0-9_]+)" % re.escape(key), text)
    return int(m.group(1).replace("_", "")) if m else None


def decode_shape_roofline(dev, caches, num_blocks, ctx, hq, what, traffic=None, width=None, layers=None, steps=None):
    """Paged decode attention for the context lengths ``ctx``: block tables drawn without
    replacement from the pool, timed with HIP events while rotating through `caches` (separate
    K/V pools, so neither L2 nor the 256 MB Infinity Cache can serve re-reads).  With ``layers``
    the calls are grouped as the engine groups them: every ``layers`` consecutive calls share
    one work split, derived by the first of them (the layers of one decode step)."""
    import torch
    import nanovllm_amd as nva
    from nanovllm_amd import synthetic
    g = torch.Generator().manual_seed(1)
    batch = ctx.numel()
    tables = synthetic.decode_tables(ctx.tolist(), num_blocks, g, width=width).to(dev)
    ctx_d = ctx.to(dev)
    hkv, dh = caches[0][0].shape[2], caches[0][0].shape[3]
    q = torch.randn(batch, hq, dh, device=dev).to(torch.bfloat16)
    out = torch.empty(batch, 1, hq, dh, dtype=torch.bfloat16, device=dev)
    scale = dh ** -0.5
    from nanovllm_amd.context import DecodePlan
    state = {"calls": 0, "plan": None}

    def call(kc, vc):
        if layers:
            if state["calls"] % layers == 0:
                state["plan"] = DecodePlan()
            state["calls"] += 1
        nva.paged_decode_attention(q, kc, vc, ctx_d, tables, scale, out=out, plan=state["plan"])

    fns = [lambda kc=kc, vc=vc: call(kc, vc) for kc, vc in caches]
    reps = 3 * layers if layers else max(5 * len(fns), 60)      # whole steps: one build per `layers` calls
    if steps and steps > 1:
        reps = -(-steps // layers) * layers if layers else steps
    ms = _event_time_ms(fns, reps, layers if layers else len(fns)) / reps
    alg = int(ctx.sum()) * hkv * dh * 2 * 2 + 2 * q.numel() * 2
    gbps = alg / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": traffic,
            "kernel": "decode_stream_kernel<%d> (+ decode_merge_kernel<%d>): paged decode attention, %s, mean ctx %d%s"
                      % (hq // hkv, hq // hkv, what, int(ctx.float().mean()),
                         ", %d layers per work split" % layers if layers else ""),
            "algorithmic_bytes_per_launch": alg, "us_per_launch": round(ms * 1e3, 2)}


def decode_e2e_shape_roofline(dev, caches, num_blocks):
    """The e2e workload's own decode shape: the 256 requests of the bench mix mid-flight (context =
    prompt + half of the output, mean 813 tokens)."""
    import torch
    prompts, params = e2e_workload()
    ctx = torch.tensor([len(p) + sp.max_tokens // 2 for p, sp in zip(prompts, params)], dtype=torch.int32)
    roof = decode_shape_roofline(dev, caches, num_blocks, ctx, 16, "batch 256", measured_traffic("decode_e2e_shape"),
                                 width=16,           # the engine's static table width at max_model_len 4096
                                 layers=28)          # Qwen3-0.6B
    roof["traffic_source"] = TRAFFIC_PROFILE
    return roof


def bench_decode_longctx_shape(args, dev):
    """One layer of the long-context stress (config 5): batch 128, contexts U[4096,16384], 32 query
    / 8 kv heads; 4 private pools sized to the drawn contexts (about 5300 blocks, 2.8 GB each for K and for V)."""
    import random
    import torch
    rng = random.Random(0)
    ctx = torch.tensor([rng.randint(4096, 16384) for _ in range(128)], dtype=torch.int32)
    need = int(((ctx + 255) // 256).sum())
    caches = []
    for p in range(4):
        g = torch.Generator(device=dev).manual_seed(300 + p)
        caches.append(tuple(torch.empty((need + 8, 256, 8, 128), device=dev, dtype=torch.bfloat16).normal_(generator=g)
                            for _ in range(2)))
    roof = decode_shape_roofline(dev, caches, need + 8, ctx, 32, "batch 128, ctx U[4096,16384]", layers=36)
    result = {"metric": "paged decode attention at the long-context shape (config 5, one layer), achieved HBM GB/s",
              "value": roof["achieved"], "unit": "GB/s", "ms_per_step": round(roof["us_per_launch"] / 1e3, 5),
              "config": {"workload": "paged_decode_attn, batch 128, 32q/8kv heads, contexts U[4096,16384], "
                                     "4 rotating pools of %d blocks" % (need + 8)}, "roofline": roof}
    return result, (lambda: None)


def bench_decode_e2e_shape(args, dev):
    """Only the roofline leg of the e2e workload (for profiling runs): 4 private 4096-block pools."""
    import torch
    caches = []
    for p in range(4):
        g = torch.Generator(device=dev).manual_seed(200 + p)
        caches.append(tuple(torch.randn((4096, 256, 8, 128), generator=g, device=dev, dtype=torch.float32)
                            .to(torch.bfloat16) for _ in range(2)))
    roof = decode_e2e_shape_roofline(dev, caches, 4096)
    result = {"metric": "paged decode attention at the e2e decode shape, achieved HBM GB/s", "value": roof["achieved"],
              "unit": "GB/s", "ms_per_step": round(roof["us_per_launch"] / 1e3, 5),
              "config": {"workload": "paged_decode_attn, batch 256, contexts of the e2e bench mix mid-flight, "
                                     "4 rotating 4 GiB KV pools"}, "roofline": roof}
    return result, (lambda: None)


def bench_copy(args, dev):
    """A plain device-to-device copy of known size: the calibration kernel for FETCH_SIZE / WRITE_SIZE."""
    import torch
    n = 256 << 20
    src = torch.empty(n, dtype=torch.uint8, device=dev).random_(0, 255)
    dsts = [torch.empty_like(src) for _ in range(3)]
    ms = _event_time_ms([lambda d=d: d.copy_(src) for d in dsts], args.steps, args.warmup) / args.steps
    gbps = 2 * n / (ms * 1e-3) / 1e9
    result = {"metric": "plain copy kernel, read + write GB/s", "value": round(gbps, 1), "unit": "GB/s",
              "ms_per_step": round(ms, 5),
              "config": {"workload": "torch copy_ of 268,435,456 bytes (reads 256 MiB, writes 256 MiB)"},
              "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                           "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": 2 * n, "kernel": "copy",
                           "algorithmic_bytes_per_launch": 2 * n}}
    return result, (lambda: None)


def stream_read_us(dev, nbytes, steps=60, graph=False):
    """Microseconds a bare streaming read of `nbytes` takes (nva_probe_stream_read: the decode kernel's access
    discipline and nothing else), rotating through buffers that together exceed the 256 MB Infinity Cache.
    `graph`: as one replayed hipGraph of the launches (for sizes where a Python call lasts as long as the kernel)."""
    import torch
    from nanovllm_amd import _lib
    lib = _lib.load()
    nbytes = nbytes // 16 * 16
    n_buf = max(2, -(-(640 << 20) // nbytes))
    bufs = [torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(n_buf)]
    sink = torch.zeros(4, dtype=torch.int32, device=dev)

    def call(b):
        _lib.check(lib.nva_probe_stream_read(b.data_ptr(), nbytes, sink.data_ptr(), torch.cuda.current_stream().cuda_stream),
                   "nva_probe_stream_read")
    fns = [lambda b=b: call(b) for b in bufs]
    if graph:
        ms, _ = _graph_time_ms(fns, steps, 5)
    else:
        ms = _event_time_ms(fns, steps, 5)
    return ms / steps * 1e3


def device_copy_us(dev, nbytes, steps=400):
    """Microseconds the runtime's own device-to-device copy of `nbytes` takes (reads nbytes, writes nbytes), as one
    replayed hipGraph of the copies, rotating through buffers that together exceed the Infinity Cache: the attainable
    side of the kernels that read and write in equal parts (the scatters)."""
    import torch
    nbytes = nbytes // 16 * 16
    n_buf = max(2, -(-(400 << 20) // nbytes))
    src = [torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(n_buf)]
    dst = [torch.empty_like(b) for b in src]
    ms, _ = _graph_time_ms([lambda a=a, b=b: b.copy_(a) for a, b in zip(src, dst)], steps, 5)
    return ms / steps * 1e3


def bench_read_probe(args, dev):
    """What a bare streaming read costs at the sizes of the bandwidth-bound kernels' workloads."""
    sizes = {"scatter_config1 (read half of 31.9 MB)": 15_945_728, "sampler 256 x 151,936": 77_791_232,
             "decode config 2": 291_000_000, "decode e2e shape": 855_318_528}
    if getattr(args, "tokens", None):
        sizes = {"%d bytes" % args.tokens: int(args.tokens)}
    rows = {k: round(stream_read_us(dev, v, args.steps, graph=v < (64 << 20)), 2) for k, v in sizes.items()}
    big = max(sizes.values())
    us = rows[[k for k, v in sizes.items() if v == big][0]]
    gbps = big / us / 1e3
    result = {"metric": "bare streaming read (calibration), GB/s", "value": round(gbps, 1), "unit": "GB/s", "ms_per_step": round(us / 1e3, 5),
              "config": {"workload": "nva_probe_stream_read over %d bytes; us per launch at the other sizes in `us_by_size`" % big,
                         "us_by_size": rows},
              "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                           "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None, "kernel": "probe_stream_read_kernel",
                           "algorithmic_bytes_per_launch": big}}
    return result, (lambda: None)


def fresh_prompts(prompts, pass_index, vocab=151936):
    """Prompts of the same lengths with newly drawn token ids: every timed pass must prefill prompts
    the engine has never seen (its prefix cache keeps the hashes of freed blocks), as the reference's
    single timed generate() does (bench.py:22-27)."""
    import random
    rng = random.Random(10_000 + pass_index)
    return [[rng.randint(0, vocab - 1) for _ in p] for p in prompts]


def _e2e_passes(llm, prompts, params, passes, first_pass):
    """Time `passes` generate() calls, each on freshly drawn prompt ids; returns seconds."""
    import torch
    for k in llm.stats:
        llm.stats[k] = 0
    batches = [fresh_prompts(prompts, first_pass + i) for i in range(passes)]      # drawn outside the timed region
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for batch in batches:
        outs = llm.generate(batch, params)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert all(len(o["token_ids"]) == p.max_tokens for o, p in zip(outs, params))
    return dt


def collect_extra(dev, model, prompts, params):
    """The other configurations, each timed in isolation (a second or less of GPU time each), and one
    eager pass of the e2e workload, for the `extra` object of the default line."""
    import gc
    import torch
    from types import SimpleNamespace
    from nanovllm_amd.engine.llm import LLM
    extra = {}
    for name, fn, steps, kw in (("scatter_config1", bench_scatter, 400, {}), ("rope_scatter_16384_tokens", bench_rope_scatter, 100, {}),
                                ("decode_config2", bench_decode, 112, {}), ("prefill_config3", bench_prefill, 50, {}),
                                ("prefill_2x16384_tokens", bench_prefill, 10, {"uniform": "2x16384"}),
                                ("sampler_256x151936", bench_sampler, 100, {}),
                                ("sampler_with_noise_256x151936", bench_sampler, 50, {"noise": True}),
                                ("decode_config5_shape", bench_decode_longctx_shape, 1, {})):
        result, _ = fn(SimpleNamespace(steps=steps, warmup=max(3, steps // 10), **kw), dev)
        extra[name] = dict(result["roofline"], us_per_launch=round(result["ms_per_step"] * 1e3, 2))
        del result
        gc.collect()
        torch.cuda.empty_cache()
    # what a kernel that only reads the same bytes takes (launch, first-load latency and the streaming rate
    # of the part included): the attainable side of the HBM rooflines above
    extra["attainable"] = {"what": "us per launch of a bare streaming read of the same bytes (nva_probe_stream_read)",
                           "decode_config2_291MB_us": round(stream_read_us(dev, extra["decode_config2"]["algorithmic_bytes_per_launch"]), 2),
                           "sampler_78MB_us": round(stream_read_us(dev, extra["sampler_256x151936"]["algorithmic_bytes_per_launch"]), 2),
                           "decode_config5_shape_us": round(stream_read_us(dev, extra["decode_config5_shape"]["algorithmic_bytes_per_launch"], steps=12), 2),
                           "decode_e2e_shape_855MB_us": round(stream_read_us(dev, 855_318_528, steps=40), 2),
                           "scatter_config1_read_16MB_us": round(stream_read_us(dev, extra["scatter_config1"]["algorithmic_bytes_per_launch"] // 2, steps=400, graph=True), 2),
                           "scatter_config1_copy_16MB_to_16MB_us": round(device_copy_us(dev, extra["scatter_config1"]["algorithmic_bytes_per_launch"] // 2), 2),
                           "rope_scatter_copy_155MB_to_155MB_us": round(device_copy_us(dev, extra["rope_scatter_16384_tokens"]["algorithmic_bytes_per_launch"] // 2, steps=100), 2)}
    gc.collect()
    torch.cuda.empty_cache()
    llm = LLM(model, enforce_eager=True, max_model_len=4096, num_kvcache_blocks=4096)
    llm.generate(fresh_prompts(prompts[:32], 9_000), params[:32])
    dt = _e2e_passes(llm, prompts, params, 1, 5_000)
    total_out = sum(p.max_tokens for p in params)
    extra["e2e_eager"] = {"value": round(total_out / dt, 1), "unit": "tok/s", "s_per_pass": round(dt, 3),
                          "what": "the same 256-request workload with enforce_eager=True (no hipGraph decode), one pass",
                          "prefill_s": round(llm.stats["prefill_s"], 3), "decode_s": round(llm.stats["decode_s"], 3)}
    del llm
    gc.collect()
    torch.cuda.empty_cache()
    # config 5 end to end (Qwen3-8B architecture, batch 128, contexts U[4096,16384], 128 decode steps, greedy + T=1.0):
    # one warm-up pass and one timed pass of the engine, no profiler attached
    t0 = time.perf_counter()
    res, _ = bench_longctx(SimpleNamespace(steps=1, warmup=1, eager=False, requests=128), dev)
    extra["longctx_e2e"] = {"value": res["value"], "unit": "tok/s", "ms_per_decode_step": res["config"]["ms_per_decode_step"],
                            "kv_gbps_over_the_whole_step": res["roofline"]["achieved"], "frac_of_hbm_peak": res["roofline"]["frac"],
                            "kv_bytes_per_decode_step": res["config"]["kv_bytes_per_decode_step"],
                            "kv_cache_bytes": res["config"]["kv_cache_bytes"], "kv_cache_blocks": res["config"]["kv_cache_blocks"],
                            "what": res["config"]["workload"] + "; one timed pass of 128 engine decode steps after one warm-up pass",
                            "wall_s_including_setup": round(time.perf_counter() - t0, 1)}
    gc.collect()
    torch.cuda.empty_cache()
    return extra


def bench_e2e(args, dev):
    """Qwen3-0.6B architecture, random weights, 256 requests, hipGraph decode: output tok/s."""
    import gc
    import torch
    import nanovllm_amd as nva
    from nanovllm_amd.engine import SamplingParams, qwen3_0_6b
    from nanovllm_amd.engine.llm import LLM
    model = qwen3_0_6b()
    llm = LLM(model, enforce_eager=args.eager, max_model_len=4096, num_kvcache_blocks=4096, graph_bucket_step=args.bucket_step)
    prompts, params = e2e_workload(num_seqs=args.requests, max_output_len=args.max_output_len)
    total_out = sum(p.max_tokens for p in params)
    llm.generate([[1, 2, 3, 4]], SamplingParams(max_tokens=8, ignore_eos=True))     # reference warm-up call
    for w in range(args.warmup):
        llm.generate(fresh_prompts(prompts[:32], 9_000 + w), params[:32])
    mr = llm.model_runner
    mr.decode_step_events, kv_tokens0 = [], mr.kv_tokens_attended          # per-step HIP events from here on
    dt = _e2e_passes(llm, prompts, params, args.steps, 0)
    tok_s = total_out * args.steps / dt
    # what the decode steps of the timed passes really read: every step attends over sum(context_lens) tokens in
    # every layer (K and V rows of all kv heads); their GPU time is taken from a pair of events around every step
    decode_gpu_s = sum(a.elapsed_time(b) for a, b in mr.decode_step_events) * 1e-3
    n_decode_steps = len(mr.decode_step_events)
    mr.decode_step_events = None
    kv_bytes = (mr.kv_tokens_attended - kv_tokens0) * model.num_hidden_layers * model.num_key_value_heads * model.head_dim * 2 * 2

    layers = [m for m in llm.model_runner.model.modules() if isinstance(m, nva.Attention)]
    roof = decode_e2e_shape_roofline(dev, [(a.k_cache, a.v_cache) for a in layers], llm.config.num_kvcache_blocks)
    in_run_gbps = kv_bytes / decode_gpu_s / 1e9
    roof["in_run"] = {"what": "K/V bytes the decode steps of the timed passes attended over (sum of context_lens x layers x kv heads "
                              "x 128 x 2 B x 2) / GPU time of those steps (HIP events around every step: staging, 28 layers with "
                              "GEMMs, norms and attention, LM head, sampler) -- the whole step, not the attention kernel alone",
                      "kv_bytes_per_pass": kv_bytes // args.steps, "decode_steps_per_pass": n_decode_steps // args.steps,
                      "decode_gpu_s_per_pass": round(decode_gpu_s / args.steps, 4),
                      "mean_kv_bytes_per_attention_launch": kv_bytes // max(n_decode_steps * model.num_hidden_layers, 1),
                      "achieved": round(in_run_gbps, 1), "unit": "GB/s", "frac": round(in_run_gbps / HBM_PEAK_GBPS, 4)}
    st = dict(llm.stats)
    used, replayed = llm.model_runner.bucket_rows
    buckets = {"graph_bucket_step": llm.config.graph_bucket_step, "decode_rows_used": used, "decode_rows_replayed": replayed,
               "padded_fraction": round(1 - used / max(replayed, 1), 4)}
    del layers, llm, mr
    gc.collect()
    torch.cuda.empty_cache()
    result = {
        "metric": "output tok/s, Qwen3-0.6B bench shape; decode-attn HBM GB/s vs ~8 TB/s",
        "value": round(tok_s, 1), "unit": "tok/s", "ms_per_step": round(dt / args.steps * 1e3, 2),
        "config": {"workload": "e2e generate: Qwen3-0.6B architecture (28 layers, hidden 1024, 16q/8kv heads x 128, "
                               "MLP 3072, vocab 151936, random bf16 weights), 256 requests, prompt and output lengths "
                               "U[100,1024], temperature 0.6, ignore_eos, prompt ids drawn afresh for every pass, "
                               + ("eager" if args.eager else "hipGraph decode"),
                   "requests": args.requests, "output_tokens": total_out, "engine_steps_per_pass": (st["prefill_steps"] + st["decode_steps"]) // args.steps,
                   "prefill_s_per_pass": round(st["prefill_s"] / args.steps, 3), "decode_s_per_pass": round(st["decode_s"] / args.steps, 3),
                   "decode_buckets": buckets, "kv_bytes_per_pass": kv_bytes // args.steps},
        "roofline": roof,
    }
    if not args.no_extra:
        result["extra"] = collect_extra(dev, model, prompts, params)

    def cpu():
        from oracle import engine_cpu
        # the same mix at one eighth of the lengths (prompt and output alike, so the share of prefill
        # and decode work is the workload's), first 16 requests: what the host finishes in ~20 s
        short = [p[: max(1, len(p) // 8)] for p in prompts[:16]]
        sp = [SamplingParams(temperature=q.temperature, ignore_eos=True, max_tokens=max(1, q.max_tokens // 8)) for q in params[:16]]
        base = engine_cpu.baseline(model, short, sp, num_requests=16, max_new_tokens=1 << 30, budget_s=40.0)
        base["sample"] = "prompt and output lengths of the bench mix divided by 8: " + base["sample"]
        base.update(_cpu_cores())
        return base
    return result, cpu


def bench_longctx(args, dev):
    """Long-context decode stress (config 5): Qwen3-8B architecture, batch 128, contexts U[4096,16384],
    256-token KV blocks scattered randomly over a cache sized to the drawn contexts, 128 decode steps,
    even requests greedy and odd requests at temperature 1.0.  The prompts' KV is synthetic (the
    cache is filled with N(0,1) noise and the sequences are placed directly), so only the decode
    phase is run and timed; a step = one pass of 128 engine decode steps."""
    import random
    import torch
    from nanovllm_amd.engine import SamplingParams, Sequence, SequenceStatus, qwen3_8b
    from nanovllm_amd.engine.llm import LLM
    model = qwen3_8b()
    rng = random.Random(0)
    n_req, n_steps = args.requests if args.requests != 256 else 128, 128
    ctx = [rng.randint(4096, 16384) for _ in range(n_req)]
    need = sum(-(-(c + n_steps) // 256) for c in ctx)
    # (every request runs the same 128 steps, so only the full batch size is ever replayed: no intermediate graph buckets)
    llm = LLM(model, enforce_eager=args.eager, max_model_len=16384 + 256, max_num_batched_tokens=32768,
              max_num_seqs=n_req, num_kvcache_blocks=need + 8, graph_bucket_step=max(n_req, 1))
    mr, sch = llm.model_runner, llm.scheduler
    with torch.inference_mode():
        for l in range(model.num_hidden_layers):                 # synthetic KV content
            mr.kv_cache[0, l].normal_()
            mr.kv_cache[1, l].normal_()
    torch.cuda.synchronize()

    def place():
        free = list(range(llm.config.num_kvcache_blocks))
        rng.shuffle(free)                                        # blocks scattered randomly over the cache
        bm = sch.block_manager
        seqs = []
        for i, c in enumerate(ctx):
            s = Sequence([rng.randint(0, model.vocab_size - 1) for _ in range(c)],
                         SamplingParams(temperature=0.0 if i % 2 == 0 else 1.0, max_tokens=n_steps, ignore_eos=True))
            # the state a real prefill leaves behind: blocks for the first c-1 tokens (the scheduler adds the
            # block of the token being decoded), full blocks sealed with their chained hash
            for _ in range(-(-(c - 1) // 256)):
                blk = bm._take(free.pop())
                s.block_table.append(blk.block_id)
            for j in range((c - 1) // 256):
                blk = bm.blocks[s.block_table[j]]
                blk.hash = bm.compute_hash(s.block(j), bm.blocks[s.block_table[j - 1]].hash if j else -1)
                blk.token_ids = s.block(j)
            s.num_prompt_tokens = len(s)
            s.status = SequenceStatus.RUNNING
            sch.running.append(s)
            seqs.append(s)
        return seqs

    def one_pass():
        seqs = place()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        steps = 0
        while not llm.is_finished():
            llm.step()
            steps += 1
        torch.cuda.synchronize()
        assert steps in (n_steps, n_steps + 1) and all(s.num_completion_tokens == n_steps for s in seqs)   # +1: the last tokens are read back
        return time.perf_counter() - t0

    for _ in range(args.warmup):
        one_pass()
    dt = sum(one_pass() for _ in range(args.steps)) / args.steps
    tok_s = n_req * n_steps / dt
    kv_bytes_per_step = sum(c + n_steps // 2 for c in ctx) * model.num_hidden_layers * model.num_key_value_heads * model.head_dim * 2 * 2
    result = {
        "metric": "output tok/s, Qwen3-8B long-context decode (config 5)", "value": round(tok_s, 1), "unit": "tok/s",
        "ms_per_step": round(dt * 1e3, 2),
        "config": {"workload": "long-context decode: Qwen3-8B architecture (36 layers, hidden 4096, 32q/8kv heads x 128, "
                               "MLP 12288, random bf16 weights), batch %d, contexts U[4096,16384] (mean %d), synthetic KV in "
                               "%d randomly scattered 256-token blocks (%.1f GB cache), 128 decode steps, greedy + T=1.0, %s"
                               % (n_req, sum(ctx) // n_req, need, (need + 8) * 37.75e6 / 1e9,
                                  "eager" if args.eager else "hipGraph decode"),
                   "ms_per_decode_step": round(dt / n_steps * 1e3, 2), "kv_cache_blocks": need + 8,
                   "kv_cache_bytes": int(mr.kv_cache.numel()) * 2, "kv_bytes_per_decode_step": kv_bytes_per_step},
        "roofline": {"bound": "hbm", "achieved": round(kv_bytes_per_step / (dt / n_steps) / 1e9, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(kv_bytes_per_step / (dt / n_steps) / 1e9 / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "whole decode step (36 x decode_stream_kernel<4> dominate): KV bytes of one step / step time",
                     "algorithmic_bytes_per_launch": kv_bytes_per_step},
    }
    return result, (lambda: None)


WORKLOADS = {"rope-scatter": bench_rope_scatter, "glue": bench_glue, "e2e": bench_e2e, "longctx": bench_longctx, "decode-e2e-shape": bench_decode_e2e_shape,
             "decode-longctx-shape": bench_decode_longctx_shape, "copy": bench_copy, "read-probe": bench_read_probe, "decode": bench_decode, "scatter": bench_scatter, "prefill": bench_prefill, "sampler": bench_sampler}
DEFAULT_STEPS = {"rope-scatter": 100, "glue": 100, "e2e": 1, "longctx": 1, "decode-e2e-shape": 1, "decode-longctx-shape": 1, "copy": 50, "read-probe": 60, "decode": 200, "scatter": 400, "prefill": 50, "sampler": 100}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="e2e")
    ap.add_argument("--eager", action="store_true", help="e2e only: no hipGraph decode")
    ap.add_argument("--requests", type=int, default=256, help="e2e only: number of requests (profiling runs)")
    ap.add_argument("--max-output-len", type=int, default=1024, help="e2e only: cap on output lengths (profiling runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--grid-order", action="store_true", help="glue last-token-norm: norm every row, then gather (the reference's order) instead of the gathering kernel")
    ap.add_argument("--workspace", action="store_true", help="sampler: the two-kernel form with a workspace tensor (nva_sample) instead of nva_sample_static")
    ap.add_argument("--tokens", type=int, default=None, help="scatter / rope-scatter: number of tokens (default 4096 / 16384)")
    ap.add_argument("--contiguous", action="store_true", help="scatter: slots in ascending order instead of a random permutation")
    ap.add_argument("--noise", action="store_true", help="sampler: time the replayable path that reads an Exp(1) noise tensor")
    ap.add_argument("--glue", choices=["add-rms-norm", "silu-mul", "last-token-norm"], default="add-rms-norm", help="glue: which elementwise kernel")
    ap.add_argument("--uniform", default=None, metavar="SxL", help="prefill: S packed sequences of L tokens each instead of config 3 (e.g. 2x16384)")
    ap.add_argument("--bucket-step", type=int, default=16, help="e2e only: spacing of the captured decode batch sizes")
    ap.add_argument("--no-extra", action="store_true", help="e2e only: skip the per-configuration rooflines and the eager pass")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the hot path needs no collectives); "
                 "run with --gpus 1")
    if args.steps is None:
        args.steps = DEFAULT_STEPS[args.workload]
    if args.warmup is None:
        args.warmup = 1 if args.workload in ("e2e", "longctx") else max(3, args.steps // 10)

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible (the hot path has no CPU fallback)")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    from nanovllm_amd import _lib
    _lib.load()

    result, cpu_fn = WORKLOADS[args.workload](args, dev)
    line = {
        "metric": result["metric"], "value": result["value"], "unit": result["unit"],
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": result["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic", "config": result["config"], "roofline": result["roofline"],
    }
    if "extra" in result:
        line["extra"] = result["extra"]
    if not args.no_cpu_baseline:
        base = cpu_fn()
        if base is not None:
            line["cpu_baseline"] = base
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
