"""The sampler entry point that allocates nothing (nva_sample_static) against nva_sample.

Called through the C ABI with caller-owned inputs and outputs only.  Both entry points run the same
kernels, so for the same (seed, offset) -- or the same noise tensor -- the tokens must be identical.
Two calls in a row on the shared built-in scratch array, the second on a smaller problem."""
import pytest
import torch

from nanovllm_amd import _lib

pytestmark = pytest.mark.gpu


def _both(dev, batch, vocab, with_noise, seed, offset, temperature=0.6):
    lib = _lib.load()
    g = torch.Generator().manual_seed(batch * 1000 + vocab)
    logits = (torch.randn(batch, vocab, generator=g) * 2).to(torch.bfloat16).to(dev)
    temps = torch.full((batch,), temperature, device=dev)
    temps[::5] = 0.0                                                     # some greedy rows
    noise = torch.empty(batch, vocab).exponential_(1.0, generator=g).to(dev) if with_noise else None
    out_ws = torch.full((batch,), -1, dtype=torch.int64, device=dev)
    out_static = torch.full((batch,), -2, dtype=torch.int64, device=dev)
    ws = torch.empty(lib.nva_sample_workspace_bytes(batch, vocab), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    nptr, nstride = (noise.data_ptr(), noise.stride(0)) if with_noise else (None, 0)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    rc = lib.nva_sample_static(logits.data_ptr(), logits.stride(0), temps.data_ptr(), nptr, nstride, seed, offset,
                               out_static.data_ptr(), batch, vocab, stream)
    assert rc == _lib.OK, _lib.status_string(rc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before                    # (torch's allocator was not involved either)
    rc = lib.nva_sample(logits.data_ptr(), logits.stride(0), temps.data_ptr(), nptr, nstride, seed, offset,
                        out_ws.data_ptr(), ws.data_ptr(), ws.numel(), batch, vocab, stream)
    assert rc == _lib.OK, _lib.status_string(rc)
    torch.cuda.synchronize()
    assert torch.equal(out_static, out_ws), (out_static, out_ws)
    assert int(out_static.min()) >= 0 and int(out_static.max()) < vocab
    greedy = logits.float().argmax(-1)
    assert torch.equal(out_static[::5], greedy[::5])
    return out_static.cpu()


@pytest.mark.parametrize("with_noise", [False, True])
def test_sample_static_matches_sample_on_two_calls_in_a_row(dev, with_noise):
    big = _both(dev, 256, 151936, with_noise, seed=17, offset=3)          # up to 256 x 75 records of the scratch array
    small = _both(dev, 7, 5000, with_noise, seed=17, offset=4)            # then 7 records: stale ones beyond must not matter
    again = _both(dev, 256, 151936, with_noise, seed=17, offset=3)
    assert torch.equal(big, again) and small.numel() == 7


def test_sample_static_takes_no_device_memory_and_replays_from_a_graph(dev):
    """After a first call has looked the scratch array up: (1) the free device memory the driver
    reports is the same before and after a call -- the caching allocator's own counter would not see
    a hipMalloc inside the library; (2) the call can be captured in a HIP graph, and every replay, on
    new logits and with eager work and synchronisation in between, gives what nva_sample gives."""
    lib = _lib.load()
    batch, vocab, seed, offset = 64, 151936, 5, 9
    g = torch.Generator().manual_seed(123)
    logits = (torch.randn(batch, vocab, generator=g) * 2).to(torch.bfloat16).to(dev)
    temps = torch.full((batch,), 0.8, device=dev)
    out = torch.full((batch,), -1, dtype=torch.int64, device=dev)
    want = torch.full((batch,), -2, dtype=torch.int64, device=dev)
    ws = torch.empty(lib.nva_sample_workspace_bytes(batch, vocab), dtype=torch.uint8, device=dev)

    def static_call():
        rc = lib.nva_sample_static(logits.data_ptr(), logits.stride(0), temps.data_ptr(), None, 0, seed, offset,
                                   out.data_ptr(), batch, vocab, torch.cuda.current_stream().cuda_stream)
        assert rc == _lib.OK, _lib.status_string(rc)

    def eager_reference():
        rc = lib.nva_sample(logits.data_ptr(), logits.stride(0), temps.data_ptr(), None, 0, seed, offset,
                            want.data_ptr(), ws.data_ptr(), ws.numel(), batch, vocab,
                            torch.cuda.current_stream().cuda_stream)
        assert rc == _lib.OK, _lib.status_string(rc)

    static_call()                                                        # warm: address look-up, code object load
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    static_call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free_before

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_call()
    seen = set()
    for replay in range(4):
        logits.copy_((torch.randn(batch, vocab, generator=g) * 2).to(torch.bfloat16))
        out.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        eager_reference()                                                # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(out, want), replay
        assert int(out.min()) >= 0 and int(out.max()) < vocab
        seen.add(tuple(out[:8].tolist()))
    assert len(seen) == 4                                                # the replays really saw different logits


def test_sample_static_rejects_what_does_not_fit(dev):
    """Inputs and outputs are real tensors: a library that wrongly accepted the call would still touch only memory it may."""
    lib = _lib.load()
    batch, vocab = 1748, 151936                                           # 1748 * 75 records of 2048 columns > 131072
    logits = torch.zeros(batch, vocab, dtype=torch.bfloat16, device=dev)
    temps = torch.ones(batch, device=dev)
    out = torch.full((batch,), -5, dtype=torch.int64, device=dev)
    rc = lib.nva_sample_static(logits.data_ptr(), vocab, temps.data_ptr(), None, 0, 0, 0, out.data_ptr(), batch, vocab,
                               torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.ERR_SCRATCH_TOO_SMALL and "scratch" in _lib.status_string(rc)
    torch.cuda.synchronize()
    assert bool((out == -5).all())                                        # nothing was launched
    rc = lib.nva_sample_static(logits.data_ptr(), vocab, temps.data_ptr(), None, 0, 0, 0, out.data_ptr(), 1747, vocab,
                               torch.cuda.current_stream().cuda_stream)   # the largest batch that fits
    assert rc == _lib.OK
    torch.cuda.synchronize()
    assert bool((out[:1747] >= 0).all()) and bool((out[:1747] < vocab).all()) and int(out[1747]) == -5
