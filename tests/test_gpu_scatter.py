"""KV-cache slot scatter on the GPU, through the C ABI, bit-exact against the oracle."""
import pytest
import torch

import oracle
from nanovllm_amd import store_kvcache
from nanovllm_amd import synthetic
from helpers import bits

pytestmark = pytest.mark.gpu


def _run(case, dev):
    kc, vc = case.k_cache.to(dev), case.v_cache.to(dev)
    value = case.value
    if not value.is_contiguous():                      # keep the strided layout on the device
        base = value._base.to(dev)
        d = value.shape[1] * value.shape[2]
        value_d = base[:, base.shape[1] - d:].view(value.shape)
        assert value_d.stride() == value.stride()
    else:
        value_d = value.to(dev)
    store_kvcache(case.key.to(dev), value_d, kc, vc, case.slot_mapping.to(dev))
    torch.cuda.synchronize()
    ek, ev = case.k_cache.clone(), case.v_cache.clone()
    oracle.store_kvcache(case.key, case.value, ek, ev, case.slot_mapping)
    assert torch.equal(bits(kc), bits(ek)) and torch.equal(bits(vc), bits(ev))
    return kc, vc


@pytest.mark.parametrize("strided", [False, True])
def test_scatter_config1_bit_exact(dev, strided):
    """N=4096, 8 kv heads x 128, 512 blocks x 256 slots, 5% of the slots -1."""
    case = synthetic.scatter_case(seed=0, strided_value=strided)
    assert case.n_valid == 4096 - 205 and case.algorithmic_bytes == 31_891_456
    _run(case, dev)


@pytest.mark.parametrize("n,hkv", [(1, 8), (3, 2), (256, 8), (16384, 8), (77, 1), (5, 4)])
def test_scatter_ragged_sizes(dev, n, hkv):
    case = synthetic.scatter_case(seed=n, n_tokens=n, num_kv_heads=hkv, num_blocks=max(2, (n + 255) // 256 + 1))
    _run(case, dev)


def test_scatter_empty_and_all_skipped(dev):
    case = synthetic.scatter_case(seed=3, n_tokens=64, num_blocks=2, skip_fraction=1.0)
    kc, vc = _run(case, dev)
    assert not kc.any() and not vc.any()
    empty = torch.empty(0, 8, 128, dtype=torch.bfloat16, device=dev)
    store_kvcache(empty, empty, kc, vc, torch.empty(0, dtype=torch.int32, device=dev))
    torch.cuda.synchronize()
    assert not kc.any()


def test_scatter_duplicate_slots_are_safe(dev):
    """Graph capture runs with slot_mapping == 0 for every row: no fault, slot 0 holds
    pieces of the competing rows, everything else untouched."""
    case = synthetic.scatter_case(seed=4, n_tokens=128, num_blocks=2, skip_fraction=0.0)
    kc, vc = case.k_cache.to(dev), case.v_cache.to(dev)
    store_kvcache(case.key.to(dev), case.value.to(dev), kc, vc, torch.zeros(128, dtype=torch.int32, device=dev))
    torch.cuda.synchronize()
    assert not kc.view(-1, 1024)[1:].any() and not vc.view(-1, 1024)[1:].any()
    # rows race chunk by chunk: every 16-byte chunk of slot 0 is the same chunk of SOME token
    got = bits(kc.view(-1, 1024)[0]).view(128, 8)
    src = bits(case.key.reshape(128, 1024)).view(128, 128, 8)          # [token, chunk, 8]
    assert bool((got.unsqueeze(0) == src).all(-1).any(0).all())


def test_scatter_out_of_range_slots_are_skipped(dev):
    case = synthetic.scatter_case(seed=5, n_tokens=32, num_blocks=1, skip_fraction=0.0)
    slots = case.slot_mapping.clone()
    slots[::2] = 256 + 7            # beyond the single block
    kc, vc = case.k_cache.to(dev), case.v_cache.to(dev)
    store_kvcache(case.key.to(dev), case.value.to(dev), kc, vc, slots.to(dev))
    torch.cuda.synchronize()
    ek, ev = case.k_cache.clone(), case.v_cache.clone()
    keep = slots.clone()
    keep[::2] = -1
    oracle.store_kvcache(case.key, case.value, ek, ev, keep)
    assert torch.equal(bits(kc), bits(ek)) and torch.equal(bits(vc), bits(ev))


def test_calibration_read_touches_nothing(dev):
    """nva_probe_stream_read only reads: the source is unchanged and the sink keeps its value."""
    from nanovllm_amd import _lib
    lib = _lib.load()
    src = torch.randint(0, 255, (3 * 1024 * 1024 + 48,), dtype=torch.uint8, device=dev)
    before = src.clone()
    sink = torch.full((4,), 7, dtype=torch.int32, device=dev)
    for nbytes in (16, 4096 + 16, src.numel()):
        rc = lib.nva_probe_stream_read(src.data_ptr(), nbytes, sink.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert rc == _lib.OK
    torch.cuda.synchronize()
    assert torch.equal(src, before) and sink.tolist() == [7] * 4
