"""Host-side checks of the C ABI that need no GPU: the library loads, exports every symbol
the header declares, and rejects bad arguments before any launch."""
import ctypes as C
import os
import re

import pytest
import torch

from nanovllm_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "nanovllm_amd.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nva_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 9
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names


def test_version_and_status_strings():
    lib = _lib.load()
    assert lib.nva_version() >= 1
    seen = {_lib.status_string(c) for c in range(10)}
    assert len(seen) == 10 and _lib.status_string(0) == "ok"
    assert _lib.status_string(1234) == "unknown status"


def test_device_count_reports_no_device_cleanly():
    lib = _lib.load()
    n = C.c_int(-1)
    rc = lib.nva_device_count(C.byref(n))
    if torch.cuda.is_available():
        assert rc == _lib.OK and n.value >= 1
    else:
        assert rc == _lib.ERR_NO_DEVICE and n.value == 0
    assert lib.nva_device_count(None) == _lib.ERR_NULL_POINTER


A = 0x1000   # a fake, 16-byte aligned address: validation fails before anything dereferences it


def test_store_kvcache_validation():
    f = _lib.load().nva_store_kvcache
    assert f(None, 1024, A, 1024, A, A, A, 4, 8, 128, 512, None) == _lib.ERR_NULL_POINTER
    assert f(A, 1024, A, 1024, A, A, None, 4, 8, 128, 512, None) == _lib.ERR_NULL_POINTER
    assert f(A, 1024, A, 1024, A, A, A, -1, 8, 128, 512, None) == _lib.ERR_BAD_SHAPE
    assert f(A, 1000, A, 1024, A, A, A, 4, 8, 128, 512, None) == _lib.ERR_BAD_STRIDE     # stride < row
    assert f(A, 1024, A, 4100, A, A, A, 4, 8, 128, 512, None) == _lib.ERR_BAD_STRIDE     # not 16-byte rows
    assert f(A + 2, 1024, A, 1024, A, A, A, 4, 8, 128, 512, None) == _lib.ERR_MISALIGNED
    assert f(A, 1024, A, 1024, A, A, A, 4, 8, 100, 512, None) == _lib.ERR_UNSUPPORTED_GEOMETRY
    assert f(None, 0, None, 0, None, None, None, 0, 8, 128, 512, None) == _lib.OK        # empty batch


def test_decode_validation_and_workspace_size():
    lib = _lib.load()
    ws = lib.nva_paged_decode_workspace_bytes
    # prefix sums and context lengths (each 256-byte aligned) + a 32-byte record per worker + 8 bytes per
    # (sequence, head) pair (256-byte aligned) + (2048 wavefronts * min(heads, 8) + 4 * batch * heads) partial rows of 130 floats
    assert ws(64, 16, 128, 8) == 512 + 256 + 2048 * 32 + 64 * 16 * 8 + (2048 * 8 + 4 * 64 * 16) * 130 * 4
    assert ws(3, 2, 128, 1) == 256 + 256 + 2048 * 32 + 256 + (2048 * 2 + 4 * 3 * 2) * 130 * 4
    assert ws(0, 16, 128, 8) == 0
    f = lib.nva_paged_decode_attn
    ok = dict(q=A, qs=2048, kc=A, vc=A, bt=A, bts=8, mb=8, cl=A, out=A, ws=A, wsb=ws(4, 16, 128, 8),
              b=4, hq=16, hkv=8, dh=128, bs=256, nb=64, scale=0.088, stream=None)

    def call(**kw):
        a = dict(ok, **kw)
        return f(a["q"], a["qs"], a["kc"], a["vc"], a["bt"], a["bts"], a["mb"], a["cl"], a["out"], a["ws"],
                 a["wsb"], a["b"], a["hq"], a["hkv"], a["dh"], a["bs"], a["nb"], a["scale"], a["stream"])

    assert call(q=None) == _lib.ERR_NULL_POINTER
    assert call(bt=None) == _lib.ERR_NULL_POINTER
    assert call(dh=64) == _lib.ERR_UNSUPPORTED_GEOMETRY
    assert call(bs=128) == _lib.ERR_UNSUPPORTED_GEOMETRY
    assert call(bs=768) == _lib.ERR_UNSUPPORTED_GEOMETRY             # blocks of 256 * 2^k tokens only
    assert call(hq=72, hkv=8) == _lib.ERR_UNSUPPORTED_GEOMETRY        # group 9 (1 to 8 are built)
    assert call(hq=16, hkv=3) == _lib.ERR_UNSUPPORTED_GEOMETRY
    assert call(qs=1024) == _lib.ERR_BAD_STRIDE
    assert call(bts=4) == _lib.ERR_BAD_STRIDE
    assert call(ws=A + 4) == _lib.ERR_MISALIGNED
    assert call(wsb=ok["wsb"] - 1) == _lib.ERR_WORKSPACE_TOO_SMALL
    assert call(b=-2) == _lib.ERR_BAD_SHAPE
    assert call(b=0) == _lib.OK
    g = lib.nva_paged_decode_attn_planned
    a = ok
    args = [a["q"], a["qs"], a["kc"], a["vc"], a["bt"], a["bts"], a["mb"], a["cl"], a["out"], a["ws"], a["wsb"],
            a["b"], a["hq"], a["hkv"], a["dh"], a["bs"], a["nb"], a["scale"]]
    assert g(*args, 2, None) == _lib.ERR_BAD_SHAPE                    # neither build nor reuse
    assert g(*(args[:11] + [0] + args[12:]), 1, None) == _lib.OK      # empty batch
    assert g(*(args[:9] + [A + 4] + args[10:]), 1, None) == _lib.ERR_MISALIGNED


def test_prefill_validation():
    f = _lib.load().nva_varlen_prefill_attn
    ok = dict(q=A, qs=2048, k=A, ks=1024, v=A, vs=4096, kc=None, vc=None, bt=None, bts=0, mb=0, cq=A, ck=A,
              b=2, mq=100, mk=100, out=A, hq=16, hkv=8, dh=128, bs=256, nb=0, scale=0.088, stream=None)

    def call(**kw):
        a = dict(ok, **kw)
        return f(a["q"], a["qs"], a["k"], a["ks"], a["v"], a["vs"], a["kc"], a["vc"], a["bt"], a["bts"], a["mb"],
                 a["cq"], a["ck"], a["b"], a["mq"], a["mk"], a["out"], a["hq"], a["hkv"], a["dh"], a["bs"],
                 a["nb"], a["scale"], a["stream"])

    assert call(q=None) == _lib.ERR_NULL_POINTER
    assert call(k=None) == _lib.ERR_NULL_POINTER                       # packed mode needs k/v
    assert call(cq=None) == _lib.ERR_NULL_POINTER
    assert call(dh=256) == _lib.ERR_UNSUPPORTED_GEOMETRY
    assert call(vs=1000) == _lib.ERR_BAD_STRIDE
    assert call(out=A + 8) == _lib.ERR_MISALIGNED
    paged = dict(k=None, v=None, kc=A, vc=A, bt=A, bts=4, mb=4, nb=32)
    assert call(**dict(paged, kc=None)) == _lib.ERR_NULL_POINTER
    assert call(**dict(paged, bs=768)) == _lib.ERR_UNSUPPORTED_GEOMETRY   # blocks of 256 * 2^k tokens only
    assert call(**dict(paged, bts=2)) == _lib.ERR_BAD_STRIDE
    assert call(**dict(paged, mk=4 * 256 + 1)) == _lib.ERR_BAD_SHAPE   # table too narrow for max_seqlen_k
    assert call(b=0) == _lib.OK and call(mq=0) == _lib.OK


def test_sampler_validation_and_workspace_size():
    lib = _lib.load()
    ws = lib.nva_sample_workspace_bytes
    assert ws(256, 151936) == 256 * 75 * 16 and ws(1, 1) == 16 and ws(2, 2049) == 64 and ws(0, 10) == 0   # one 16-byte record per 2048-column chunk
    f = lib.nva_sample
    assert f(None, 100, A, None, 0, 0, 0, A, A, 1 << 20, 4, 100, None) == _lib.ERR_NULL_POINTER
    assert f(A, 100, A, None, 0, 0, 0, A, None, 1 << 20, 4, 100, None) == _lib.ERR_NULL_POINTER
    assert f(A, 99, A, None, 0, 0, 0, A, A, 1 << 20, 4, 100, None) == _lib.ERR_BAD_STRIDE
    assert f(A, 100, A, A, 50, 0, 0, A, A, 1 << 20, 4, 100, None) == _lib.ERR_BAD_STRIDE
    assert f(A, 100, A, None, 0, 0, 0, A, A, 8, 4, 100, None) == _lib.ERR_WORKSPACE_TOO_SMALL
    assert f(A, 100, A, None, 0, 0, 0, A, A, 1 << 20, 4, 0, None) == _lib.ERR_BAD_SHAPE
    assert f(A, 100, A, None, 0, 0, 0, A, A, 1 << 20, 0, 100, None) == _lib.OK


def test_gather_last_rms_norm_validation():
    f = _lib.load().nva_gather_last_rms_norm
    assert f(None, 1024, A, 1024, A, A, A, 4, 100, 1024, 1e-6, None) == _lib.ERR_NULL_POINTER
    assert f(A, 1024, A, 1024, None, A, A, 4, 100, 1024, 1e-6, None) == _lib.ERR_NULL_POINTER    # cu_seqlens_q
    assert f(A, 1024, A, 1024, A, A, None, 4, 100, 1024, 1e-6, None) == _lib.ERR_NULL_POINTER    # out
    assert f(A, 1024, A, 1024, A, A, A, -1, 100, 1024, 1e-6, None) == _lib.ERR_BAD_SHAPE
    assert f(A, 1024, A, 1024, A, A, A, 4, 0, 1024, 1e-6, None) == _lib.ERR_BAD_SHAPE            # rows to pick from nothing
    assert f(A, 1000, A, 1024, A, A, A, 4, 100, 1024, 1e-6, None) == _lib.ERR_BAD_STRIDE
    assert f(A, 1024, A, 1028, A, A, A, 4, 100, 1024, 1e-6, None) == _lib.ERR_BAD_STRIDE
    assert f(A + 4, 1024, A, 1024, A, A, A, 4, 100, 1024, 1e-6, None) == _lib.ERR_MISALIGNED
    assert f(A, 1024, A, 1024, A, A, A, 4, 100, 1020, 1e-6, None) == _lib.ERR_UNSUPPORTED_GEOMETRY
    assert f(A, 8192, A, 8192, A, A, A, 4, 100, 8192, 1e-6, None) == _lib.ERR_UNSUPPORTED_GEOMETRY
    assert f(None, 0, None, 0, None, None, None, 0, 0, 1024, 1e-6, None) == _lib.OK               # empty batch


def test_stage_decode_inputs_validation():
    f = _lib.load().nva_stage_decode_inputs
    # (dst, src_host, nbytes, ids_offset, index_offset, n, prev_tokens, n_prev, stream)
    assert f(None, A, 4096, 0, 2048, 16, None, 0, None) == _lib.ERR_NULL_POINTER
    assert f(A, A, 4096, 0, 2048, 16, None, 4, None) == _lib.ERR_NULL_POINTER               # tokens announced, none given
    assert f(A, A, 4100, 0, 2048, 16, None, 0, None) == _lib.ERR_MISALIGNED                 # whole 16-byte chunks only
    assert f(A, A, 4096, 8, 2048, 16, None, 0, None) == _lib.ERR_MISALIGNED
    assert f(A + 8, A, 4096, 0, 2048, 16, None, 0, None) == _lib.ERR_MISALIGNED
    assert f(A, A, 4096, 0, 2048, 1024, None, 0, None) == _lib.ERR_BAD_SHAPE                # ids run past the buffer
    assert f(A, A, 4096, 0, 4090, 16, None, 0, None) == _lib.ERR_MISALIGNED
    assert f(A, A, 4096, 0, 4092, 16, None, 0, None) == _lib.ERR_BAD_SHAPE                  # index runs past the buffer
    assert f(A, A, -16, 0, 0, 0, None, 0, None) == _lib.ERR_BAD_SHAPE
    assert f(None, None, 0, 0, 0, 0, None, 0, None) == _lib.OK                              # nothing to move


def test_python_wrappers_refuse_cpu_tensors_and_keep_reference_asserts():
    import nanovllm_amd as nva
    k = torch.zeros(4, 8, 128, dtype=torch.bfloat16)
    cache = torch.zeros(2, 256, 8, 128, dtype=torch.bfloat16)
    slots = torch.arange(4, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="GPU only"):
        nva.store_kvcache(k, k, cache, cache, slots)
    with pytest.raises(AssertionError):                                # slot_mapping.numel() == N
        nva.store_kvcache(k, k, cache, cache, slots[:3])
    with pytest.raises(AssertionError):                                # stride(1) == head_dim
        nva.store_kvcache(k.transpose(1, 2).contiguous().transpose(1, 2), k, cache, cache, slots)
    with pytest.raises(RuntimeError, match="GPU only"):
        nva.sample(torch.zeros(2, 10, dtype=torch.bfloat16), torch.ones(2))


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libnanovllm_amd.so")
    with pytest.raises(_lib.HipLibraryMissing, match="no CPU fallback"):
        _lib.load()


def test_sample_static_validation():
    """The allocation-free sampler rejects bad arguments and problems beyond its built-in scratch
    array before it touches a device."""
    f = _lib.load().nva_sample_static
    # (logits, row_stride, temperatures, noise, noise_stride, seed, offset, out_tokens, batch, vocab, stream)
    assert f(None, 100, A, None, 0, 0, 0, A, 4, 100, None) == _lib.ERR_NULL_POINTER
    assert f(A, 99, A, None, 0, 0, 0, A, 4, 100, None) == _lib.ERR_BAD_STRIDE
    assert f(A, 100, A, None, 0, 0, 0, A, 4, 0, None) == _lib.ERR_BAD_SHAPE
    assert f(A, 100, A, None, 0, 0, 0, A, 0, 100, None) == _lib.OK
    assert f(A, 151936, A, None, 0, 0, 0, A, 1748, 151936, None) == _lib.ERR_SCRATCH_TOO_SMALL    # 1748 * 75 records > 131072
    assert f(A, 1 << 29, A, None, 0, 0, 0, A, 1, 1 << 29, None) == _lib.ERR_SCRATCH_TOO_SMALL     # 262144 records


def test_probe_validation():
    """The calibration read rejects bad arguments before any launch."""
    f = _lib.load().nva_probe_stream_read
    # (src, nbytes, sink, stream)
    assert f(None, 1024, A, None) == _lib.ERR_NULL_POINTER
    assert f(A, 1024, None, None) == _lib.ERR_NULL_POINTER
    assert f(A + 8, 1024, A, None) == _lib.ERR_MISALIGNED
    assert f(A, 1000, A, None) == _lib.ERR_MISALIGNED               # not a multiple of 16
    assert f(A, -16, A, None) == _lib.ERR_BAD_SHAPE
    assert f(A, 0, A, None) == _lib.OK                               # nothing to read
