"""ctypes binding of the C ABI declared in include/nanovllm_amd.h.

The shared library is built in-tree (``libnanovllm_amd.so`` next to this file) by
``csrc/Makefile``.  There is no fallback: if the library is missing every op raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnanovllm_amd.so")

# status codes of enum nva_status
OK = 0
ERR_NULL_POINTER = 1
ERR_BAD_SHAPE = 2
ERR_UNSUPPORTED_GEOMETRY = 3
ERR_BAD_STRIDE = 4
ERR_MISALIGNED = 5
ERR_WORKSPACE_TOO_SMALL = 6
ERR_LAUNCH_FAILED = 7
ERR_NO_DEVICE = 8
ERR_SCRATCH_TOO_SMALL = 9

_vp, _i32, _i64, _u64, _f32, _sz = C.c_void_p, C.c_int32, C.c_int64, C.c_uint64, C.c_float, C.c_size_t

# name -> (restype, argtypes); must list every symbol the header declares
SIGNATURES = {
    "nva_version": (C.c_int, []),
    "nva_status_string": (C.c_char_p, [C.c_int]),
    "nva_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "nva_store_kvcache": (C.c_int, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _i64, _vp]),
    "nva_paged_decode_workspace_bytes": (_sz, [_i32, _i32, _i32, _i32]),
    "nva_paged_decode_attn": (C.c_int, [_vp, _i64, _vp, _vp, _vp, _i32, _i32, _vp, _vp, _vp, _sz,
                                        _i32, _i32, _i32, _i32, _i32, _i32, _f32, _vp]),
    "nva_paged_decode_attn_planned": (C.c_int, [_vp, _i64, _vp, _vp, _vp, _i32, _i32, _vp, _vp, _vp, _sz,
                                                _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp]),
    "nva_varlen_prefill_attn": (C.c_int, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _i32, _i32,
                                          _vp, _vp, _i32, _i32, _i32, _vp, _i32, _i32, _i32, _i32, _i32,
                                          _f32, _vp]),
    "nva_sample_workspace_bytes": (_sz, [_i32, _i32]),
    "nva_rms_norm": (C.c_int, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _i32, _i32, _f32, _vp]),
    "nva_gather_last_rms_norm": (C.c_int, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _f32, _vp]),
    "nva_qk_norm_rope": (C.c_int, [_vp, _i64, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _i64,
                                   _i32, _i32, _i32, _i32, _f32, _vp]),
    "nva_silu_and_mul": (C.c_int, [_vp, _i64, _vp, _i32, _i32, _vp]),
    "nva_stage_decode_inputs": (C.c_int, [_vp, _vp, _i64, _i64, _i64, _i32, _vp, _i32, _vp]),
    "nva_sample": (C.c_int, [_vp, _i64, _vp, _vp, _i64, _u64, _u64, _vp, _vp, _sz, _i32, _i32, _vp]),
    "nva_sample_static": (C.c_int, [_vp, _i64, _vp, _vp, _i64, _u64, _u64, _vp, _i32, _i32, _vp]),
    "nva_probe_stream_read": (C.c_int, [_vp, _i64, _vp, _vp]),
}

_lib = None


class HipLibraryMissing(RuntimeError):
    pass


def load():
    """Load the library once; raise loudly when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HipLibraryMissing(
                f"{LIB_PATH} not found: build it with `make -C nano-vllm_amd/csrc` "
                "(or __graft_entry__.build()); there is no CPU fallback")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def status_string(code: int) -> str:
    return load().nva_status_string(int(code)).decode()


def check(code: int, what: str) -> None:
    if code != OK:
        raise RuntimeError(f"{what}: {status_string(code)} (nva_status {code})")
