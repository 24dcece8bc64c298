// Library-level entry points of the C ABI: version, status strings, device probe.
#include "nva_common.h"

extern "C" int nva_version(void) { return (0 << 16) | 1; }

extern "C" const char *nva_status_string(int status) {
    switch (status) {
        case NVA_OK: return "ok";
        case NVA_ERR_NULL_POINTER: return "null pointer";
        case NVA_ERR_BAD_SHAPE: return "bad shape";
        case NVA_ERR_UNSUPPORTED_GEOMETRY: return "unsupported geometry (head_dim 128, block_size 256 * 2^k up to 4096, GQA group 1 to 8 only)";
        case NVA_ERR_BAD_STRIDE: return "bad stride";
        case NVA_ERR_MISALIGNED: return "pointer not 16-byte aligned";
        case NVA_ERR_WORKSPACE_TOO_SMALL: return "workspace too small";
        case NVA_ERR_LAUNCH_FAILED: return "kernel launch failed";
        case NVA_ERR_NO_DEVICE: return "no HIP device";
        case NVA_ERR_SCRATCH_TOO_SMALL: return "problem exceeds the built-in scratch array";
        default: return "unknown status";
    }
}

extern "C" int nva_device_count(int *count) {
    if (!count) return NVA_ERR_NULL_POINTER;
    int n = 0;
    const hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        (void)hipGetLastError();   // do not leave a sticky error for the next call
        *count = 0;
        return NVA_ERR_NO_DEVICE;
    }
    *count = n;
    return NVA_OK;
}
