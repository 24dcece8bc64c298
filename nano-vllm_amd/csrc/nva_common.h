// Shared device/host helpers for the gfx950 hot-path kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nanovllm_amd.h"

namespace nva {

constexpr int kHeadDim = 128;    // the only head_dim the kernels are built for
constexpr int kBlockSize = 256;  // smallest KV block, in tokens (nanovllm/config.py:17,22: multiples of 256)
constexpr int kWave = 64;        // CDNA wavefront width

using bf16_t = uint16_t;         // raw bf16 bits

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(static_cast<uint32_t>(v) << 16);
}
// low / high half of a packed pair of bf16
__device__ __forceinline__ float bf16lo_to_f32(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }

// fp32 -> bf16, round to nearest even (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    return __builtin_bit_cast(unsigned short, static_cast<__bf16>(f));
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const bf16x2_t v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ void unpack8(const uint4 &r, float (&f)[8]) {
    f[0] = bf16lo_to_f32(r.x); f[1] = bf16hi_to_f32(r.x);
    f[2] = bf16lo_to_f32(r.y); f[3] = bf16hi_to_f32(r.y);
    f[4] = bf16lo_to_f32(r.z); f[5] = bf16hi_to_f32(r.z);
    f[6] = bf16lo_to_f32(r.w); f[7] = bf16hi_to_f32(r.w);
}

// ---- cross-lane helpers (DPP: no LDS traffic) ------------------------------------------
template <int kCtrl>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xf, 0xf, true));
}
// sum over each aligned group of 16 lanes, result in all 16 lanes
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);  // row_half_mirror
    v += dpp_f32<0x140>(v);  // row_mirror
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    v = fmaxf(v, dpp_f32<0x140>(v));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    v = row16_max(v);
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

// log2 of a KV block size the kernels are built for (256, 512, 1024, 2048, 4096 tokens), else -1
inline int block_shift_of(int32_t block_size) {
    for (int sh = 8; sh <= 12; ++sh)
        if (block_size == (1 << sh)) return sh;
    return -1;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int launch_status() {
    return hipGetLastError() == hipSuccess ? NVA_OK : NVA_ERR_LAUNCH_FAILED;
}

}  // namespace nva
