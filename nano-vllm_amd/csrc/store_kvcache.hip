// KV-cache slot scatter for gfx950.
//
// Replaces the Triton store_kvcache_kernel of nanovllm/layers/attention.py:10-30: token row
// i (D = num_kv_heads*head_dim bf16 elements of K and of V) is copied bit-exactly to row
// slot_mapping[i] of the flat caches; slot -1 skips the row.
//
// Layout / mapping: one workgroup of 256 lanes per token.  A row is D*2/16 16-byte chunks
// (128 for D = 1024); lanes 0..127 copy the K chunks and lanes 128..255 the V chunks, so each
// (token, head) row of 256 B is written by 16 consecutive lanes, one dwordx4 store per lane.  The kernel
// is pure HBM traffic: D*2 B read + D*2 B written per tensor per stored token.
#include "nva_common.h"

namespace nva {

__global__ __launch_bounds__(256) void store_kvcache_kernel(
    const uint4 *__restrict__ key, int64_t key_stride16,      // row strides in 16-byte units
    const uint4 *__restrict__ value, int64_t value_stride16,
    uint4 *__restrict__ k_cache, uint4 *__restrict__ v_cache,
    const int32_t *__restrict__ slot_mapping, int32_t chunks_per_row, int64_t num_slots) {
    const int64_t token = blockIdx.x;
    const int64_t slot = slot_mapping[token];
    if (slot < 0 || slot >= num_slots) return;   // -1 = skip (attention.py:22); never write OOB
    const uint4 *ksrc = key + token * key_stride16;
    const uint4 *vsrc = value + token * value_stride16;
    uint4 *kdst = k_cache + slot * chunks_per_row;
    uint4 *vdst = v_cache + slot * chunks_per_row;
    // lanes [0, chunks) move K, lanes [chunks, 2*chunks) move V: wave-uniform for D = 1024
    for (int c = threadIdx.x; c < 2 * chunks_per_row; c += blockDim.x) {
        const bool is_v = c >= chunks_per_row;
        const int cc = is_v ? c - chunks_per_row : c;
        const uint4 row = is_v ? vsrc[cc] : ksrc[cc];
        (is_v ? vdst : kdst)[cc] = row;
    }
}

}  // namespace nva

extern "C" int nva_store_kvcache(const void *key, int64_t key_row_stride,
                                 const void *value, int64_t value_row_stride,
                                 void *k_cache, void *v_cache, const int32_t *slot_mapping,
                                 int32_t n_tokens, int32_t num_kv_heads, int32_t head_dim,
                                 int64_t num_slots, void *stream) {
    if (n_tokens < 0 || num_kv_heads <= 0 || head_dim <= 0 || num_slots < 0) return NVA_ERR_BAD_SHAPE;
    if (n_tokens == 0) return NVA_OK;
    if (!key || !value || !k_cache || !v_cache || !slot_mapping) return NVA_ERR_NULL_POINTER;
    const int64_t d = static_cast<int64_t>(num_kv_heads) * head_dim;
    if (head_dim % 8 != 0) return NVA_ERR_UNSUPPORTED_GEOMETRY;       // 16-byte chunks per head row
    if (key_row_stride < d || value_row_stride < d) return NVA_ERR_BAD_STRIDE;
    if (key_row_stride % 8 != 0 || value_row_stride % 8 != 0) return NVA_ERR_BAD_STRIDE;
    if (!nva::aligned16(key) || !nva::aligned16(value) || !nva::aligned16(k_cache) ||
        !nva::aligned16(v_cache))
        return NVA_ERR_MISALIGNED;
    const int32_t chunks = static_cast<int32_t>(d / 8);
    hipLaunchKernelGGL(nva::store_kvcache_kernel, dim3(n_tokens), dim3(256), 0,
                       static_cast<hipStream_t>(stream),
                       static_cast<const uint4 *>(key), key_row_stride / 8,
                       static_cast<const uint4 *>(value), value_row_stride / 8,
                       static_cast<uint4 *>(k_cache), static_cast<uint4 *>(v_cache),
                       slot_mapping, chunks, num_slots);
    return nva::launch_status();
}
