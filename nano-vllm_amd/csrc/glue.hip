// Fused element-wise steps that sit between the GEMMs and the attention hot path.
//
// They replace the torch.compile'd fusions of the reference:
//   rms_norm / add_rms_norm   nanovllm/layers/layernorm.py:16-40
//   qk_norm_rope              nanovllm/models/qwen3.py:76-79 (per-head RMSNorm of q and k)
//                             + nanovllm/layers/rotary_embedding.py:6-48 (neox rotation)
//   silu_and_mul              nanovllm/layers/activation.py:11-14
// and keep the reference's rounding points: fp32 math, one rounding to bf16 after the
// normalisation, a bf16 multiply by the bf16 weight, fp32 rotation of the rounded values.
// All three are pure HBM traffic: every input element is read once, every output written once.
#include "nva_common.h"

#include <math.h>

namespace nva {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kNormMaxChunks = 8;     // 8 x (64 lanes x 8 elements) = hidden sizes up to 4096

__device__ __forceinline__ float round_bf16(float v) { return bf16_to_f32(f32_to_bf16(v)); }

// One wavefront per row, the row lives in registers between the two passes.  NC = chunks of 512
// elements per row; every load of the row (input, residual and weight) is issued before the first
// use, so the kernel costs one memory round trip instead of one per chunk and tensor.
// kResidual false: out = bf16(x * rsqrt(mean(x^2) + eps)) * w
// else:            s = x + residual (fp32); residual_out = bf16(s); out = bf16(s * rsqrt(mean(s^2) + eps)) * w
// kGather: output row b is computed from input row ends[b + 1] - 1 (ends = the cumulative query
// lengths of a prefill batch: the last token of sequence b), wrapped like a Python index when it is
// negative; only those rows are read and no residual_out is written.
template <int NC, bool kResidual, bool kGather>
__global__ __launch_bounds__(256) void rms_norm_kernel(
    const bf16_t *__restrict__ x, int64_t x_stride, const bf16_t *__restrict__ residual, int64_t res_stride,
    const bf16_t *__restrict__ weight, bf16_t *__restrict__ out, bf16_t *__restrict__ residual_out,
    const int32_t *__restrict__ ends, int32_t src_rows, int32_t rows, int32_t hidden, float eps) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    int64_t src = row;
    if (kGather) {
        src = static_cast<int64_t>(ends[row + 1]) - 1;
        if (src < 0) src += src_rows;                             // (x[-1] is the last row)
        src = min(max(src, static_cast<int64_t>(0)), static_cast<int64_t>(src_rows) - 1);   // device data the host could not check
    }
    const bf16_t *xr = x + src * x_stride;
    const bf16_t *rr = kResidual ? residual + src * res_stride : nullptr;
    uint4 xv[NC], rv[NC], wv[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int e = min(c * 512 + lane * 8, hidden - 8);       // lanes past the row re-read its end
        xv[c] = *reinterpret_cast<const uint4 *>(xr + e);
        if (kResidual) rv[c] = *reinterpret_cast<const uint4 *>(rr + e);
        wv[c] = *reinterpret_cast<const uint4 *>(weight + e);
    }
    float v[NC][8];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const bool live = c * 512 + lane * 8 < hidden;
        unpack8(xv[c], v[c]);
        if (kResidual) {
            float rf[8];
            unpack8(rv[c], rf);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[c][i] += rf[i];
            if (live && !kGather) {
                uint4 ro;
                ro.x = pack_bf16x2(v[c][0], v[c][1]); ro.y = pack_bf16x2(v[c][2], v[c][3]);
                ro.z = pack_bf16x2(v[c][4], v[c][5]); ro.w = pack_bf16x2(v[c][6], v[c][7]);
                *reinterpret_cast<uint4 *>(residual_out + static_cast<int64_t>(row) * hidden + c * 512 + lane * 8) = ro;
            }
        }
        if (live) {
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = fmaf(v[c][i], v[c][i], ss);
        }
    }
    ss = wave_sum(ss);
    const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        if (c * 512 + lane * 8 < hidden) {
            float wf[8], y[8];
            unpack8(wv[c], wf);
#pragma unroll
            for (int i = 0; i < 8; ++i) y[i] = round_bf16(v[c][i] * inv) * wf[i];
            uint4 o;
            o.x = pack_bf16x2(y[0], y[1]); o.y = pack_bf16x2(y[2], y[3]);
            o.z = pack_bf16x2(y[4], y[5]); o.w = pack_bf16x2(y[6], y[7]);
            *reinterpret_cast<uint4 *>(out + static_cast<int64_t>(row) * hidden + c * 512 + lane * 8) = o;
        }
    }
}

template <int NC>
static void launch_rms_norm(hipStream_t stream, const bf16_t *x, int64_t x_stride, const bf16_t *residual,
                            int64_t res_stride, const bf16_t *weight, bf16_t *out, bf16_t *residual_out,
                            const int32_t *ends, int32_t src_rows, int32_t rows, int32_t hidden, float eps) {
    const dim3 grid((rows + 3) / 4), block(256);
    if (ends && residual)
        hipLaunchKernelGGL((rms_norm_kernel<NC, true, true>), grid, block, 0, stream, x, x_stride, residual, res_stride,
                           weight, out, residual_out, ends, src_rows, rows, hidden, eps);
    else if (ends)
        hipLaunchKernelGGL((rms_norm_kernel<NC, false, true>), grid, block, 0, stream, x, x_stride, residual, res_stride,
                           weight, out, residual_out, ends, src_rows, rows, hidden, eps);
    else if (residual)
        hipLaunchKernelGGL((rms_norm_kernel<NC, true, false>), grid, block, 0, stream, x, x_stride, residual, res_stride,
                           weight, out, residual_out, ends, src_rows, rows, hidden, eps);
    else
        hipLaunchKernelGGL((rms_norm_kernel<NC, false, false>), grid, block, 0, stream, x, x_stride, residual, res_stride,
                           weight, out, residual_out, ends, src_rows, rows, hidden, eps);
}

static void dispatch_rms_norm(hipStream_t st, const bf16_t *xp, int64_t x_row_stride, const bf16_t *rp,
                              int64_t residual_row_stride, const bf16_t *wp, bf16_t *op, bf16_t *rop,
                              const int32_t *ends, int32_t src_rows, int32_t rows, int32_t hidden, float eps) {
    switch ((hidden + 511) / 512) {
        case 1: launch_rms_norm<1>(st, xp, x_row_stride, rp, residual_row_stride, wp, op, rop, ends, src_rows, rows, hidden, eps); break;
        case 2: launch_rms_norm<2>(st, xp, x_row_stride, rp, residual_row_stride, wp, op, rop, ends, src_rows, rows, hidden, eps); break;
        case 3: launch_rms_norm<3>(st, xp, x_row_stride, rp, residual_row_stride, wp, op, rop, ends, src_rows, rows, hidden, eps); break;
        case 4: launch_rms_norm<4>(st, xp, x_row_stride, rp, residual_row_stride, wp, op, rop, ends, src_rows, rows, hidden, eps); break;
        case 5: launch_rms_norm<5>(st, xp, x_row_stride, rp, residual_row_stride, wp, op, rop, ends, src_rows, rows, hidden, eps); break;
        case 6: launch_rms_norm<6>(st, xp, x_row_stride, rp, residual_row_stride, wp, op, rop, ends, src_rows, rows, hidden, eps); break;
        case 7: launch_rms_norm<7>(st, xp, x_row_stride, rp, residual_row_stride, wp, op, rop, ends, src_rows, rows, hidden, eps); break;
        default: launch_rms_norm<8>(st, xp, x_row_stride, rp, residual_row_stride, wp, op, rop, ends, src_rows, rows, hidden, eps); break;
    }
}

// Eight lanes per (token, head) row of 128 elements: lane j of a row holds elements [8j, 8j+8) and
// [64+8j, 64+8j+8) -- the two halves the neox rotation mixes element by element -- so every access
// to qkv, the weights, the rope table, q_out, k_out and the caches is one 16-byte load or store, and
// a cache head row of 256 B is written by 8 consecutive lanes (16 for a value row) with dwordx4 stores.  A wavefront covers 8 rows,
// a workgroup 32.  Heads [0, hq) are queries, [hq, hq+hkv) keys.  With a cache (k_cache != nullptr)
// the rotated key row is also written to its cache slot and rows [hq+hkv, hq+2*hkv) copy the value
// heads to theirs -- the KV scatter fused into the step that produces k (slot -1 or out of range
// skips the row); without a cache the value rows are not visited at all.
__global__ __launch_bounds__(256) void qk_norm_rope_kernel(
    const bf16_t *__restrict__ qkv, int64_t row_stride, const int64_t *__restrict__ positions,
    const bf16_t *__restrict__ q_weight, const bf16_t *__restrict__ k_weight,
    const float *__restrict__ rope_cache, bf16_t *__restrict__ q_out, bf16_t *__restrict__ k_out,
    bf16_t *__restrict__ k_cache, bf16_t *__restrict__ v_cache, const int32_t *__restrict__ slot_mapping,
    int64_t num_slots, int64_t n_rows, int32_t hq, int32_t hkv, int32_t heads, int32_t max_position, float eps) {
    const int j = threadIdx.x & 7;
    const int64_t r = static_cast<int64_t>(blockIdx.x) * 32 + (threadIdx.x >> 3);
    if (r >= n_rows) return;                                             // (whole groups of 8 lanes; the sums below stay inside a group)
    const int64_t tok = r / heads;
    const int head = static_cast<int>(r % heads);
    const bf16_t *src = qkv + tok * row_stride + head * kHeadDim;     // q, k and v heads are adjacent
    // every load of the row goes out before the first use
    const u32x4_t lo = *reinterpret_cast<const u32x4_t *>(src + 8 * j);
    const u32x4_t hi = *reinterpret_cast<const u32x4_t *>(src + 64 + 8 * j);
    int64_t slot = -1;
    if (k_cache != nullptr && head >= hq) {
        slot = slot_mapping[tok];
        if (slot >= num_slots) slot = -1;
    }
    if (head >= hq + hkv) {                                            // value head: cache write only
        if (slot >= 0) {
            bf16_t *dst = v_cache + (slot * hkv + (head - hq - hkv)) * kHeadDim;
            *reinterpret_cast<u32x4_t *>(dst + 8 * j) = lo;
            *reinterpret_cast<u32x4_t *>(dst + 64 + 8 * j) = hi;
        }
        return;
    }
    const bool is_q = head < hq;
    const bf16_t *w = is_q ? q_weight : k_weight;
    const uint4 w1v = *reinterpret_cast<const uint4 *>(w + 8 * j);
    const uint4 w2v = *reinterpret_cast<const uint4 *>(w + 64 + 8 * j);
    // positions outside the table are clamped instead of read out of bounds
    const int64_t pos = min(max(positions[tok], static_cast<int64_t>(0)), static_cast<int64_t>(max_position) - 1);
    const float4 *cs = reinterpret_cast<const float4 *>(rope_cache + pos * kHeadDim);
    const float4 c0 = cs[2 * j], c1 = cs[2 * j + 1], s0 = cs[16 + 2 * j], s1 = cs[16 + 2 * j + 1];
    const float cv[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
    float x1[8], x2[8], w1[8], w2[8];
    unpack8(make_uint4(lo[0], lo[1], lo[2], lo[3]), x1);
    unpack8(make_uint4(hi[0], hi[1], hi[2], hi[3]), x2);
    unpack8(w1v, w1);
    unpack8(w2v, w2);
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss = fmaf(x1[i], x1[i], fmaf(x2[i], x2[i], ss));
    ss += dpp_f32<0xB1>(ss);                                           // sum over the row's 8 lanes: quad_perm [1,0,3,2],
    ss += dpp_f32<0x4E>(ss);                                           // quad_perm [2,3,0,1],
    ss += dpp_f32<0x141>(ss);                                          // row_half_mirror
    const float inv = rsqrtf(ss * (1.0f / kHeadDim) + eps);
    float o1[8], o2[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float y1 = round_bf16(round_bf16(x1[i] * inv) * w1[i]);
        const float y2 = round_bf16(round_bf16(x2[i] * inv) * w2[i]);
        o1[i] = y1 * cv[i] - y2 * sv[i];
        o2[i] = y2 * cv[i] + y1 * sv[i];
    }
    const u32x4_t p1 = {pack_bf16x2(o1[0], o1[1]), pack_bf16x2(o1[2], o1[3]), pack_bf16x2(o1[4], o1[5]), pack_bf16x2(o1[6], o1[7])};
    const u32x4_t p2 = {pack_bf16x2(o2[0], o2[1]), pack_bf16x2(o2[2], o2[3]), pack_bf16x2(o2[4], o2[5]), pack_bf16x2(o2[6], o2[7])};
    bf16_t *dst = is_q ? q_out + (tok * hq + head) * kHeadDim : k_out + (tok * hkv + (head - hq)) * kHeadDim;
    *reinterpret_cast<u32x4_t *>(dst + 8 * j) = p1;
    *reinterpret_cast<u32x4_t *>(dst + 64 + 8 * j) = p2;
    if (slot >= 0) {
        bf16_t *cd = k_cache + (slot * hkv + (head - hq)) * kHeadDim;
        *reinterpret_cast<u32x4_t *>(cd + 8 * j) = p1;
        *reinterpret_cast<u32x4_t *>(cd + 64 + 8 * j) = p2;
    }
}

// out[r, i] = bf16(silu(x[r, i])) * x[r, inter + i], 8 elements per lane
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const bf16_t *__restrict__ x, int64_t row_stride,
                                                           bf16_t *__restrict__ out, int64_t total_chunks,
                                                           int32_t chunks_per_row, int32_t inter) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total_chunks) return;
    const int64_t row = idx / chunks_per_row;
    const int e = static_cast<int>(idx % chunks_per_row) * 8;
    const bf16_t *xr = x + row * row_stride;
    float g[8], u[8];
    unpack8(*reinterpret_cast<const uint4 *>(xr + e), g);
    unpack8(*reinterpret_cast<const uint4 *>(xr + inter + e), u);
    float y[8];
#pragma unroll
    // (silu through the hardware exp2 and reciprocal, one ulp each: the library expf and an IEEE division are
    // ~25 instructions per element and made this kernel instruction-bound at prefill sizes)
    for (int i = 0; i < 8; ++i)
        y[i] = round_bf16(g[i] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g[i]))) * u[i];
    uint4 o;
    o.x = pack_bf16x2(y[0], y[1]); o.y = pack_bf16x2(y[2], y[3]);
    o.z = pack_bf16x2(y[4], y[5]); o.w = pack_bf16x2(y[6], y[7]);
    *reinterpret_cast<uint4 *>(out + row * inter + e) = o;
}

// host staging buffer -> device buffer, 16 bytes per lane; the input ids that name a row of the
// previous step's sampler output are taken from there instead
__global__ void stage_decode_inputs_kernel(uint4 *dst, const uint4 *src, int64_t chunks, int64_t ids_chunk0,
                                           const int32_t *index, int32_t n, const int64_t *prev, int32_t n_prev) {
    const int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (c >= chunks) return;
    uint4 v = src[c];
    const int64_t i0 = (c - ids_chunk0) * 2;                       // first of the two ids in this chunk
    if (c >= ids_chunk0 && i0 < n) {
        const int32_t j0 = index[i0];
        if (static_cast<uint32_t>(j0) < static_cast<uint32_t>(n_prev)) {
            const int64_t t = prev[j0];
            v.x = static_cast<uint32_t>(t);
            v.y = static_cast<uint32_t>(t >> 32);
        }
        if (i0 + 1 < n) {
            const int32_t j1 = index[i0 + 1];
            if (static_cast<uint32_t>(j1) < static_cast<uint32_t>(n_prev)) {
                const int64_t t = prev[j1];
                v.z = static_cast<uint32_t>(t);
                v.w = static_cast<uint32_t>(t >> 32);
            }
        }
    }
    dst[c] = v;
}

}  // namespace nva

extern "C" int nva_rms_norm(const void *x, int64_t x_row_stride, const void *residual, int64_t residual_row_stride,
                            const void *weight, void *out, void *residual_out, int32_t rows, int32_t hidden,
                            float eps, void *stream) {
    using namespace nva;
    if (rows < 0 || hidden <= 0) return NVA_ERR_BAD_SHAPE;
    if (hidden % 8 != 0 || hidden > kNormMaxChunks * 512) return NVA_ERR_UNSUPPORTED_GEOMETRY;
    if (rows == 0) return NVA_OK;
    if (!x || !weight || !out) return NVA_ERR_NULL_POINTER;
    if (residual && !residual_out) return NVA_ERR_NULL_POINTER;
    if (x_row_stride < hidden || x_row_stride % 8 != 0) return NVA_ERR_BAD_STRIDE;
    if (residual && (residual_row_stride < hidden || residual_row_stride % 8 != 0)) return NVA_ERR_BAD_STRIDE;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(out) || (residual && (!aligned16(residual) || !aligned16(residual_out))))
        return NVA_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bf16_t *xp = static_cast<const bf16_t *>(x), *rp = static_cast<const bf16_t *>(residual);
    const bf16_t *wp = static_cast<const bf16_t *>(weight);
    bf16_t *op = static_cast<bf16_t *>(out), *rop = static_cast<bf16_t *>(residual_out);
    dispatch_rms_norm(st, xp, x_row_stride, rp, residual_row_stride, wp, op, rop, nullptr, rows, rows, hidden, eps);
    return launch_status();
}

extern "C" int nva_gather_last_rms_norm(const void *x, int64_t x_row_stride, const void *residual,
                                        int64_t residual_row_stride, const int32_t *cu_seqlens_q, const void *weight,
                                        void *out, int32_t batch, int32_t total_rows, int32_t hidden, float eps,
                                        void *stream) {
    using namespace nva;
    if (batch < 0 || total_rows < 0 || hidden <= 0) return NVA_ERR_BAD_SHAPE;
    if (hidden % 8 != 0 || hidden > kNormMaxChunks * 512) return NVA_ERR_UNSUPPORTED_GEOMETRY;
    if (batch == 0) return NVA_OK;
    if (total_rows == 0) return NVA_ERR_BAD_SHAPE;                 // rows to pick, none to pick from
    if (!x || !weight || !out || !cu_seqlens_q) return NVA_ERR_NULL_POINTER;
    if (x_row_stride < hidden || x_row_stride % 8 != 0) return NVA_ERR_BAD_STRIDE;
    if (residual && (residual_row_stride < hidden || residual_row_stride % 8 != 0)) return NVA_ERR_BAD_STRIDE;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(out) || (residual && !aligned16(residual)))
        return NVA_ERR_MISALIGNED;
    dispatch_rms_norm(static_cast<hipStream_t>(stream), static_cast<const bf16_t *>(x), x_row_stride,
                      static_cast<const bf16_t *>(residual), residual_row_stride, static_cast<const bf16_t *>(weight),
                      static_cast<bf16_t *>(out), nullptr, cu_seqlens_q, total_rows, batch, hidden, eps);
    return launch_status();
}

extern "C" int nva_qk_norm_rope(const void *qkv, int64_t qkv_row_stride, const int64_t *positions,
                                const void *q_weight, const void *k_weight, const float *rope_cache,
                                int32_t max_position, void *q_out, void *k_out, void *k_cache, void *v_cache,
                                const int32_t *slot_mapping, int64_t num_slots, int32_t n_tokens,
                                int32_t num_heads, int32_t num_kv_heads, int32_t head_dim, float eps,
                                void *stream) {
    using namespace nva;
    if (n_tokens < 0 || num_heads <= 0 || num_kv_heads <= 0 || max_position <= 0 || num_slots < 0)
        return NVA_ERR_BAD_SHAPE;
    if (head_dim != kHeadDim) return NVA_ERR_UNSUPPORTED_GEOMETRY;
    if (n_tokens == 0) return NVA_OK;
    if (!qkv || !positions || !q_weight || !k_weight || !rope_cache || !q_out || !k_out) return NVA_ERR_NULL_POINTER;
    const bool store = k_cache != nullptr || v_cache != nullptr || slot_mapping != nullptr;
    if (store && (!k_cache || !v_cache || !slot_mapping)) return NVA_ERR_NULL_POINTER;
    if (qkv_row_stride < static_cast<int64_t>(num_heads + 2 * num_kv_heads) * head_dim || qkv_row_stride % 8 != 0)
        return NVA_ERR_BAD_STRIDE;
    if (!aligned16(qkv) || !aligned16(q_weight) || !aligned16(k_weight) || !aligned16(rope_cache) || !aligned16(q_out) ||
        !aligned16(k_out) || (store && (!aligned16(k_cache) || !aligned16(v_cache))))
        return NVA_ERR_MISALIGNED;
    const int32_t heads = num_heads + (store ? 2 : 1) * num_kv_heads;   // value rows only when they are stored
    const int64_t n_rows = static_cast<int64_t>(n_tokens) * heads;
    if ((n_rows + 31) / 32 > 0x7fffffffLL) return NVA_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(qk_norm_rope_kernel, dim3(static_cast<uint32_t>((n_rows + 31) / 32)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const bf16_t *>(qkv), qkv_row_stride, positions,
                       static_cast<const bf16_t *>(q_weight), static_cast<const bf16_t *>(k_weight), rope_cache,
                       static_cast<bf16_t *>(q_out), static_cast<bf16_t *>(k_out), static_cast<bf16_t *>(k_cache),
                       static_cast<bf16_t *>(v_cache), slot_mapping, num_slots, n_rows, num_heads, num_kv_heads,
                       heads, max_position, eps);
    return launch_status();
}

extern "C" int nva_silu_and_mul(const void *x, int64_t x_row_stride, void *out, int32_t rows, int32_t inter,
                                void *stream) {
    using namespace nva;
    if (rows < 0 || inter <= 0) return NVA_ERR_BAD_SHAPE;
    if (inter % 8 != 0) return NVA_ERR_UNSUPPORTED_GEOMETRY;
    if (rows == 0) return NVA_OK;
    if (!x || !out) return NVA_ERR_NULL_POINTER;
    if (x_row_stride < 2 * static_cast<int64_t>(inter) || x_row_stride % 8 != 0) return NVA_ERR_BAD_STRIDE;
    if (!aligned16(x) || !aligned16(out)) return NVA_ERR_MISALIGNED;
    const int32_t chunks_per_row = inter / 8;
    const int64_t total = static_cast<int64_t>(rows) * chunks_per_row;
    if ((total + 255) / 256 > 0x7fffffffLL) return NVA_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(silu_and_mul_kernel, dim3(static_cast<uint32_t>((total + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const bf16_t *>(x), x_row_stride,
                       static_cast<bf16_t *>(out), total, chunks_per_row, inter);
    return launch_status();
}

extern "C" int nva_stage_decode_inputs(void *dst, const void *src_host, int64_t nbytes, int64_t ids_offset,
                                       int64_t index_offset, int32_t n, const int64_t *prev_tokens, int32_t n_prev,
                                       void *stream) {
    using namespace nva;
    if (nbytes < 0 || n < 0 || n_prev < 0 || ids_offset < 0 || index_offset < 0) return NVA_ERR_BAD_SHAPE;
    if (nbytes % 16 != 0 || ids_offset % 16 != 0 || index_offset % 4 != 0) return NVA_ERR_MISALIGNED;
    if (ids_offset + static_cast<int64_t>(n) * 8 > nbytes || index_offset + static_cast<int64_t>(n) * 4 > nbytes)
        return NVA_ERR_BAD_SHAPE;
    if (nbytes == 0) return NVA_OK;
    if (!dst || !src_host || (n_prev > 0 && !prev_tokens)) return NVA_ERR_NULL_POINTER;
    if (!aligned16(dst) || !aligned16(src_host)) return NVA_ERR_MISALIGNED;
    const int64_t chunks = nbytes / 16;
    if ((chunks + 255) / 256 > 0x7fffffffLL) return NVA_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(stage_decode_inputs_kernel, dim3(static_cast<uint32_t>((chunks + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<uint4 *>(dst), static_cast<const uint4 *>(src_host),
                       chunks, ids_offset / 16,
                       reinterpret_cast<const int32_t *>(static_cast<const char *>(src_host) + index_offset), n,
                       prev_tokens, n_prev);
    return launch_status();
}
