// Paged single-query (decode) attention for gfx950: split-K over 256-token KV blocks.
//
// Replaces flash_attn_with_kvcache as called by nanovllm/layers/attention.py:71-74.
//
// Stage 1 (decode_split_kernel): one workgroup of 4 wavefronts per
// (KV block j of the sequence, kv head g, sequence b).  Wavefront w owns tokens
// [64w, 64w+64) of the block.  A K (or V) head row is 128 bf16 = 256 B = 16 lanes x 16 B, so a
// wavefront reads 4 token rows per dwordx4 load instruction; it issues all 16 K loads and
// all 16 V loads of its 64 tokens up front (32 KB in flight per wavefront) and only then
// starts the arithmetic, which keeps the memory pipe full without any software pipeline.
// The G = num_heads/num_kv_heads query heads that share kv head g are processed together
// from the same registers (K and V are read once per kv head, not once per query head).
// Scores are reduced over the 16 lanes of a row with DPP adds; the softmax is the usual
// running-max form in base 2 (scale * log2(e) folded into q).  The four wavefronts merge
// through LDS and write one unnormalised partial (max, sum, o[128]) per query head.
// Stage 2 (decode_merge_kernel): one workgroup per (query head, sequence) merges the
// ceil(ctx/256) partials and writes bf16.
//
// HBM traffic per sequence and layer: ctx * num_kv_heads * 128 * 2 B for K plus the same for
// V (4096 B per token at 8 kv heads); partials add (128+2)*4 B per (block, query head), 1.6 %.
//
// Launch geometry is a function of (batch, max_blocks, heads) only; context_lens and the
// block table are read on the device, so the launch can be captured in a HIP graph and
// replayed with new contents.  Workgroups whose block lies beyond context_lens[b] exit at
// once; only block_tables[b][j] with j*256 < context_lens[b] is dereferenced.
#include "nva_common.h"

#include <math.h>

namespace nva {

constexpr int kSplitThreads = 256;
constexpr int kTokPerWave = 64;
constexpr int kIters = kTokPerWave / 4;   // 4 token rows per load instruction

template <int G>
__global__ __launch_bounds__(kSplitThreads) void decode_split_kernel(
    const bf16_t *__restrict__ q, int64_t q_row_stride,
    const bf16_t *__restrict__ k_cache, const bf16_t *__restrict__ v_cache,
    const int32_t *__restrict__ block_tables, int32_t bt_row_stride,
    const int32_t *__restrict__ context_lens,
    float *__restrict__ part_o, float *__restrict__ part_ml,
    int32_t max_blocks, int32_t num_heads, int32_t num_kv_heads, int32_t num_blocks,
    float scale_log2e) {
    const int j = blockIdx.x;
    const int g = blockIdx.y;
    const int b = blockIdx.z;
    const int ctx = context_lens[b];
    const int blk_tok0 = j * kBlockSize;
    if (blk_tok0 >= ctx) return;                       // uniform for the whole workgroup
    const int32_t blk = block_tables[static_cast<int64_t>(b) * bt_row_stride + j];
    const bool blk_ok = static_cast<uint32_t>(blk) < static_cast<uint32_t>(num_blocks);
    const int n_blk = min(kBlockSize, ctx - blk_tok0); // valid tokens in this block, >= 1

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int tg = lane >> 4;                           // token row within a load instruction
    const int dl = lane & 15;                           // 16-byte chunk of the head row
    const int w0 = wave * kTokPerWave;

    float m_w[G], l_w[G], o[G][8];
#pragma unroll
    for (int h = 0; h < G; ++h) {
        m_w[h] = -INFINITY;
        l_w[h] = 0.f;
#pragma unroll
        for (int d = 0; d < 8; ++d) o[h][d] = 0.f;
    }

    if (blk_ok && w0 < n_blk) {
        const int last = n_blk - 1;
        const int64_t row = static_cast<int64_t>(num_kv_heads) * kHeadDim;   // elements per token
        const int64_t base = static_cast<int64_t>(blk) * kBlockSize * row + g * kHeadDim + dl * 8;
        const bf16_t *kb = k_cache + base;
        const bf16_t *vb = v_cache + base;
        uint4 kr[kIters], vr[kIters];
#pragma unroll
        for (int i = 0; i < kIters; ++i) {
            const int t = min(w0 + i * 4 + tg, last);   // clamp: stay on rows that were written
            kr[i] = *reinterpret_cast<const uint4 *>(kb + t * row);
        }
#pragma unroll
        for (int i = 0; i < kIters; ++i) {
            const int t = min(w0 + i * 4 + tg, last);
            vr[i] = *reinterpret_cast<const uint4 *>(vb + t * row);
        }

        float qf[G][8];
#pragma unroll
        for (int h = 0; h < G; ++h) {
            const bf16_t *qp = q + static_cast<int64_t>(b) * q_row_stride + (g * G + h) * kHeadDim + dl * 8;
            const uint4 qr = *reinterpret_cast<const uint4 *>(qp);
            unpack8(qr, qf[h]);
#pragma unroll
            for (int d = 0; d < 8; ++d) qf[h][d] *= scale_log2e;
        }

        float s[kIters][G];
#pragma unroll
        for (int i = 0; i < kIters; ++i) {
            float kf[8];
            unpack8(kr[i], kf);
            const bool valid = (w0 + i * 4 + tg) <= last;
#pragma unroll
            for (int h = 0; h < G; ++h) {
                float acc = 0.f;
#pragma unroll
                for (int d = 0; d < 8; ++d) acc = fmaf(qf[h][d], kf[d], acc);
                acc = row16_sum(acc);
                s[i][h] = valid ? acc : -INFINITY;
            }
        }
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float mx = s[0][h];
#pragma unroll
            for (int i = 1; i < kIters; ++i) mx = fmaxf(mx, s[i][h]);
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));   // finite: token w0 of this wave is valid
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < kIters; ++i) {
                s[i][h] = exp2f(s[i][h] - mx);
                sum += s[i][h];
            }
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            m_w[h] = mx;
            l_w[h] = sum;
        }
#pragma unroll
        for (int i = 0; i < kIters; ++i) {
            float vf[8];
            unpack8(vr[i], vf);
#pragma unroll
            for (int h = 0; h < G; ++h)
#pragma unroll
                for (int d = 0; d < 8; ++d) o[h][d] = fmaf(s[i][h], vf[d], o[h][d]);
        }
#pragma unroll
        for (int h = 0; h < G; ++h)
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                o[h][d] += __shfl_xor(o[h][d], 16, 64);
                o[h][d] += __shfl_xor(o[h][d], 32, 64);
            }
    }

    // ---- merge the four wavefronts through LDS ------------------------------------------
    __shared__ float sh_m[4][G];
    __shared__ float sh_l[4][G];
    __shared__ float sh_o[4][G][kHeadDim];
    if (tg == 0) {
#pragma unroll
        for (int h = 0; h < G; ++h)
#pragma unroll
            for (int d = 0; d < 8; ++d) sh_o[wave][h][dl * 8 + d] = o[h][d];
    }
    if (lane == 0) {
#pragma unroll
        for (int h = 0; h < G; ++h) {
            sh_m[wave][h] = m_w[h];
            sh_l[wave][h] = l_w[h];
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * kHeadDim; idx += kSplitThreads) {
        const int h = idx / kHeadDim;
        const int d = idx % kHeadDim;
        float m = sh_m[0][h];
#pragma unroll
        for (int w = 1; w < 4; ++w) m = fmaxf(m, sh_m[w][h]);
        float l = 0.f, acc = 0.f;
        if (m > -INFINITY) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float f = exp2f(sh_m[w][h] - m);   // exp2(-inf) = 0 for idle wavefronts
                l = fmaf(f, sh_l[w][h], l);
                acc = fmaf(f, sh_o[w][h][d], acc);
            }
        }
        const int64_t slot = (static_cast<int64_t>(b) * max_blocks + j) * num_heads + g * G + h;
        part_o[slot * kHeadDim + d] = acc;
        if (d == 0) {
            part_ml[slot * 2 + 0] = m;
            part_ml[slot * 2 + 1] = l;
        }
    }
}

// One workgroup of 128 lanes (lane = output dim) per (query head, sequence).
__global__ __launch_bounds__(kHeadDim) void decode_merge_kernel(
    const float *__restrict__ part_o, const float *__restrict__ part_ml,
    const int32_t *__restrict__ context_lens, bf16_t *__restrict__ out,
    int32_t max_blocks, int32_t num_heads) {
    const int h = blockIdx.x;
    const int b = blockIdx.y;
    const int d = threadIdx.x;
    const int ctx = context_lens[b];
    const int nsplit = min(max_blocks, (ctx + kBlockSize - 1) / kBlockSize);
    const int64_t first = (static_cast<int64_t>(b) * max_blocks) * num_heads + h;
    float m = -INFINITY;
    for (int j = 0; j < nsplit; ++j) m = fmaxf(m, part_ml[(first + static_cast<int64_t>(j) * num_heads) * 2]);
    float acc = 0.f, l = 0.f;
    if (m > -INFINITY) {
        for (int j = 0; j < nsplit; ++j) {
            const int64_t slot = first + static_cast<int64_t>(j) * num_heads;
            const float f = exp2f(part_ml[slot * 2] - m);
            l = fmaf(f, part_ml[slot * 2 + 1], l);
            acc = fmaf(f, part_o[slot * kHeadDim + d], acc);
        }
    }
    const float r = l > 0.f ? acc / l : 0.f;             // no visible key -> zeros
    out[(static_cast<int64_t>(b) * num_heads + h) * kHeadDim + d] = f32_to_bf16(r);
}

template <int G>
static void launch_split(const void *q, int64_t q_row_stride, const void *k_cache, const void *v_cache,
                         const int32_t *block_tables, int32_t bt_row_stride, const int32_t *context_lens,
                         float *part_o, float *part_ml, int32_t max_blocks, int32_t batch,
                         int32_t num_heads, int32_t num_kv_heads, int32_t num_blocks, float scale_log2e,
                         hipStream_t stream) {
    hipLaunchKernelGGL(decode_split_kernel<G>, dim3(max_blocks, num_kv_heads, batch), dim3(kSplitThreads),
                       0, stream, static_cast<const bf16_t *>(q), q_row_stride,
                       static_cast<const bf16_t *>(k_cache), static_cast<const bf16_t *>(v_cache),
                       block_tables, bt_row_stride, context_lens, part_o, part_ml, max_blocks, num_heads,
                       num_kv_heads, num_blocks, scale_log2e);
}

}  // namespace nva

extern "C" size_t nva_paged_decode_workspace_bytes(int32_t batch, int32_t num_heads, int32_t head_dim,
                                                   int32_t max_blocks) {
    if (batch <= 0 || num_heads <= 0 || head_dim <= 0 || max_blocks <= 0) return 0;
    const size_t slots = static_cast<size_t>(batch) * max_blocks * num_heads;
    return slots * (static_cast<size_t>(head_dim) + 2) * sizeof(float);
}

extern "C" int nva_paged_decode_attn(const void *q, int64_t q_row_stride, const void *k_cache,
                                     const void *v_cache, const int32_t *block_tables,
                                     int32_t bt_row_stride, int32_t max_blocks,
                                     const int32_t *context_lens, void *out, void *workspace,
                                     size_t workspace_bytes, int32_t batch, int32_t num_heads,
                                     int32_t num_kv_heads, int32_t head_dim, int32_t block_size,
                                     int32_t num_blocks, float scale, void *stream) {
    using namespace nva;
    if (batch < 0 || num_heads <= 0 || num_kv_heads <= 0 || max_blocks < 0 || num_blocks < 0)
        return NVA_ERR_BAD_SHAPE;
    if (head_dim != kHeadDim || block_size != kBlockSize) return NVA_ERR_UNSUPPORTED_GEOMETRY;
    if (num_heads % num_kv_heads != 0) return NVA_ERR_UNSUPPORTED_GEOMETRY;
    const int group = num_heads / num_kv_heads;
    if (group != 1 && group != 2 && group != 4 && group != 8) return NVA_ERR_UNSUPPORTED_GEOMETRY;
    if (batch == 0) return NVA_OK;
    if (batch > 65535 || num_kv_heads > 65535) return NVA_ERR_BAD_SHAPE;      // grid y/z limits
    if (!q || !k_cache || !v_cache || !context_lens || !out) return NVA_ERR_NULL_POINTER;
    if (max_blocks > 0 && (!block_tables || !workspace)) return NVA_ERR_NULL_POINTER;
    if (q_row_stride < static_cast<int64_t>(num_heads) * head_dim || q_row_stride % 8 != 0)
        return NVA_ERR_BAD_STRIDE;
    if (bt_row_stride < max_blocks) return NVA_ERR_BAD_STRIDE;
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(workspace))
        return NVA_ERR_MISALIGNED;
    if (workspace_bytes < nva_paged_decode_workspace_bytes(batch, num_heads, head_dim, max_blocks))
        return NVA_ERR_WORKSPACE_TOO_SMALL;

    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t slots = static_cast<size_t>(batch) * max_blocks * num_heads;
    float *part_o = static_cast<float *>(workspace);
    float *part_ml = part_o + slots * kHeadDim;
    const float scale_log2e = scale * 1.4426950408889634f;
    if (max_blocks > 0) {
        switch (group) {
#define NVA_CASE(G)                                                                                      \
    case G:                                                                                              \
        launch_split<G>(q, q_row_stride, k_cache, v_cache, block_tables, bt_row_stride, context_lens,    \
                        part_o, part_ml, max_blocks, batch, num_heads, num_kv_heads, num_blocks,         \
                        scale_log2e, s);                                                                 \
        break;
            NVA_CASE(1)
            NVA_CASE(2)
            NVA_CASE(4)
            NVA_CASE(8)
#undef NVA_CASE
        }
        if (launch_status() != NVA_OK) return NVA_ERR_LAUNCH_FAILED;
    }
    hipLaunchKernelGGL(decode_merge_kernel, dim3(num_heads, batch), dim3(kHeadDim), 0, s, part_o, part_ml,
                       context_lens, static_cast<bf16_t *>(out), max_blocks, num_heads);
    return launch_status();
}
