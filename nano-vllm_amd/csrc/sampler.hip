// Temperature / exponential-race sampler for gfx950.
//
// Replaces Sampler.forward of nanovllm/layers/sampler.py:10-15:
//     x = float(logits) / T;  p = softmax(x);  token = argmax_i p_i / max(E_i, 1e-10)
// E ~ Exp(1) is either read from a caller-supplied tensor (replayable; used for parity) or
// drawn in-kernel from Philox4x32-10 (no noise traffic).  The arithmetic keeps the
// reference's operation order -- true fp32 division by T, exp(x - rowmax) / rowsum, then the
// division by the clamped noise -- so the argmax can only differ from the reference where
// two scores are equal to within fp32 rounding.
//
// A row of 151,936 logits is far too little work for one workgroup and 64..256 rows are
// too few workgroups for 256 CUs, so a row is cut into chunks of 2048 columns (one
// workgroup of 256 lanes, one 16-byte load of 8 bf16 per lane):
// With a caller-supplied noise tensor (the replayable form):
//   pass 1  per (chunk, row): chunk max and sum exp(x - chunk max)          -> workspace
//   pass 2  per (chunk, row): merge the row's partials into (max, sum), then
//           best p_i / E_i and its column inside the chunk                   -> workspace
//   pass 3  per row: best chunk, lowest column on ties                       -> int64 token
// Pass 2 re-reads the logits (2 B/col) that pass 1 pulled through L2 / Infinity Cache.
// With in-kernel noise there is nothing to replay against, so the draw uses the equivalent
// Gumbel form argmax_i (x_i - log E_i), which needs no softmax: ONE pass over the logits
// (sampler_gumbel_kernel, chunks of 8192 columns) followed by the per-row pick -- the same exact
// categorical draw.
// Algorithmic HBM bytes per row: vocab * 2 B (+ vocab * 4 B when the noise is read).
#include "nva_common.h"

#include <math.h>

namespace nva {

constexpr int kSampThreads = 256;
constexpr int kSampChunk = kSampThreads * 8;   // columns per workgroup

__host__ __device__ inline int samp_chunks(int vocab) { return (vocab + kSampChunk - 1) / kSampChunk; }

struct Philox {
    // Philox4x32-10 (Salmon et al., SC'11): counter (c0..c3), key (k0,k1)
    __device__ static inline uint4 draw(uint4 c, uint2 k) {
#pragma unroll
        for (int r = 0; r < 10; ++r) {
            // one 32x32 -> 64-bit multiply per product (integer multiplies are the slow ops here)
            const uint64_t p0 = static_cast<uint64_t>(0xD2511F53u) * c.x, p1 = static_cast<uint64_t>(0xCD9E8D57u) * c.z;
            const uint32_t hi0 = static_cast<uint32_t>(p0 >> 32), lo0 = static_cast<uint32_t>(p0);
            const uint32_t hi1 = static_cast<uint32_t>(p1 >> 32), lo1 = static_cast<uint32_t>(p1);
            c = make_uint4(hi1 ^ c.y ^ k.x, lo1, hi0 ^ c.w ^ k.y, lo0);
            k.x += 0x9E3779B9u;
            k.y += 0xBB67AE85u;
        }
        return c;
    }
};

// Loads the 8 columns [col0, col0+8) of a row as x = float(logit) / T (greedy: T = 1).
// Columns >= vocab come back as -inf.  vec_ok: the row start is 16-byte aligned.
__device__ __forceinline__ void load_x8(const bf16_t *row, int col0, int vocab, float temp,
                                        bool vec_ok, float (&x)[8]) {
    if (vec_ok && col0 + 8 <= vocab) {
        const uint4 r = *reinterpret_cast<const uint4 *>(row + col0);
        unpack8(r, x);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = x[i] / temp;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            x[i] = (col0 + i < vocab) ? bf16_to_f32(row[col0 + i]) / temp : -INFINITY;
    }
}

__global__ __launch_bounds__(kSampThreads) void sampler_partials_kernel(
    const bf16_t *__restrict__ logits, int64_t row_stride, const float *__restrict__ temperatures,
    float *__restrict__ part_max, float *__restrict__ part_sum, int32_t vocab, int32_t nchunks) {
    const int chunk = blockIdx.x;
    const int b = blockIdx.y;
    const bf16_t *row = logits + static_cast<int64_t>(b) * row_stride;
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(row) & 15u) == 0);
    float temp = temperatures[b];
    if (temp == 0.f) temp = 1.f;
    const int col0 = chunk * kSampChunk + threadIdx.x * 8;
    float x[8];
    load_x8(row, col0, vocab, temp, vec_ok, x);
    float m = x[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) m = fmaxf(m, x[i]);
    m = wave_max(m);
    __shared__ float sh[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) sh[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
    const float mm = (m == -INFINITY) ? 0.f : m;           // a chunk of -inf logits sums to 0
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += expf(x[i] - mm);      // exp(-inf) = 0 past the row end
    s = wave_sum(s);
    __syncthreads();
    if (lane == 0) sh[wave] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        part_max[static_cast<int64_t>(b) * nchunks + chunk] = m;
        part_sum[static_cast<int64_t>(b) * nchunks + chunk] = (sh[0] + sh[1]) + (sh[2] + sh[3]);
    }
}

__device__ __forceinline__ void better(float &bs, int &bi, float s, int i) {
    // larger score wins, lower column wins ties (torch.argmax returns the first maximum)
    if (s > bs || (s == bs && i < bi)) { bs = s; bi = i; }
}

__global__ __launch_bounds__(kSampThreads) void sampler_argmax_kernel(
    const bf16_t *__restrict__ logits, int64_t row_stride, const float *__restrict__ temperatures,
    const float *__restrict__ noise, int64_t noise_row_stride,
    const float *__restrict__ part_max, const float *__restrict__ part_sum,
    float *__restrict__ part_best, int32_t *__restrict__ part_idx, int32_t vocab, int32_t nchunks) {
    const int chunk = blockIdx.x;
    const int b = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __shared__ float sh[4];
    __shared__ int shi[4];

    // row max and row sum from the chunk partials
    float m = -INFINITY;
    for (int c = threadIdx.x; c < nchunks; c += kSampThreads)
        m = fmaxf(m, part_max[static_cast<int64_t>(b) * nchunks + c]);
    m = wave_max(m);
    if (lane == 0) sh[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
    float s = 0.f;
    for (int c = threadIdx.x; c < nchunks; c += kSampThreads) {
        const int64_t at = static_cast<int64_t>(b) * nchunks + c;
        s += part_sum[at] * expf(part_max[at] - m);
    }
    s = wave_sum(s);
    __syncthreads();
    if (lane == 0) sh[wave] = s;
    __syncthreads();
    s = (sh[0] + sh[1]) + (sh[2] + sh[3]);
    __syncthreads();

    const bf16_t *row = logits + static_cast<int64_t>(b) * row_stride;
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(row) & 15u) == 0);
    const float t_in = temperatures[b];
    const bool greedy = (t_in == 0.f);
    const float temp = greedy ? 1.f : t_in;
    const int col0 = chunk * kSampChunk + threadIdx.x * 8;
    float x[8];
    load_x8(row, col0, vocab, temp, vec_ok, x);

    float e[8];
    if (greedy) {
#pragma unroll
        for (int i = 0; i < 8; ++i) e[i] = 1.f;
    } else {
        const float *nrow = noise + static_cast<int64_t>(b) * noise_row_stride;
        if (((reinterpret_cast<uintptr_t>(nrow) & 15u) == 0) && col0 + 8 <= vocab) {
            const float4 a = *reinterpret_cast<const float4 *>(nrow + col0);
            const float4 c = *reinterpret_cast<const float4 *>(nrow + col0 + 4);
            e[0] = a.x; e[1] = a.y; e[2] = a.z; e[3] = a.w;
            e[4] = c.x; e[5] = c.y; e[6] = c.z; e[7] = c.w;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) e[i] = (col0 + i < vocab) ? nrow[col0 + i] : 1.f;
        }
    }

    float best = -INFINITY;
    int best_i = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (col0 + i < vocab) {
            float score;
            if (greedy) {
                score = x[i];
            } else {
                const float p = expf(x[i] - m) / s;
                score = p / fmaxf(e[i], 1e-10f);
            }
            better(best, best_i, score, col0 + i);
        }
    }
    // wavefront, then workgroup arg-max
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float os = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(best_i, off, 64);
        better(best, best_i, os, oi);
    }
    if (lane == 0) { sh[wave] = best; shi[wave] = best_i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w) better(best, best_i, sh[w], shi[w]);
        part_best[static_cast<int64_t>(b) * nchunks + chunk] = best;
        part_idx[static_cast<int64_t>(b) * nchunks + chunk] = best_i;
    }
}

// In-kernel noise: score_i = logit_i * log2(e)/T - log2(-log2(u_i)), u_i uniform in (0,1) from Philox.
// (E_i = -ln(u_i); log2(E_i) = log2(-log2(u_i)) + const, and constants do not move the argmax.)
// Greedy rows (T == 0) use score_i = logit_i.
// One pass over the logits with in-kernel noise.  A workgroup takes kGumbelChunk columns of one
// row: every lane issues its kGumbelVec 16-byte loads up front, then scores 8 columns per load.
// (Four loads per lane instead of one: the cross-lane reduction and the per-workgroup overhead are
// paid once per 8192 columns instead of once per 2048 -- they were a quarter of the kernel.)
constexpr int kGumbelVec = 4;
constexpr int kGumbelChunk = kSampChunk * kGumbelVec;

__host__ __device__ inline int gumbel_chunks(int vocab) { return (vocab + kGumbelChunk - 1) / kGumbelChunk; }

__global__ __launch_bounds__(kSampThreads) void sampler_gumbel_kernel(
    const bf16_t *__restrict__ logits, int64_t row_stride, const float *__restrict__ temperatures,
    uint64_t seed, uint64_t offset, float *__restrict__ part_best, int32_t *__restrict__ part_idx,
    int32_t vocab, int32_t nchunks) {
    const int chunk = blockIdx.x;
    const int b = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const bf16_t *row = logits + static_cast<int64_t>(b) * row_stride;
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(row) & 15u) == 0);
    const float t_in = temperatures[b];
    const bool greedy = (t_in == 0.f);
    const float k = greedy ? 1.f : 1.4426950408889634f / t_in;
    uint4 raw[kGumbelVec];
    int col0[kGumbelVec];
#pragma unroll
    for (int v = 0; v < kGumbelVec; ++v) {
        col0[v] = chunk * kGumbelChunk + v * kSampChunk + threadIdx.x * 8;
        raw[v] = make_uint4(0u, 0u, 0u, 0u);
        if (vec_ok && col0[v] + 8 <= vocab) raw[v] = *reinterpret_cast<const uint4 *>(row + col0[v]);
    }
    const uint2 key = make_uint2(static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32));
    const uint32_t o_lo = static_cast<uint32_t>(offset), o_hi = static_cast<uint32_t>(offset >> 32);
    float best = -INFINITY;
    int best_i = 0x7fffffff;
#pragma unroll
    for (int v = 0; v < kGumbelVec; ++v) {
        if (col0[v] >= vocab) continue;
        float x[8];
        if (vec_ok && col0[v] + 8 <= vocab) {
            unpack8(raw[v], x);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = (col0[v] + i < vocab) ? bf16_to_f32(row[col0[v] + i]) : -INFINITY;
        }
        float g[8];
        if (greedy) {
#pragma unroll
            for (int i = 0; i < 8; ++i) g[i] = 0.f;
        } else {
            const uint4 r0 = Philox::draw(make_uint4(static_cast<uint32_t>(col0[v] >> 2), b, o_lo, o_hi), key);
            const uint4 r1 = Philox::draw(make_uint4(static_cast<uint32_t>(col0[v] >> 2) + 1u, b, o_lo, o_hi), key);
            const uint32_t r[8] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w};
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                // u in (0, 1): 23 random bits plus one half, so that neither log below sees 0 or 1
                const float u = (static_cast<float>(r[i] >> 9) + 0.5f) * 1.1920928955078125e-7f;
                g[i] = __builtin_amdgcn_logf(-__builtin_amdgcn_logf(u));      // log2(-log2 u)
            }
        }
        // columns are visited in increasing order, so a strict comparison keeps the lowest column on ties
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float sc = fmaf(x[i], k, -g[i]);
            if (col0[v] + i < vocab && sc > best) { best = sc; best_i = col0[v] + i; }
        }
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float os = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(best_i, off, 64);
        better(best, best_i, os, oi);
    }
    __shared__ float sh[4];
    __shared__ int shi[4];
    if (lane == 0) { sh[wave] = best; shi[wave] = best_i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w) better(best, best_i, sh[w], shi[w]);
        part_best[static_cast<int64_t>(b) * nchunks + chunk] = best;
        part_idx[static_cast<int64_t>(b) * nchunks + chunk] = best_i;
    }
}

__global__ __launch_bounds__(kWave) void sampler_pick_kernel(
    const float *__restrict__ part_best, const int32_t *__restrict__ part_idx,
    int64_t *__restrict__ out_tokens, int32_t nchunks) {
    const int b = blockIdx.x;
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int c = threadIdx.x; c < nchunks; c += kWave)
        better(best, best_i, part_best[static_cast<int64_t>(b) * nchunks + c],
               part_idx[static_cast<int64_t>(b) * nchunks + c]);
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float os = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(best_i, off, 64);
        better(best, best_i, os, oi);
    }
    if (threadIdx.x == 0) out_tokens[b] = (best_i == 0x7fffffff) ? 0 : static_cast<int64_t>(best_i);
}

}  // namespace nva

extern "C" size_t nva_sample_workspace_bytes(int32_t batch, int32_t vocab) {
    if (batch <= 0 || vocab <= 0) return 0;
    return static_cast<size_t>(batch) * nva::samp_chunks(vocab) * 4 * sizeof(float);
}

extern "C" int nva_sample(const void *logits, int64_t logits_row_stride, const float *temperatures,
                          const float *noise, int64_t noise_row_stride, uint64_t seed, uint64_t offset,
                          int64_t *out_tokens, void *workspace, size_t workspace_bytes, int32_t batch,
                          int32_t vocab, void *stream) {
    using namespace nva;
    if (batch < 0 || vocab <= 0) return NVA_ERR_BAD_SHAPE;
    if (batch == 0) return NVA_OK;
    if (batch > 65535) return NVA_ERR_BAD_SHAPE;
    if (!logits || !temperatures || !out_tokens || !workspace) return NVA_ERR_NULL_POINTER;
    if (logits_row_stride < vocab) return NVA_ERR_BAD_STRIDE;
    if (noise && noise_row_stride < vocab) return NVA_ERR_BAD_STRIDE;
    if (!aligned16(workspace)) return NVA_ERR_MISALIGNED;
    if (workspace_bytes < nva_sample_workspace_bytes(batch, vocab)) return NVA_ERR_WORKSPACE_TOO_SMALL;
    const int nchunks = samp_chunks(vocab);
    const size_t n = static_cast<size_t>(batch) * nchunks;
    float *part_max = static_cast<float *>(workspace);
    float *part_sum = part_max + n;
    float *part_best = part_sum + n;
    int32_t *part_idx = reinterpret_cast<int32_t *>(part_best + n);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bf16_t *lg = static_cast<const bf16_t *>(logits);
    if (noise == nullptr) {
        const int gchunks = gumbel_chunks(vocab);              // fewer, wider chunks: fits the same workspace
        hipLaunchKernelGGL(sampler_gumbel_kernel, dim3(gchunks, batch), dim3(kSampThreads), 0, s, lg,
                           logits_row_stride, temperatures, seed, offset, part_best, part_idx, vocab, gchunks);
        if (launch_status() != NVA_OK) return NVA_ERR_LAUNCH_FAILED;
        hipLaunchKernelGGL(sampler_pick_kernel, dim3(batch), dim3(kWave), 0, s, part_best, part_idx, out_tokens,
                           gchunks);
        return launch_status();
    }
    hipLaunchKernelGGL(sampler_partials_kernel, dim3(nchunks, batch), dim3(kSampThreads), 0, s, lg,
                       logits_row_stride, temperatures, part_max, part_sum, vocab, nchunks);
    if (launch_status() != NVA_OK) return NVA_ERR_LAUNCH_FAILED;
    hipLaunchKernelGGL(sampler_argmax_kernel, dim3(nchunks, batch), dim3(kSampThreads), 0, s, lg,
                       logits_row_stride, temperatures, noise, noise_row_stride, part_max,
                       part_sum, part_best, part_idx, vocab, nchunks);
    if (launch_status() != NVA_OK) return NVA_ERR_LAUNCH_FAILED;
    hipLaunchKernelGGL(sampler_pick_kernel, dim3(batch), dim3(kWave), 0, s, part_best, part_idx, out_tokens,
                       nchunks);
    return launch_status();
}
