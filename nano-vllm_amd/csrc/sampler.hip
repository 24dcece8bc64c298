// Temperature sampler for gfx950.
//
// Replaces Sampler.forward of nanovllm/layers/sampler.py:10-15:
//     x = float(logits) / T;  p = softmax(x);  token = argmax_i p_i / max(E_i, 1e-10)
// With a caller-supplied tensor of E ~ Exp(1) draws (replayable; used for parity) the arithmetic
// keeps the reference's operation order -- true fp32 division by T, exp(x - rowmax) / rowsum, then
// the division by the clamped noise -- so the argmax can only differ from the reference where two
// scores are equal to within fp32 rounding.  Without one (what serving uses) the token is drawn
// from the same categorical distribution by inverse CDF with one in-kernel uniform per row.
//
// A row of 151,936 logits is far too little work for one workgroup and 64..256 rows are
// too few workgroups for 256 CUs, so a row is cut into chunks (one workgroup of 256 lanes each,
// 16-byte loads of 8 bf16 per lane).
// With a caller-supplied noise tensor, chunks of 2048 columns:
//   pass 1  per (chunk, row): chunk max and sum exp(x - chunk max)          -> workspace
//   pass 2  per (chunk, row): merge the row's partials into (max, sum), then
//           best p_i / E_i and its column inside the chunk                   -> workspace
//   pass 3  per row: best chunk, lowest column on ties                       -> int64 token
// Pass 2 re-reads the logits (2 B/col) that pass 1 pulled through L2 / Infinity Cache.
// Without noise, chunks of 8192 columns: one pass for the chunk sums, then a per-row selection
// that re-reads a single chunk (see sampler_cdf_sums_kernel below).
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

// ---- in-kernel randomness: one uniform per row, inverse-CDF draw -----------------------------
// Without a noise tensor to replay against, the exponential race is replaced by the textbook
// draw from the same categorical distribution: with w_i = exp2((x_i - M) * log2(e)/T) and one
// uniform u per row, the token is the first i (in column order) whose running sum of w exceeds
// u * sum(w).  One Philox call per ROW instead of one random number and two logarithms per
// column leaves a multiply, an exponential and an add per column -- the pass over the logits
// runs at memory speed.
//   pass A  per (8192-column chunk, row): chunk max m_c, s_c = sum exp2(y - m_c), and the chunk's
//           arg-max (used by temperature-0 rows)                                -> workspace
//   pass B  per row: M = max m_c, chunk weights s_c * exp2(m_c - M), their running sum picks
//           the chunk; its 8192 logits are read once more (32 consecutive columns per lane), a
//           workgroup scan picks the lane and the lane walks its columns        -> int64 token
// Rounding can leave the target a hair beyond the last running sum; it then falls on the last
// column of positive weight.  A row without any finite logit yields token 0.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
constexpr int kCdfVec = 4;                                    // 16-byte loads per lane in pass A
constexpr int kCdfChunk = kSampChunk * kCdfVec;               // 8192 columns per workgroup

__host__ __device__ inline int cdf_chunks(int vocab) { return (vocab + kCdfChunk - 1) / kCdfChunk; }

__device__ __forceinline__ float block_max4(float v, float *sh, int lane, int wave) {
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    return fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
}

__device__ __forceinline__ float block_sum4(float v, float *sh, int lane, int wave) {
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    return (sh[0] + sh[1]) + (sh[2] + sh[3]);
}

__global__ __launch_bounds__(kSampThreads) void sampler_cdf_sums_kernel(
    const bf16_t *__restrict__ logits, int64_t row_stride, const float *__restrict__ temperatures,
    float *__restrict__ part_max, float *__restrict__ part_sum, float *__restrict__ part_best,
    int32_t *__restrict__ part_idx, int32_t vocab, int32_t nchunks) {
    const int chunk = blockIdx.x;
    const int b = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const bf16_t *row = logits + static_cast<int64_t>(b) * row_stride;
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(row) & 15u) == 0);
    const float t_in = temperatures[b];
    const bool greedy = (t_in == 0.f);
    const float k = greedy ? 1.f : 1.4426950408889634f / t_in;
    u32x4_t raw[kCdfVec];
    int col0[kCdfVec];
#pragma unroll
    for (int v = 0; v < kCdfVec; ++v) {
        col0[v] = chunk * kCdfChunk + v * kSampChunk + threadIdx.x * 8;
        raw[v] = u32x4_t{0u, 0u, 0u, 0u};
        // (streamed once: non-temporal, so that the rows do not displace one another in L2)
        if (vec_ok && col0[v] + 8 <= vocab) raw[v] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(row + col0[v]));
    }
    float y[kCdfVec][8];
    float m = -INFINITY;
#pragma unroll
    for (int v = 0; v < kCdfVec; ++v) {
        if (vec_ok && col0[v] + 8 <= vocab) {
            unpack8(make_uint4(raw[v][0], raw[v][1], raw[v][2], raw[v][3]), y[v]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) y[v][i] = (col0[v] + i < vocab) ? bf16_to_f32(row[col0[v] + i]) : -INFINITY;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            y[v][i] *= k;
            m = fmaxf(m, y[v][i]);
        }
    }
    __shared__ float sh[4];
    __shared__ int shi[4];
    if (greedy) {                                        // row-uniform branch: chunk arg-max, lowest column on ties
        float best = -INFINITY;
        int best_i = 0x7fffffff;
#pragma unroll
        for (int v = 0; v < kCdfVec; ++v)
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (col0[v] + i < vocab && y[v][i] > best) { best = y[v][i]; best_i = col0[v] + i; }
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
        return;
    }
    m = block_max4(m, sh, lane, wave);
    const float mm = (m == -INFINITY) ? 0.f : m;           // a chunk of -inf logits sums to 0
    float ssum = 0.f;
#pragma unroll
    for (int v = 0; v < kCdfVec; ++v) {
        float part = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) part += __builtin_amdgcn_exp2f(y[v][i] - mm);     // exp2(-inf) = 0 past the row end
        ssum += part;
    }
    ssum = block_sum4(ssum, sh, lane, wave);
    if (threadIdx.x == 0) {
        part_max[static_cast<int64_t>(b) * nchunks + chunk] = m;
        part_sum[static_cast<int64_t>(b) * nchunks + chunk] = ssum;
    }
}

__global__ __launch_bounds__(kSampThreads) void sampler_cdf_select_kernel(
    const bf16_t *__restrict__ logits, int64_t row_stride, const float *__restrict__ temperatures,
    uint64_t seed, uint64_t offset, const float *__restrict__ part_max, const float *__restrict__ part_sum,
    const float *__restrict__ part_best, const int32_t *__restrict__ part_idx,
    int64_t *__restrict__ out_tokens, int32_t vocab, int32_t nchunks) {
    const int b = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float t_in = temperatures[b];
    __shared__ float sh[4];
    __shared__ int sh_pick[1];
    if (t_in == 0.f) {                                   // greedy: best chunk, lowest column on ties
        if (wave == 0) {
            float best = -INFINITY;
            int best_i = 0x7fffffff;
            for (int c = lane; c < nchunks; c += kWave)
                better(best, best_i, part_best[static_cast<int64_t>(b) * nchunks + c],
                       part_idx[static_cast<int64_t>(b) * nchunks + c]);
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const float os = __shfl_xor(best, off, 64);
                const int oi = __shfl_xor(best_i, off, 64);
                better(best, best_i, os, oi);
            }
            if (lane == 0) out_tokens[b] = (best_i == 0x7fffffff) ? 0 : static_cast<int64_t>(best_i);
        }
        return;
    }
    const float k = 1.4426950408889634f / t_in;
    // ---- wavefront 0: row maximum, chunk weights relative to it, and the chunk that holds u * total ----
    if (wave == 0) {
        const float *pm = part_max + static_cast<int64_t>(b) * nchunks;
        const float *ps = part_sum + static_cast<int64_t>(b) * nchunks;
        float m = -INFINITY;
        for (int c = lane; c < nchunks; c += kWave) m = fmaxf(m, pm[c]);
        m = wave_max(m);
        int pick = -2;                                   // -2: no finite logit in the row
        float rest_in_chunk = 0.f;
        if (m != -INFINITY) {
            float total = 0.f;
            for (int c = lane; c < nchunks; c += kWave) total += ps[c] * __builtin_amdgcn_exp2f(pm[c] - m);
            total = wave_sum(total);
            // one uniform per row, in (0, 1): 24 random bits plus one half
            const uint2 key = make_uint2(static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32));
            const uint4 r = Philox::draw(make_uint4(static_cast<uint32_t>(b), 0x5a17u, static_cast<uint32_t>(offset),
                                                    static_cast<uint32_t>(offset >> 32)), key);
            const float u = (static_cast<float>(r.x >> 8) + 0.5f) * 5.9604644775390625e-8f;
            const float target = u * total;
            // running sum in chunk order, 64 chunks at a time
            float carry = 0.f;
            int last_live = 0;
            pick = -1;
            for (int base = 0; base < nchunks; base += kWave) {
                const int c = base + lane;
                const float w = c < nchunks ? ps[c] * __builtin_amdgcn_exp2f(pm[c] - m) : 0.f;
                float incl = w;
#pragma unroll
                for (int off = 1; off < 64; off <<= 1) {
                    const float up = __shfl_up(incl, off, 64);
                    if (lane >= off) incl += up;
                }
                incl += carry;
                const uint64_t live = __builtin_amdgcn_ballot_w64(w > 0.f);
                const uint64_t hit = __builtin_amdgcn_ballot_w64(w > 0.f && incl > target);
                if (live != 0) last_live = base + 63 - __builtin_clzll(live);
                if (pick < 0 && hit != 0) {
                    const int l = __builtin_ctzll(hit);
                    pick = base + l;
                    rest_in_chunk = target - __shfl(incl - w, l, 64);     // what is left to walk inside the chunk
                }
                carry = __shfl(incl, 63, 64);
            }
            if (pick < 0) { pick = last_live; rest_in_chunk = INFINITY; }   // rounding: beyond the last running sum
        }
        if (lane == 0) { sh_pick[0] = pick; sh[0] = rest_in_chunk; sh[1] = m; }
    }
    __syncthreads();
    const int chunk = sh_pick[0];
    const float rest = sh[0];
    const float m = sh[1];
    if (chunk == -2) {
        if (threadIdx.x == 0) out_tokens[b] = 0;
        return;
    }
    // ---- inside the chunk: 32 consecutive columns per lane, scan over the 256 lanes -------------
    const bf16_t *row = logits + static_cast<int64_t>(b) * row_stride;
    const int c0 = chunk * kCdfChunk + threadIdx.x * 32;
    float w[32];
    float mine = 0.f;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        float x[8];
        const int cc = c0 + v * 8;
        if (((reinterpret_cast<uintptr_t>(row + cc) & 15u) == 0) && cc + 8 <= vocab) {
            unpack8(*reinterpret_cast<const uint4 *>(row + cc), x);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = (cc + i < vocab) ? bf16_to_f32(row[cc + i]) : -INFINITY;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            w[v * 8 + i] = __builtin_amdgcn_exp2f(x[i] * k - m);
            mine += w[v * 8 + i];
        }
    }
    // inclusive scan of `mine` over the workgroup, in lane order
    float incl = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float up = __shfl_up(incl, off, 64);
        if (lane >= off) incl += up;
    }
    if (lane == 63) sh[wave] = incl;
    __syncthreads();
    for (int wv = 0; wv < wave; ++wv) incl += sh[wv];
    // owner: the first lane whose running sum exceeds `rest` (its span then contains it); if rounding
    // put `rest` beyond the chunk's total, the last lane of positive weight
    int first = (mine > 0.f && incl > rest) ? static_cast<int>(threadIdx.x) : 0x7fffffff;
    int live = (mine > 0.f) ? static_cast<int>(threadIdx.x) : -1;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        first = min(first, __shfl_xor(first, off, 64));
        live = max(live, __shfl_xor(live, off, 64));
    }
    __shared__ int sh_first[4], sh_live[4];
    if (lane == 0) { sh_first[wave] = first; sh_live[wave] = live; }
    __syncthreads();
    first = min(min(sh_first[0], sh_first[1]), min(sh_first[2], sh_first[3]));
    live = max(max(sh_live[0], sh_live[1]), max(sh_live[2], sh_live[3]));
    const int owner = first != 0x7fffffff ? first : live;
    if (owner < 0) {                                     // every weight of the chunk underflowed: its first column
        if (threadIdx.x == 0) out_tokens[b] = min(chunk * kCdfChunk, vocab - 1);
        return;
    }
    if (static_cast<int>(threadIdx.x) == owner) {
        float run = incl - mine;
        int tok = -1, last = c0;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            if (w[j] > 0.f) last = c0 + j;
            if (tok < 0 && w[j] > 0.f && run + w[j] > rest) tok = c0 + j;
            run += w[j];
        }
        out_tokens[b] = tok < 0 ? last : tok;
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
        const int cchunks = cdf_chunks(vocab);                 // fewer, wider chunks: fits the same workspace
        hipLaunchKernelGGL(sampler_cdf_sums_kernel, dim3(cchunks, batch), dim3(kSampThreads), 0, s, lg,
                           logits_row_stride, temperatures, part_max, part_sum, part_best, part_idx, vocab, cchunks);
        if (launch_status() != NVA_OK) return NVA_ERR_LAUNCH_FAILED;
        hipLaunchKernelGGL(sampler_cdf_select_kernel, dim3(batch), dim3(kSampThreads), 0, s, lg, logits_row_stride,
                           temperatures, seed, offset, part_max, part_sum, part_best, part_idx, out_tokens, vocab,
                           cchunks);
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
