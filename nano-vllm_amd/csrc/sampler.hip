// Temperature sampler for gfx950: one pass over the logits, one tiny merge per row.
//
// Replaces Sampler.forward of nanovllm/layers/sampler.py:10-15:
//     x = float(logits) / T;  p = softmax(x);  token = argmax_i p_i / max(E_i, 1e-10)
//
// A row of 151,936 logits is far too little work for one workgroup and 64..256 rows are too few
// workgroups for 256 CUs, so a row is cut into chunks of 8192 columns (one workgroup of 256 lanes,
// four 16-byte loads of 8 bf16 per lane, all issued before the first use, non-temporal: the logits
// are read exactly once).  sampler_chunk_kernel leaves one 16-byte record per (row, chunk);
// sampler_row_kernel (one wavefront per row) merges a row's records into the token.
//
// With a caller-supplied tensor of E ~ Exp(1) draws (replayable; used for parity) the score of
// column i is evaluated relative to the CHUNK maximum m_c, e_i = exp(x_i - m_c) / max(E_i, 1e-10)
// with the reference's true fp32 division by T, and the record keeps (m_c, sum exp, best e_i, its
// column).  The row merge scales every chunk's best by exp(m_c - M) / S: the same quantity
// softmax(x)_i / E_i the reference maximises, factored as exp(x_i - m_c) * exp(m_c - M) instead of
// exp(x_i - M), so the argmax can differ from the reference only where two scores agree to within
// a few fp32 roundings.  Ties go to the lowest column, as torch.argmax does.
//
// Without a noise tensor (what serving uses) there is nothing to replay against, and the token is
// drawn from the same categorical distribution softmax(x) by a tree of inverse-CDF draws over the
// columns in column order, every level with a uniform of its own (32 random bits, compared in
// double precision; a conditional probability below 2^-32 at some level is therefore not
// resolved, and sums are fp32):
//     row      -> chunk (8192 columns)   by the chunk weights s_c * exp2(m_c - M)   [row kernel]
//     chunk    -> slice (2048 columns)   by the four slice sums                     [chunk kernel]
//     slice    -> wavefront (512)        by the four wavefront sums
//     wavefront-> lane (8 columns)       by an inclusive scan over the 64 lanes
//     lane     -> column                 by a walk over its 8 weights
// The four in-chunk levels run in the chunk kernel on the weights it already holds in registers,
// so the logits are read once and the row kernel touches only the records.  Uniforms come from
// Philox4x32-10 keyed by (seed, offset): counter (row, 0x5a17, offset) for the row level, counter
// (row, 0x10000 + chunk, offset) for the four levels inside a chunk (one output word each).
// Temperature 0 = greedy argmax of the logits (an extension; nanovllm/sampling_params.py:11
// forbids it).  A row without any finite logit yields token 0.
// Algorithmic HBM bytes per row: vocab * 2 B (+ vocab * 4 B when the noise is read).
#include "nva_common.h"

#include <math.h>

#include <mutex>

namespace nva {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr int kSampThreads = 256;
constexpr int kSampWaves = kSampThreads / kWave;
constexpr int kSampVec = 4;                               // 16-byte logit loads per lane
constexpr int kSampSlice = kSampThreads * 8;              // 2048 columns: one load of the whole workgroup
constexpr int kSampChunk = kSampSlice * kSampVec;         // 8192 columns per workgroup
constexpr int kNoToken = 0x7fffffff;

__host__ __device__ inline int samp_chunks(int vocab) { return (vocab + kSampChunk - 1) / kSampChunk; }

// One record per (row, chunk), written by the chunk kernel and read by the row kernel.
//   noise:   {m_c, sum exp(x - m_c), best exp(x - m_c) / max(E, 1e-10), its column}
//   no noise:{m_c (base 2), sum exp2(y - m_c), unused, the column drawn inside the chunk}
//   greedy:  {unused, unused, largest logit, its column}
struct __attribute__((aligned(16))) SampRecord {
    float m, s, best;
    int32_t col;
};

struct Philox {
    // Philox4x32-10 (Salmon et al., SC'11): counter (c0..c3), key (k0,k1)
    __device__ static inline uint4 draw(uint4 c, uint2 k) {
#pragma unroll
        for (int r = 0; r < 10; ++r) {
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

// 32 random bits -> uniform in (0, 1), exact in double
__device__ __forceinline__ double unit_uniform(uint32_t r) { return (static_cast<double>(r) + 0.5) * 2.3283064365386963e-10; }

__device__ __forceinline__ void better(float &bs, int &bi, float s, int i) {
    // larger score wins, lower column wins ties (torch.argmax returns the first maximum)
    if (s > bs || (s == bs && i < bi)) { bs = s; bi = i; }
}

__device__ __forceinline__ void wave_best(float &best, int &best_i) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float os = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(best_i, off, 64);
        better(best, best_i, os, oi);
    }
}

// First index i in [0, 4) with w[i] > 0 whose running sum exceeds u * total; the last index of
// positive weight when rounding leaves the target beyond the last running sum; -1 if no weight is
// positive.  The same rule, level by level, is what the oracle restates in float64.
__device__ __forceinline__ int pick4(const float (&w)[4], double u) {
    const float total = (w[0] + w[1]) + (w[2] + w[3]);
    const double t = u * static_cast<double>(total);
    float run = 0.f;
    int pick = -1, live = -1;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        run += w[i];
        if (w[i] > 0.f) {
            live = i;
            if (pick < 0 && static_cast<double>(run) > t) pick = i;
        }
    }
    return pick >= 0 ? pick : live;
}

template <bool kNoise>
__global__ __launch_bounds__(kSampThreads) void sampler_chunk_kernel(
    const bf16_t *__restrict__ logits, int64_t row_stride, const float *__restrict__ temperatures,
    const float *__restrict__ noise, int64_t noise_row_stride, uint64_t seed, uint64_t offset,
    SampRecord *__restrict__ records, int32_t vocab, int32_t nchunks) {
    const int chunk = blockIdx.x;
    const int b = blockIdx.y;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const bf16_t *row = logits + static_cast<int64_t>(b) * row_stride;
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(row) & 15u) == 0);
    const float t_in = temperatures[b];
    const bool greedy = (t_in == 0.f);

    // ---- every load of the chunk goes out before the first use ----------------------------------
    u32x4_t raw[kSampVec];
    int col0[kSampVec];
    bool full[kSampVec];
#pragma unroll
    for (int v = 0; v < kSampVec; ++v) {
        col0[v] = chunk * kSampChunk + v * kSampSlice + tid * 8;
        full[v] = vec_ok && col0[v] + 8 <= vocab;
        raw[v] = u32x4_t{0u, 0u, 0u, 0u};
        if (full[v]) raw[v] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(row + col0[v]));
    }
    float e[kSampVec][8];                                  // noise, where it is read
    if (kNoise && !greedy) {
        const float *nrow = noise + static_cast<int64_t>(b) * noise_row_stride;
        const bool nvec_ok = ((reinterpret_cast<uintptr_t>(nrow) & 15u) == 0);
#pragma unroll
        for (int v = 0; v < kSampVec; ++v) {
            if (nvec_ok && col0[v] + 8 <= vocab) {
                const f32x4_t a = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(nrow + col0[v]));
                const f32x4_t c = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(nrow + col0[v] + 4));
#pragma unroll
                for (int i = 0; i < 4; ++i) { e[v][i] = a[i]; e[v][4 + i] = c[i]; }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) e[v][i] = (col0[v] + i < vocab) ? nrow[col0[v] + i] : 1.f;
            }
        }
    }
    float x[kSampVec][8];                                  // columns past the row end read as -inf
#pragma unroll
    for (int v = 0; v < kSampVec; ++v) {
        if (full[v]) {
            unpack8(make_uint4(raw[v][0], raw[v][1], raw[v][2], raw[v][3]), x[v]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) x[v][i] = (col0[v] + i < vocab) ? bf16_to_f32(row[col0[v] + i]) : -INFINITY;
        }
    }

    __shared__ float sh_max[kSampWaves];
    __shared__ float sh_sum[kSampWaves][kSampVec];
    __shared__ float sh_best[kSampWaves];
    __shared__ int sh_col[kSampWaves];
    SampRecord *rec = records + static_cast<int64_t>(b) * nchunks + chunk;

    if (greedy) {                                          // row-uniform branch: chunk arg-max of the logits
        float best = -INFINITY;
        int best_i = kNoToken;
#pragma unroll
        for (int v = 0; v < kSampVec; ++v)
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (col0[v] + i < vocab && x[v][i] > best) { best = x[v][i]; best_i = col0[v] + i; }
        wave_best(best, best_i);
        if (lane == 0) { sh_best[wave] = best; sh_col[wave] = best_i; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < kSampWaves; ++w) better(best, best_i, sh_best[w], sh_col[w]);
            *rec = SampRecord{0.f, 0.f, best, best_i};
        }
        return;
    }

    // ---- x / T (noise: the reference's division; otherwise folded into the base-2 exponent) ------
    const float k = 1.4426950408889634f / t_in;
    float m = -INFINITY;
#pragma unroll
    for (int v = 0; v < kSampVec; ++v)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            x[v][i] = kNoise ? x[v][i] / t_in : x[v][i] * k;
            m = fmaxf(m, x[v][i]);
        }
    m = wave_max(m);
    if (lane == 0) sh_max[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(sh_max[0], sh_max[1]), fmaxf(sh_max[2], sh_max[3]));
    const float mm = (m == -INFINITY) ? 0.f : m;           // a chunk of -inf logits: every weight is 0

    if (kNoise) {
        float ssum = 0.f, best = -INFINITY;
        int best_i = kNoToken;
#pragma unroll
        for (int v = 0; v < kSampVec; ++v)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float ex = expf(x[v][i] - mm);       // exp(-inf) = 0 past the row end
                ssum += ex;
                if (col0[v] + i < vocab) better(best, best_i, ex / fmaxf(e[v][i], 1e-10f), col0[v] + i);
            }
        ssum = wave_sum(ssum);
        wave_best(best, best_i);
        if (lane == 0) { sh_sum[wave][0] = ssum; sh_best[wave] = best; sh_col[wave] = best_i; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < kSampWaves; ++w) better(best, best_i, sh_best[w], sh_col[w]);
            *rec = SampRecord{m, (sh_sum[0][0] + sh_sum[1][0]) + (sh_sum[2][0] + sh_sum[3][0]), best, best_i};
        }
        return;
    }

    // ---- no noise tensor: weights, and the draw inside the chunk -----------------------------------
    // (the counter is wave-uniform, so the generator runs on the scalar unit beside the exponentials)
    const uint4 r = Philox::draw(make_uint4(static_cast<uint32_t>(b), 0x10000u + static_cast<uint32_t>(chunk),
                                            static_cast<uint32_t>(offset), static_cast<uint32_t>(offset >> 32)),
                                 make_uint2(static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32)));
    float part[kSampVec];                                  // this lane's 8-column sums, one per slice
#pragma unroll
    for (int v = 0; v < kSampVec; ++v) {
        float p = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            x[v][i] = __builtin_amdgcn_exp2f(x[v][i] - mm);    // from here on x holds the weights
            p += x[v][i];
        }
        part[v] = p;
    }
#pragma unroll
    for (int v = 0; v < kSampVec; ++v) {
        const float ws = wave_sum(part[v]);
        if (lane == 0) sh_sum[wave][v] = ws;
    }
    __syncthreads();
    float slice_sum[kSampVec];
#pragma unroll
    for (int v = 0; v < kSampVec; ++v) slice_sum[v] = (sh_sum[0][v] + sh_sum[1][v]) + (sh_sum[2][v] + sh_sum[3][v]);
    const float chunk_sum = (slice_sum[0] + slice_sum[1]) + (slice_sum[2] + slice_sum[3]);
    const int vsel = pick4(slice_sum, unit_uniform(r.x));                     // workgroup-uniform
    if (vsel < 0) {                                        // no positive weight: the chunk can never be chosen
        if (tid == 0) *rec = SampRecord{m, 0.f, 0.f, min(chunk * kSampChunk, vocab - 1)};
        return;
    }
    const float wsum[kSampWaves] = {sh_sum[0][vsel], sh_sum[1][vsel], sh_sum[2][vsel], sh_sum[3][vsel]};
    const int wsel = pick4(wsum, unit_uniform(r.y));                          // > = 0: the slice has weight
    if (wave != wsel) return;                              // (wave-uniform; no barrier follows)
    const float mine = vsel == 0 ? part[0] : vsel == 1 ? part[1] : vsel == 2 ? part[2] : part[3];
    float incl = mine;                                     // inclusive scan over the 64 lanes
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float up = __shfl_up(incl, off, 64);
        if (lane >= off) incl += up;
    }
    const double t3 = unit_uniform(r.z) * static_cast<double>(__shfl(incl, 63, 64));
    const uint64_t live = __builtin_amdgcn_ballot_w64(mine > 0.f);            // != 0: the wavefront has weight
    const uint64_t hit = __builtin_amdgcn_ballot_w64(mine > 0.f && static_cast<double>(incl) > t3);
    const int lsel = hit != 0 ? __builtin_ctzll(hit) : 63 - __builtin_clzll(live);
    if (lane != lsel) return;
    float w8[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        w8[i] = vsel == 0 ? x[0][i] : vsel == 1 ? x[1][i] : vsel == 2 ? x[2][i] : x[3][i];
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) total += w8[i];
    const double t4 = unit_uniform(r.w) * static_cast<double>(total);
    float run = 0.f;
    int isel = -1, ilive = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        run += w8[i];
        if (w8[i] > 0.f) {
            ilive = i;
            if (isel < 0 && static_cast<double>(run) > t4) isel = i;
        }
    }
    if (isel < 0) isel = ilive;
    *rec = SampRecord{m, chunk_sum, 0.f, chunk * kSampChunk + vsel * kSampSlice + tid * 8 + isel};
}

// One wavefront per row: merges the row's chunk records into the token.
__global__ __launch_bounds__(kSampThreads) void sampler_row_kernel(
    const SampRecord *__restrict__ records, const float *__restrict__ temperatures, int32_t with_noise,
    uint64_t seed, uint64_t offset, int64_t *__restrict__ out_tokens, int32_t batch, int32_t nchunks) {
    const int lane = threadIdx.x & 63;
    const int b = blockIdx.x * kSampWaves + (threadIdx.x >> 6);
    if (b >= batch) return;                                // wave-uniform; the kernel has no barrier
    const SampRecord *rec = records + static_cast<int64_t>(b) * nchunks;
    const float t_in = temperatures[b];
    if (t_in == 0.f || with_noise) {
        // greedy: best logit; noise: best of exp(x - m_c) / E scaled to the row maximum and row sum
        float m = -INFINITY;
        if (t_in != 0.f) {
            for (int c = lane; c < nchunks; c += kWave) m = fmaxf(m, rec[c].m);
            m = wave_max(m);
        }
        float s = 0.f;
        if (t_in != 0.f && m != -INFINITY) {
            for (int c = lane; c < nchunks; c += kWave) s += rec[c].s * expf(rec[c].m - m);
            s = wave_sum(s);
        }
        float best = -INFINITY;
        int best_i = kNoToken;
        for (int c = lane; c < nchunks; c += kWave) {
            const SampRecord r = rec[c];
            if (r.col == kNoToken) continue;
            float score = r.best;
            if (t_in != 0.f) score = (m == -INFINITY) ? 0.f : r.best * expf(r.m - m) / s;
            better(best, best_i, score, r.col);
        }
        wave_best(best, best_i);
        if (lane == 0) out_tokens[b] = (best_i == kNoToken) ? 0 : static_cast<int64_t>(best_i);
        return;
    }
    // ---- no noise tensor: the chunk is drawn by the chunk weights, the column inside it is in the record
    float m = -INFINITY;
    for (int c = lane; c < nchunks; c += kWave) m = fmaxf(m, rec[c].m);
    m = wave_max(m);
    if (m == -INFINITY) {                                  // no finite logit in the row
        if (lane == 0) out_tokens[b] = 0;
        return;
    }
    double total = 0.0;
    for (int c = lane; c < nchunks; c += kWave)
        total += static_cast<double>(rec[c].s * __builtin_amdgcn_exp2f(rec[c].m - m));
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) total += __shfl_xor(total, off, 64);
    const uint4 r = Philox::draw(make_uint4(static_cast<uint32_t>(b), 0x5a17u, static_cast<uint32_t>(offset),
                                            static_cast<uint32_t>(offset >> 32)),
                                 make_uint2(static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32)));
    const double target = unit_uniform(r.x) * total;
    double carry = 0.0;
    int pick = -1, last_live = -1;
    for (int base = 0; base < nchunks; base += kWave) {    // running sum in chunk order, 64 chunks at a time
        const int c = base + lane;
        const float w = c < nchunks ? rec[c].s * __builtin_amdgcn_exp2f(rec[c].m - m) : 0.f;
        double incl = static_cast<double>(w);
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const double up = __shfl_up(incl, off, 64);
            if (lane >= off) incl += up;
        }
        incl += carry;
        const uint64_t live = __builtin_amdgcn_ballot_w64(w > 0.f);
        const uint64_t hit = __builtin_amdgcn_ballot_w64(w > 0.f && incl > target);
        if (live != 0) last_live = base + 63 - __builtin_clzll(live);
        if (pick < 0 && hit != 0) pick = base + __builtin_ctzll(hit);
        carry = __shfl(incl, 63, 64);
    }
    if (pick < 0) pick = last_live;                        // rounding: the target lies beyond the last running sum
    if (lane == 0) out_tokens[b] = pick < 0 ? 0 : static_cast<int64_t>(rec[pick].col);
}

static int launch_sample(const bf16_t *logits, int64_t logits_row_stride, const float *temperatures,
                         const float *noise, int64_t noise_row_stride, uint64_t seed, uint64_t offset,
                         int64_t *out_tokens, SampRecord *records, int32_t batch, int32_t vocab, hipStream_t s) {
    const int nchunks = samp_chunks(vocab);
    if (noise)
        hipLaunchKernelGGL(sampler_chunk_kernel<true>, dim3(nchunks, batch), dim3(kSampThreads), 0, s, logits,
                           logits_row_stride, temperatures, noise, noise_row_stride, seed, offset, records, vocab, nchunks);
    else
        hipLaunchKernelGGL(sampler_chunk_kernel<false>, dim3(nchunks, batch), dim3(kSampThreads), 0, s, logits,
                           logits_row_stride, temperatures, noise, noise_row_stride, seed, offset, records, vocab, nchunks);
    if (launch_status() != NVA_OK) return NVA_ERR_LAUNCH_FAILED;
    hipLaunchKernelGGL(sampler_row_kernel, dim3((batch + kSampWaves - 1) / kSampWaves), dim3(kSampThreads), 0, s, records,
                       temperatures, noise ? 1 : 0, seed, offset, out_tokens, batch, nchunks);
    return launch_status();
}

static int check_sample_args(const void *logits, int64_t logits_row_stride, const float *temperatures,
                             const float *noise, int64_t noise_row_stride, const int64_t *out_tokens,
                             int32_t batch, int32_t vocab) {
    if (batch < 0 || vocab <= 0) return NVA_ERR_BAD_SHAPE;
    if (batch > 65535) return NVA_ERR_BAD_SHAPE;
    if (batch == 0) return NVA_OK;
    if (!logits || !temperatures || !out_tokens) return NVA_ERR_NULL_POINTER;
    if (logits_row_stride < vocab) return NVA_ERR_BAD_STRIDE;
    if (noise && noise_row_stride < vocab) return NVA_ERR_BAD_STRIDE;
    return NVA_OK;
}

}  // namespace nva

extern "C" size_t nva_sample_workspace_bytes(int32_t batch, int32_t vocab) {
    if (batch <= 0 || vocab <= 0) return 0;
    return static_cast<size_t>(batch) * nva::samp_chunks(vocab) * sizeof(nva::SampRecord);
}

extern "C" int nva_sample(const void *logits, int64_t logits_row_stride, const float *temperatures,
                          const float *noise, int64_t noise_row_stride, uint64_t seed, uint64_t offset,
                          int64_t *out_tokens, void *workspace, size_t workspace_bytes, int32_t batch,
                          int32_t vocab, void *stream) {
    using namespace nva;
    const int rc = check_sample_args(logits, logits_row_stride, temperatures, noise, noise_row_stride, out_tokens,
                                     batch, vocab);
    if (rc != NVA_OK || batch == 0) return rc;
    if (!workspace) return NVA_ERR_NULL_POINTER;
    if (!aligned16(workspace)) return NVA_ERR_MISALIGNED;
    if (workspace_bytes < nva_sample_workspace_bytes(batch, vocab)) return NVA_ERR_WORKSPACE_TOO_SMALL;
    return launch_sample(static_cast<const bf16_t *>(logits), logits_row_stride, temperatures, noise, noise_row_stride,
                         seed, offset, out_tokens, static_cast<SampRecord *>(workspace), batch, vocab,
                         static_cast<hipStream_t>(stream));
}

// ---- the same sampler for callers that cannot allocate --------------------------------------------
// The chunk records live in a file-scope device array instead of a caller-supplied workspace.  Each
// GPU the library runs on holds its own copy of the array (2 MiB) until the process ends.  In host
// code the array's name is only a handle: its device address is looked up once per device with
// hipGetSymbolAddress and that pointer is what the kernels receive.
namespace nva {

constexpr int kStaticRecords = NVA_SAMPLE_STATIC_MAX_RECORDS;
constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[static_cast<size_t>(kStaticRecords) * sizeof(SampRecord)];

static std::mutex g_scratch_mutex;
static SampRecord *g_scratch_ptr[kMaxDevices] = {};       // device address of `scratch` on each device

// Device address of this device's copy of `scratch`; nullptr (and *status set) on failure.
static SampRecord *static_scratch(int *status) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        *status = NVA_ERR_NO_DEVICE;
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
            (void)hipGetLastError();
            *status = NVA_ERR_LAUNCH_FAILED;
            return nullptr;
        }
        g_scratch_ptr[dev] = static_cast<SampRecord *>(ptr);
    }
    return g_scratch_ptr[dev];
}

}  // namespace nva

extern "C" int nva_sample_static(const void *logits, int64_t logits_row_stride, const float *temperatures,
                                 const float *noise, int64_t noise_row_stride, uint64_t seed, uint64_t offset,
                                 int64_t *out_tokens, int32_t batch, int32_t vocab, void *stream) {
    using namespace nva;
    const int rc = check_sample_args(logits, logits_row_stride, temperatures, noise, noise_row_stride, out_tokens,
                                     batch, vocab);
    if (rc != NVA_OK || batch == 0) return rc;
    if (static_cast<int64_t>(batch) * samp_chunks(vocab) > kStaticRecords) return NVA_ERR_SCRATCH_TOO_SMALL;
    int status = NVA_OK;
    SampRecord *records = static_scratch(&status);
    if (records == nullptr) return status;
    // every record the row kernel reads is written by the chunk kernel of the same call: nothing to clear
    return launch_sample(static_cast<const bf16_t *>(logits), logits_row_stride, temperatures, noise, noise_row_stride,
                         seed, offset, out_tokens, records, batch, vocab, static_cast<hipStream_t>(stream));
}
