// Temperature sampler for gfx950: one pass over the logits, one tiny merge per row.
//
// Replaces Sampler.forward of nanovllm/layers/sampler.py:10-15:
//     x = float(logits) / T;  p = softmax(x);  token = argmax_i p_i / max(E_i, 1e-10)
//
// A row of 151,936 logits is far too little work for one workgroup and 64..256 rows are too few
// workgroups for 256 CUs, so a row is cut into chunks (one workgroup of 256 lanes each, 16-byte
// loads of 8 bf16 per lane, all issued before the first use, non-temporal: the logits are read
// exactly once).  sampler_chunk_kernel leaves one 16-byte record per (row, chunk);
// sampler_row_kernel (one wavefront per row) merges a row's records into the token.
//
// With a caller-supplied tensor of E ~ Exp(1) draws (replayable; used for parity; chunks of 4096
// columns) the score of column i is evaluated relative to the CHUNK maximum m_c,
// e_i = exp(x_i - m_c) / max(E_i, 1e-10), and the record keeps (m_c, sum exp, best e_i, its column).
// The two divisions per column (by T and by the noise) are a multiplication by 1/T and by a
// one-ulp hardware reciprocal: true fp32 divisions made this pass instruction-bound.  The row merge scales every chunk's best by
// exp(m_c - M) / S: the same quantity softmax(x)_i / E_i the reference maximises, factored as
// exp(x_i - m_c) * exp(m_c - M) instead of exp(x_i - M), so the argmax can differ from the
// reference only where two scores agree to within a few fp32 roundings.  Ties go to the lowest
// column, as torch.argmax does.
//
// Without a noise tensor (what serving uses; chunks of 8192 columns) there is nothing to replay
// against, and the token is drawn from the same categorical distribution softmax(x) by a tree of
// inverse-CDF draws, every level with a uniform of its own (32 random bits, compared in double
// precision; a conditional probability below 2^-32 at some level is therefore not resolved, and
// sums are fp32):
//     row       -> chunk (8192 columns)  by the chunk weights s_c * exp2(m_c - M)   [row kernel]
//     chunk     -> wavefront             by the four wavefront sums                 [chunk kernel]
//     wavefront -> lane                  by an inclusive scan over the 64 lane sums
//     lane      -> column                by a walk over the lane's 32 weights
// (lane t of a chunk owns columns 2048 v + 8 t + [0, 8) for v = 0..3, walked in that order).  The
// three in-chunk levels run in the chunk kernel, so the logits are read once and the row kernel
// touches only the records.  Only the packed bf16 logits stay in registers across the workgroup
// reductions (16 registers instead of 32 weights); for the last level the chosen lane hands them
// to its wavefront through LDS and 32 lanes recompute one weight each, bit for bit as summed
// (a serial walk by one lane costs a full wavefront's instruction stream, +40 % kernel time).
// Uniforms come from Philox4x32-10 keyed by (seed, offset): counter (row, 0x5a17, offset) for the
// row level, counter (row, 0x10000 + chunk, offset) for the levels inside a chunk (one output
// word each).  Temperature 0 = greedy argmax of the logits (an extension;
// nanovllm/sampling_params.py:11 forbids it).  A row without any finite logit yields token 0.
// Algorithmic HBM bytes per row: vocab * 2 B (+ vocab * 4 B when the noise is read).
#include "nva_common.h"

#include <math.h>

#include <mutex>

namespace nva {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr int kSampThreads = 256;
constexpr int kSampWaves = kSampThreads / kWave;
constexpr int kSampSlice = kSampThreads * 8;              // 2048 columns: one 16-byte load per lane
constexpr int kDrawVec = 4;                               // no noise tensor: four loads per lane, 8192 columns per workgroup
constexpr int kNoiseVec = 2;                              // with noise: 4096 columns per workgroup (16 logits + 16 noise values per lane; 2048: 55.8 us, 4096: 48.0, 8192: 50.9 at 256 x 151,936)
constexpr int kNoToken = 0x7fffffff;

__host__ __device__ inline int samp_chunks(int vocab, int vec) { return (vocab + kSampSlice * vec - 1) / (kSampSlice * vec); }

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

// Makes the compiler forget what it knows about the packed logits, so that code after this point
// unpacks them again instead of keeping the 32 floats of an earlier pass alive in registers.
template <int kVec>
__device__ __forceinline__ void forget(u32x4_t (&raw)[kVec]) {
#pragma unroll
    for (int v = 0; v < kVec; ++v) asm volatile("" : "+v"(raw[v]));
}

// The 8 packed bf16 logits of columns [col0, col0 + 8): one 16-byte non-temporal load where the
// row allows it, else element by element; columns past the row end read as -inf (bf16 0xFF80).
__device__ __forceinline__ u32x4_t load_columns8(const bf16_t *row, bool vec_ok, int col0, int vocab) {
    if (vec_ok && col0 + 8 <= vocab) return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(row + col0));
    uint32_t h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = (col0 + i < vocab) ? row[col0 + i] : 0xFF80u;
    return u32x4_t{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
}

__device__ __forceinline__ void columns8(const u32x4_t &raw, float (&x)[8]) {
    unpack8(make_uint4(raw[0], raw[1], raw[2], raw[3]), x);
}

template <int kVec, bool kNoise>
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
    const int colbase = chunk * (kSampSlice * kVec) + tid * 8;      // slice v of this lane starts at colbase + v * kSampSlice

    // ---- every load of the chunk goes out before the first use ----------------------------------
    u32x4_t raw[kVec];
#pragma unroll
    for (int v = 0; v < kVec; ++v) raw[v] = load_columns8(row, vec_ok, colbase + v * kSampSlice, vocab);
    float e[kVec][8];                                      // noise, where it is read
    if (kNoise && !greedy) {
        const float *nrow = noise + static_cast<int64_t>(b) * noise_row_stride;
        const bool nvec_ok = ((reinterpret_cast<uintptr_t>(nrow) & 15u) == 0);
#pragma unroll
        for (int v = 0; v < kVec; ++v) {
            const int c0 = colbase + v * kSampSlice;
            if (nvec_ok && c0 + 8 <= vocab) {
                const f32x4_t a = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(nrow + c0));
                const f32x4_t c = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(nrow + c0 + 4));
#pragma unroll
                for (int i = 0; i < 4; ++i) { e[v][i] = a[i]; e[v][4 + i] = c[i]; }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) e[v][i] = (c0 + i < vocab) ? nrow[c0 + i] : 1.f;
            }
        }
    }

    __shared__ float sh_max[kSampWaves];
    __shared__ float sh_sum[kSampWaves];
    __shared__ float sh_best[kSampWaves];
    __shared__ int sh_col[kSampWaves];
    SampRecord *rec = records + static_cast<int64_t>(b) * nchunks + chunk;

    if (greedy) {                                          // row-uniform branch: chunk arg-max of the logits
        float best = -INFINITY;
        int best_i = kNoToken;
#pragma unroll
        for (int v = 0; v < kVec; ++v) {
            float x[8];
            const int c0 = colbase + v * kSampSlice;
            columns8(raw[v], x);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (c0 + i < vocab && x[i] > best) { best = x[i]; best_i = c0 + i; }
        }
        wave_best(best, best_i);
        if (lane == 0) { sh_best[wave] = best; sh_col[wave] = best_i; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < kSampWaves; ++w) better(best, best_i, sh_best[w], sh_col[w]);
            *rec = SampRecord{0.f, 0.f, best, best_i};
        }
        return;
    }

    // ---- chunk maximum of x / T (noise: the reference's division; otherwise the scale is folded
    //      into the base-2 exponent: y = x * log2(e) / T) ------------------------------------------
    const float k = 1.4426950408889634f / t_in;
    const float inv_t = 1.0f / t_in;                       // x * (1 / T): within one ulp of the reference's x / T, a tenth of its instructions
    float m = -INFINITY;
    float xt[kNoise ? kVec : 1][8];                        // noise: x / T, kept (8 values per lane); else recomputed from `raw`
#pragma unroll
    for (int v = 0; v < kVec; ++v) {
        float x[8];
        columns8(raw[v], x);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (kNoise) {
                xt[v][i] = x[i] * inv_t;
                m = fmaxf(m, xt[v][i]);
            } else {
                m = fmaxf(m, x[i]);                        // scaled once below: k > 0, so max(x) * k == max(x * k) bit for bit
            }
        }
    }
    if (!kNoise) m *= k;
    m = wave_max(m);
    if (lane == 0) sh_max[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(sh_max[0], sh_max[1]), fmaxf(sh_max[2], sh_max[3]));
    const float mm = (m == -INFINITY) ? 0.f : m;           // a chunk of -inf logits: every weight is 0
    if (!kNoise) forget(raw);

    if (kNoise) {
        float ssum = 0.f, best = -INFINITY;
        int best_i = kNoToken;
#pragma unroll
        for (int v = 0; v < kVec; ++v) {
            const int c0 = colbase + v * kSampSlice;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float ex = expf(xt[v][i] - mm);      // exp(-inf) = 0 past the row end
                ssum += ex;
                if (c0 + i < vocab) better(best, best_i, ex * __builtin_amdgcn_rcpf(fmaxf(e[v][i], 1e-10f)), c0 + i);   // (one-ulp reciprocal)
            }
        }
        ssum = wave_sum(ssum);
        wave_best(best, best_i);
        if (lane == 0) { sh_sum[wave] = ssum; sh_best[wave] = best; sh_col[wave] = best_i; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < kSampWaves; ++w) better(best, best_i, sh_best[w], sh_col[w]);
            *rec = SampRecord{m, (sh_sum[0] + sh_sum[1]) + (sh_sum[2] + sh_sum[3]), best, best_i};
        }
        return;
    }

    // ---- no noise tensor: the lane sums, and the draw inside the chunk -----------------------------
    // (the counter is wave-uniform, so the generator runs on the scalar unit beside the exponentials)
    const uint4 r = Philox::draw(make_uint4(static_cast<uint32_t>(b), 0x10000u + static_cast<uint32_t>(chunk),
                                            static_cast<uint32_t>(offset), static_cast<uint32_t>(offset >> 32)),
                                 make_uint2(static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32)));
    float mine = 0.f;                                      // sum of this lane's weights, slice by slice, column by column
#pragma unroll
    for (int v = 0; v < kVec; ++v) {
        float x[8];
        columns8(raw[v], x);
#pragma unroll
        for (int i = 0; i < 8; ++i) mine += __builtin_amdgcn_exp2f(x[i] * k - mm);    // exp2(-inf) = 0 past the row end
    }
    const float wave_total = wave_sum(mine);
    if (lane == 0) sh_sum[wave] = wave_total;
    __syncthreads();
    const float wsum[kSampWaves] = {sh_sum[0], sh_sum[1], sh_sum[2], sh_sum[3]};
    const int wsel = pick4(wsum, unit_uniform(r.x));       // workgroup-uniform
    if (wsel < 0) {                                        // no positive weight: the chunk can never be chosen
        if (tid == 0) *rec = SampRecord{m, 0.f, 0.f, min(chunk * (kSampSlice * kVec), vocab - 1)};
        return;
    }
    if (wave != wsel) return;                              // (wave-uniform; no barrier follows)
    // ---- the chosen wavefront: which lane (inclusive scan of the 64 lane sums) -----------------
    float incl = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float up = __shfl_up(incl, off, 64);
        if (lane >= off) incl += up;
    }
    const double t2 = unit_uniform(r.y) * static_cast<double>(__shfl(incl, 63, 64));
    const uint64_t live = __builtin_amdgcn_ballot_w64(mine > 0.f);            // != 0: the wavefront has weight
    const uint64_t hit = __builtin_amdgcn_ballot_w64(mine > 0.f && static_cast<double>(incl) > t2);
    const int lsel = hit != 0 ? __builtin_ctzll(hit) : 63 - __builtin_clzll(live);
    // ---- which of the lane's kVec * 8 columns: the lane hands its packed logits to the wavefront
    //      through LDS and lane j recomputes the weight of the lane's j-th column (slice j / 8,
    //      element j % 8), exactly as it was summed; one more scan instead of a serial walk --------
    static_assert(kVec * 8 <= kWave, "one lane per column of the chosen lane");
    __shared__ __attribute__((aligned(16))) uint32_t sh_cols[kVec * 4];
    if (lane == lsel) {
#pragma unroll
        for (int v = 0; v < kVec; ++v) *reinterpret_cast<u32x4_t *>(&sh_cols[4 * v]) = raw[v];
    }
    __builtin_amdgcn_wave_barrier();                       // (one wavefront: its LDS accesses complete in order)
    const int jj = lane < kVec * 8 ? lane : kVec * 8 - 1;
    const uint32_t pair = sh_cols[jj >> 1];
    const float xj = (jj & 1) ? bf16hi_to_f32(pair) : bf16lo_to_f32(pair);
    const float wj = lane < kVec * 8 ? __builtin_amdgcn_exp2f(xj * k - mm) : 0.f;
    float cincl = wj;
#pragma unroll
    for (int off = 1; off < kVec * 8; off <<= 1) {
        const float up = __shfl_up(cincl, off, 64);
        if (lane >= off) cincl += up;
    }
    const double t3 = unit_uniform(r.z) * static_cast<double>(__shfl(cincl, kVec * 8 - 1, 64));
    const uint64_t clive = __builtin_amdgcn_ballot_w64(wj > 0.f);             // != 0: the lane has weight
    const uint64_t chit = __builtin_amdgcn_ballot_w64(wj > 0.f && static_cast<double>(cincl) > t3);
    const int jsel = chit != 0 ? __builtin_ctzll(chit) : 63 - __builtin_clzll(clive);
    if (lane == 0)
        *rec = SampRecord{m, (wsum[0] + wsum[1]) + (wsum[2] + wsum[3]), 0.f,
                          chunk * (kSampSlice * kVec) + (jsel >> 3) * kSampSlice + (wave * kWave + lsel) * 8 + (jsel & 7)};
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
    const uint4 r = Philox::draw(make_uint4(static_cast<uint32_t>(b), 0x5a17u, static_cast<uint32_t>(offset),
                                            static_cast<uint32_t>(offset >> 32)),
                                 make_uint2(static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32)));
    if (nchunks <= kWave) {
        // the usual case (vocabularies up to 524,288): one record per lane, read once, everything else in registers
        SampRecord mine = SampRecord{-INFINITY, 0.f, 0.f, 0};
        if (lane < nchunks) {
            const f32x4_t v = *reinterpret_cast<const f32x4_t *>(rec + lane);
            mine = SampRecord{v[0], v[1], v[2], __float_as_int(v[3])};
        }
        const float m = wave_max(mine.m);
        if (m == -INFINITY) {                              // no finite logit in the row
            if (lane == 0) out_tokens[b] = 0;
            return;
        }
        const float w = mine.s * __builtin_amdgcn_exp2f(mine.m - m);      // 0 for lanes past the last chunk
        double incl = static_cast<double>(w);
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const double up = __shfl_up(incl, off, 64);
            if (lane >= off) incl += up;
        }
        const double target = unit_uniform(r.x) * __shfl(incl, 63, 64);
        const uint64_t live = __builtin_amdgcn_ballot_w64(w > 0.f);        // != 0: the row maximum's chunk has weight
        const uint64_t hit = __builtin_amdgcn_ballot_w64(w > 0.f && incl > target);
        const int pick = hit != 0 ? __builtin_ctzll(hit) : 63 - __builtin_clzll(live);
        const int col = __shfl(mine.col, pick, 64);
        if (lane == 0) out_tokens[b] = static_cast<int64_t>(col);
        return;
    }
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
    const int nchunks = samp_chunks(vocab, noise ? kNoiseVec : kDrawVec);
    if (noise)
        hipLaunchKernelGGL((sampler_chunk_kernel<kNoiseVec, true>), dim3(nchunks, batch), dim3(kSampThreads), 0, s, logits,
                           logits_row_stride, temperatures, noise, noise_row_stride, seed, offset, records, vocab, nchunks);
    else
        hipLaunchKernelGGL((sampler_chunk_kernel<kDrawVec, false>), dim3(nchunks, batch), dim3(kSampThreads), 0, s, logits,
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
    // one record per chunk of 2048 columns: at least what either chunking needs (4096 with a noise tensor, 8192 without)
    return static_cast<size_t>(batch) * nva::samp_chunks(vocab, 1) * sizeof(nva::SampRecord);
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
    // (the documented limit counts records of 2048 columns, the finest chunking any path has used; the present ones need fewer)
    if (static_cast<int64_t>(batch) * samp_chunks(vocab, 1) > kStaticRecords) return NVA_ERR_SCRATCH_TOO_SMALL;
    int status = NVA_OK;
    SampRecord *records = static_scratch(&status);
    if (records == nullptr) return status;
    // every record the row kernel reads is written by the chunk kernel of the same call: nothing to clear
    return launch_sample(static_cast<const bf16_t *>(logits), logits_row_stride, temperatures, noise, noise_row_stride,
                         seed, offset, out_tokens, records, batch, vocab, static_cast<hipStream_t>(stream));
}
