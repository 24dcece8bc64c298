// Paged single-query (decode) attention for gfx950: persistent, evenly split stream of KV.
//
// Replaces flash_attn_with_kvcache as called by nanovllm/layers/attention.py:71-74.
//
// Work decomposition.  The unit of a wavefront's work is a "stage": 32 consecutive tokens of one kv
// head of one sequence (8 KB of K + 8 KB of V; a stage never straddles a KV block: blocks hold
// 256 * 2^k tokens).  The K rows of one kv head are 256-byte pieces 2 KB apart in the cache
// ([block, token, kv head, dim]); read head by head they stream 3-5 % slower than whole token rows.
// So the four wavefronts of a workgroup work on a "quad" of stages side by side: the same 32 tokens
// of four adjacent kv heads (HW = gcd(4, kv heads) heads x 4 / HW consecutive token ranges in
// general), which together are whole 1 KB runs of the token rows, fetched at the same time.  All
// quads of the batch form one list ordered by (sequence, group of HW kv heads, position) -- its
// length N follows from context_lens alone, which every workgroup prefix-sums in LDS.  The launch
// is a fixed set of 512 workgroups and workgroup x takes the contiguous slice [x*N/512, (x+1)*N/512)
// (one quad each when N < 512): every wavefront streams the same number of bytes whatever the mix
// of context lengths, nothing is launched for empty table entries, and the 8 XCDs (which receive
// workgroups round-robin) stay balanced.  The grid depends on no device data, so the launch can be
// captured in a HIP graph and replayed with new contents.  The split (prefix sums, clipped lengths,
// first quad and slice of every wavefront) is left in the workspace; a later launch over the same
// context_lens and block_tables -- the next layer of the same decode step -- may start from it
// (decode_stream_kernel<G, true>) and then issues its first loads after one 32-byte read instead of
// three dependent memory round trips.
//
// Per worker, a two-deep software pipeline over its stages:
//   * HBM -> VGPR: a K (or V) head row is 128 bf16 = 256 B = 16 lanes x 16 B, so one dwordx4
//     load instruction covers 4 full token rows; a stage is 8 K + 8 V loads per lane, and
//     the loads of stage x+1 are issued before the arithmetic of stage x, so every resident
//     wavefront keeps 16 KB in flight all the time (128 KB per CU at 8 wavefronts).
//   * VGPR -> LDS: rows go to a wavefront-private 16 KB region with an XOR swizzle of the
//     16-byte chunk index, so the matrix-core operand reads below are free of bank
//     conflicts although the row pitch is exactly 256 B.  No workgroup barrier is needed.
//   * S^T = K Q^T: v_mfma_f32_16x16x32_bf16, A = 16 token rows from LDS, B = Q^T in
//     registers; the G = num_heads/num_kv_heads query heads sharing the kv head are the
//     first G of the 16 columns (the rest are zero), so K is read once per kv head.
//   * softmax in base 2 on the accumulator layout (lane = head, registers = tokens): running
//     max / sum per lane, one exchange across the four 16-lane groups per stage.
//   * O^T += V^T P^T: A = V^T through ds_read_b64_tr_b16 (LDS transpose read: 4 tokens x 16
//     dims -> lane = dim, registers = tokens), B = P^T straight from the S^T registers.
// When a wavefront leaves a (sequence, kv head) pair it either writes the final bf16 rows (it
// saw all of the pair's stages) or an unnormalised partial (max, sum, o[128]) per query
// head.  A second, small kernel (decode_merge_kernel) merges the partials of the pairs that
// were split over several wavefronts; the kernel boundary is the only synchronisation.  (Workers
// sit on different XCDs, each with its own L2.  An in-kernel "last arriver merges" variant needs
// device-scope fences, which write back and invalidate the XCD's L2: measured 3x slower for
// the whole kernel.  Relaxed device-scope atomics without fences returned stale partials.)
//
// HBM traffic per sequence and layer: ctx * num_kv_heads * 128 * 2 B for K plus the same for
// V (4096 B per token at 8 kv heads).  Partials: at most (2048 + 4 * batch * num_kv_heads / HW) * G rows of
// 520 B; the stored split: 64 KB of wavefront records, 8 bytes per sequence and 8 bytes per (sequence, kv head) pair.
#include "nva_common.h"

#include <math.h>

namespace nva {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef s16x4_t __attribute__((address_space(3))) * lds_s16x4_ptr;
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));   // plain vectors: stay in registers
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kDecThreads = 256;
constexpr int kDecWaves = kDecThreads / kWave;
constexpr int kDecGrid = 512;                       // workgroups; 2 per CU on a 256-CU part
constexpr int kDecWorkers = kDecGrid * kDecWaves;   // wavefront workers
constexpr int kDecMaxBatch = 1024;                  // sequences per launch (prefix sums live in LDS)
constexpr int kStageTok = 32;                       // tokens per stage
constexpr int kStageLoads = kStageTok / 4;          // dwordx4 loads per lane per stage and tensor
constexpr int kWaveLdsChunks = 2 * kStageTok * 16;  // K then V, in 16-byte chunks

__device__ __forceinline__ bf16x8_t as_bf16x8(const u32x4_t &u) { return __builtin_bit_cast(bf16x8_t, u); }

// the workgroup that owns quad x when n quads are split over nw <= n workgroups as [w*n/nw, (w+1)*n/nw)
__device__ __forceinline__ int worker_of(int64_t x, int64_t n, int64_t nw) {
    return static_cast<int>(((x + 1) * nw - 1) / n);
}
// kv heads that the wavefronts of a workgroup take side by side: gcd(4, num_kv_heads)
__host__ __device__ inline int heads_abreast(int hkv) { return hkv % 4 == 0 ? 4 : (hkv % 2 == 0 ? 2 : 1); }

struct DecodeArgs {
    const bf16_t *q; int64_t q_row_stride;
    const bf16_t *k_cache; const bf16_t *v_cache;
    const int32_t *block_tables; int32_t bt_row_stride;
    const int32_t *context_lens;
    bf16_t *out;
    int32_t *pref_out;       // [batch + 1] quad-count prefix sums, written for the merge kernel
    int32_t *ctx_out;        // [batch] clipped context lengths         } the work split, kept for later
    int32_t *rec_out;        // [kDecWorkers][8] first quad per wavefront } launches over the same contexts
    int32_t *pair_out;       // [batch * num_kv_heads][2] first partial slot and workgroups of every pair
    float *part_ml;          // [rows][2]
    float *part_o;           // [rows][128]
    int32_t batch, max_blocks, num_heads, num_kv_heads, num_blocks;
    int32_t block_shift;     // log2 of the tokens per KV block (256, 512, ... : a power of two)
    int32_t hw, hw_shift;    // kv heads taken side by side by the wavefronts of a workgroup (1, 2 or 4) and its log2
    int32_t hgroups;         // num_kv_heads / hw
    float scale_log2e;
};

// kReuse: the workspace already holds the work split of an earlier launch (kReuse = false) over
// the same context_lens and block_tables; each wavefront then starts from its 32-byte record and
// issues its first loads before anything else, instead of prefix-summing the context lengths and
// reading the block table first.
//
// Quads.  HW = heads_abreast(num_kv_heads) kv heads side by side, PS = 4 / HW consecutive stages of
// each: wavefront j of a workgroup takes kv head hg * HW + j % HW and stage pq * PS + j / HW of quad
// (sequence b, head group hg, position pq).  A sequence of nst stages per head has
// ceil(nst / PS) * (num_kv_heads / HW) quads; a wavefront whose stage lies past the sequence end
// (PS > 1 only) runs the stage on zeros.
template <int G, bool kReuse>
__global__ __launch_bounds__(kDecThreads, 2) void decode_stream_kernel(const DecodeArgs a) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int grp = lane >> 4;     // 16-lane group: token row of a load, k-slot group of an MFMA
    const int r16 = lane & 15;     // chunk of a load; token / head / dim index of an MFMA operand
    const int hkv = a.num_kv_heads;
    const int hw = a.hw, ps = 4 >> a.hw_shift, hgroups = a.hgroups;
    const int jh = wave & (hw - 1), js = wave >> a.hw_shift;     // this wavefront's head inside the group, its stage inside the quad

    // ---- quad-count prefix sums over the batch (every workgroup computes its own copy) --------
    __shared__ int32_t sh_pref[kDecMaxBatch + 1];   // sh_pref[b] = quads of all sequences < b
    __shared__ int32_t sh_ctx[kDecMaxBatch];        // context length of sequence b, clipped to the table
    __shared__ __attribute__((aligned(16))) u32x4_t lds[kDecWaves * kWaveLdsChunks];
    const int w = blockIdx.x * kDecWaves + wave;
    u32x4_t *sK = lds + wave * kWaveLdsChunks;
    u32x4_t *sV = sK + kStageTok * 16;
    const int64_t row = static_cast<int64_t>(hkv) * kHeadDim;       // elements per token row

    // Block and number of valid rows (minus one) of stage ss of sequence bb; last = -1 when the stage
    // lies past the sequence end or behind a bad table entry (it then contributes nothing).
    auto locate = [&](int bb, int ss, int32_t &blk, int &last) __attribute__((always_inline)) {
        last = min(kStageTok, sh_ctx[bb] - ss * kStageTok) - 1;                // <= 31
        blk = 0;
        if (last >= 0) {
            blk = a.block_tables[static_cast<int64_t>(bb) * a.bt_row_stride + (ss >> (a.block_shift - 5))];
            if (static_cast<uint32_t>(blk) >= static_cast<uint32_t>(a.num_blocks)) {
                blk = 0;                                  // bad table entry
                last = -1;
            }
        } else {
            last = -1;
        }
    };
    // HBM -> registers for stage ss of kv head gg of sequence bb, which lies in block blk.  Token
    // rows are clamped to the last valid row of the stage, so only rows that were written are touched.
    // A stage without valid rows (last < 0) reads the sequence's own first query row instead of the
    // cache: every score of it is masked, so any finite data will do, and unwritten cache rows may
    // hold bit patterns that are not numbers (0 * NaN would reach the output).
    auto issue = [&](int bb, int gg, int ss, int32_t blk, int last, u32x4_t (&kr)[kStageLoads],
                     u32x4_t (&vr)[kStageLoads], u32x4_t (&qr)[4]) __attribute__((always_inline)) {
        const int tok0 = (ss << 5) & ((1 << a.block_shift) - 1);       // (kStageTok = 32 tokens per stage)
        const int64_t base = ((static_cast<int64_t>(blk) << a.block_shift) + tok0) * row + gg * kHeadDim + r16 * 8;
        const bf16_t *qrow = a.q + static_cast<int64_t>(bb) * a.q_row_stride + r16 * 8;
        const bf16_t *kb = last >= 0 ? a.k_cache + base : qrow;
        const bf16_t *vb = last >= 0 ? a.v_cache + base : qrow;
        const int lastc = max(last, 0);
        // K/V are read once and never again: non-temporal loads keep them from displacing one another in L2
        // (measured +12 % bandwidth over plain loads)
#pragma unroll
        for (int i = 0; i < kStageLoads; ++i) {
            const int t = min(i * 4 + grp, lastc);
            kr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(kb + t * row));
            vr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(vb + t * row));
        }
        // Q^T fragments (B operand): column = head r16 (zero beyond G), k-slots = dims 32i + 8grp + [0,8)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            u32x4_t u = {0u, 0u, 0u, 0u};
            if (r16 < G)
                u = *reinterpret_cast<const u32x4_t *>(a.q + static_cast<int64_t>(bb) * a.q_row_stride +
                                                       (gg * G + r16) * kHeadDim + 32 * i + 8 * grp);
            qr[i] = u;
        }
    };

    u32x4_t kr[kStageLoads], vr[kStageLoads], qr[4];
    int b, hg, pq, nqp, last;      // quad (b, hg, pq) of a sequence with nqp quads per head group
    int64_t lo, hi;                // this workgroup's slice of the quad list
    if constexpr (kReuse) {
        // ---- the split is in the workspace: first loads first, then the tables into LDS ---------
        const int4 *rec = reinterpret_cast<const int4 *>(a.rec_out) + 2 * w;
        const int4 r0 = rec[0], r1 = rec[1];
        constexpr int kPer = kDecMaxBatch / kDecThreads;
        int pv[kPer], cv[kPer];                          // table loads go out before the K/V loads
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int at = threadIdx.x + i * kDecThreads;
            pv[i] = at < a.batch ? a.pref_out[at] : 0;
            cv[i] = at < a.batch ? a.ctx_out[at] : 0;
        }
        const int total = a.pref_out[a.batch];
        b = r0.x; hg = r0.y; pq = r0.z; nqp = r0.w;
        last = r1.y; lo = r1.z; hi = r1.w;
        if (nqp > 0) issue(b, hg * hw + jh, pq * ps + js, r1.x, last, kr, vr, qr);
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int at = threadIdx.x + i * kDecThreads;
            if (at < a.batch) {
                sh_pref[at] = pv[i];
                sh_ctx[at] = cv[i];
            }
        }
        if (threadIdx.x == 0) sh_pref[a.batch] = total;
        __syncthreads();
    } else {
        if (wave == 0) {
            constexpr int kPer = kDecMaxBatch / kWave;  // 16 sequences per lane
            int cnt[kPer];
            int local = 0;
#pragma unroll
            for (int i = 0; i < kPer; ++i) {
                const int bi = lane * kPer + i;
                int c = 0;
                if (bi < a.batch) {
                    // a context that does not fit the table is clipped to it instead of read out of bounds
                    const int ctx = min(max(a.context_lens[bi], 0), a.max_blocks << a.block_shift);
                    sh_ctx[bi] = ctx;
                    c = (((ctx + kStageTok - 1) / kStageTok + ps - 1) >> (2 - a.hw_shift)) * hgroups;
                }
                cnt[i] = c;
                local += c;
            }
            int incl = local;                            // inclusive scan over the 64 lanes
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int up = __shfl_up(incl, off, 64);
                if (lane >= off) incl += up;
            }
            int run = incl - local;
            if (lane == 0) sh_pref[0] = 0;
#pragma unroll
            for (int i = 0; i < kPer; ++i) {
                run += cnt[i];
                sh_pref[lane * kPer + i + 1] = run;      // entries past the batch repeat the total
            }
        }
        __syncthreads();
        if (blockIdx.x == 0) {
            for (int i = threadIdx.x; i <= a.batch; i += kDecThreads) a.pref_out[i] = sh_pref[i];
            for (int i = threadIdx.x; i < a.batch; i += kDecThreads) a.ctx_out[i] = sh_ctx[i];
        }
    }

    // ---- sequences with no keys produce zero rows -----------------------------------------------
    for (int bz = blockIdx.x; bz < a.batch; bz += gridDim.x) {
        if (sh_pref[bz + 1] == sh_pref[bz]) {
            const int chunks = a.num_heads * kHeadDim / 8;
            u32x4_t *dst = reinterpret_cast<u32x4_t *>(a.out + static_cast<int64_t>(bz) * a.num_heads * kHeadDim);
            for (int c = threadIdx.x; c < chunks; c += kDecThreads) dst[c] = u32x4_t{0u, 0u, 0u, 0u};
        }
    }

    if constexpr (kReuse) {
        if (nqp == 0) return;                            // idle workgroup (uniform; no barrier follows)
    } else {
        // With fewer quads than workgroups only the first n_total workgroups get (one) quad each, so that
        // the workgroups of a pair are always consecutive.
        const int64_t n_total = sh_pref[a.batch];
        const int64_t n_wgs = n_total < kDecGrid ? n_total : kDecGrid;
        int4 *rec = reinterpret_cast<int4 *>(a.rec_out) + 2 * w;
        if (blockIdx.x >= n_wgs) {                       // uniform over the workgroup; no barrier follows
            if (lane == 0) rec[0] = int4{0, 0, 0, 0};
            return;
        }
        lo = static_cast<int64_t>(blockIdx.x) * n_total / n_wgs;
        hi = static_cast<int64_t>(blockIdx.x + 1) * n_total / n_wgs;   // > lo

        // ---- locate the first quad: largest b with sh_pref[b] <= lo -----------------------------
        {
            int l = 0, r = a.batch;                      // invariant: sh_pref[l] <= lo < sh_pref[r]
            while (r - l > 1) {
                const int mid = (l + r) >> 1;
                if (sh_pref[mid] <= lo) l = mid; else r = mid;
            }
            b = l;
        }
        nqp = (sh_pref[b + 1] - sh_pref[b]) / hgroups;   // quads per head group of sequence b (> 0)
        hg = static_cast<int>(lo - sh_pref[b]) / nqp;
        pq = static_cast<int>(lo - sh_pref[b]) % nqp;
        int32_t blk;
        locate(b, pq * ps + js, blk, last);
        issue(b, hg * hw + jh, pq * ps + js, blk, last, kr, vr, qr);
        if (lane == 0) {
            rec[0] = int4{b, hg, pq, nqp};
            rec[1] = int4{blk, last, static_cast<int>(lo), static_cast<int>(hi)};
        }
    }

    f32x4_t oacc[8];               // O^T: lane = head r16, tile dt register i = dim 16dt + 4grp + i
    float m_run, l_run;
    auto reset_state = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) oacc[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        m_run = -INFINITY;
        l_run = 0.f;
    };
    reset_state();

    for (int64_t x = lo; x < hi; ++x) {
        // ---- registers -> LDS (swizzled) ------------------------------------------------------
#pragma unroll
        for (int i = 0; i < kStageLoads; ++i) {
            const int t = i * 4 + grp;
            sK[t * 16 + (r16 ^ (t & 15))] = kr[i];
            sV[t * 16 + (r16 ^ (2 * (t & 7)))] = vr[i];
        }
        bf16x8_t qf[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) qf[i] = as_bf16x8(qr[i]);
        const int cur_last = last;
        const int cur_b = b, cur_hg = hg, cur_nqp = nqp;

        // ---- coordinates of the next quad; its loads fly during this stage's arithmetic -------
        const bool more = x + 1 < hi;
        bool pair_ends = true;
        if (more) {
            if (pq + 1 < nqp) {
                ++pq;
                pair_ends = false;
            } else {
                pq = 0;
                if (hg + 1 < hgroups) {
                    ++hg;
                } else {
                    hg = 0;
                    do { ++b; } while (sh_pref[b + 1] == sh_pref[b]);   // skip sequences without keys
                    nqp = (sh_pref[b + 1] - sh_pref[b]) / hgroups;
                }
            }
            int32_t blk;
            locate(b, pq * ps + js, blk, last);
            issue(b, hg * hw + jh, pq * ps + js, blk, last, kr, vr, qr);
        }
        __builtin_amdgcn_wave_barrier();

        // ---- S^T = K Q^T: two tiles of 16 tokens ------------------------------------------------
        f32x4_t sc[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
            sc[tt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const u32x4_t ka = sK[(16 * tt + r16) * 16 + ((4 * i + grp) ^ r16)];
                sc[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(ka), qf[i], sc[tt], 0, 0, 0);
            }
        }
        // register i of tile tt = token 16tt + 4grp + i of the stage
        float mloc = -INFINITY;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float v = (16 * tt + 4 * grp + i <= cur_last) ? sc[tt][i] * a.scale_log2e : -INFINITY;
                sc[tt][i] = v;
                mloc = fmaxf(mloc, v);
            }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
        const float m_new = fmaxf(m_run, mloc);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;     // nothing visible yet: p = 0, alpha = 0
        const float alpha = exp2f(m_run - m_use);
        m_run = m_new;
        float p[8];
        float psum = 0.f;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                p[4 * tt + i] = exp2f(sc[tt][i] - m_use);
                psum += p[4 * tt + i];
            }
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) oacc[dt] *= alpha;
        // P^T as B operand: k-slot i = token 4grp + i, k-slot 4+i = token 16 + 4grp + i
        const u32x4_t pu = {pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]),
                            pack_bf16x2(p[4], p[5]), pack_bf16x2(p[6], p[7])};
        const bf16x8_t pf = as_bf16x8(pu);

        // ---- O^T += V^T P^T -----------------------------------------------------------------------
        // transpose read: the 16 lanes of a group fetch [4 tokens][16 dims]; lane r16 supplies the
        // address of token r16/4, dims 4*(r16%4)..+3 and receives dim r16 of the four tokens
        {
            const int t_lo = 4 * grp + (r16 >> 2);
            const int t_hi = t_lo + 16;
            const int sub = (r16 >> 1) & 1;            // which 16-byte chunk of the 32-byte dim span
            const char *vbase = reinterpret_cast<const char *>(sV) + (r16 & 1) * 8;
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) {
                const int c = 2 * dt + sub;
                const s16x4_t vlo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4_ptr)(vbase + t_lo * 256 + ((c ^ (2 * (t_lo & 7))) * 16)));
                const s16x4_t vhi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (lds_s16x4_ptr)(vbase + t_hi * 256 + ((c ^ (2 * (t_hi & 7))) * 16)));
                const s16x8_t both = __builtin_shufflevector(vlo, vhi, 0, 1, 2, 3, 4, 5, 6, 7);
                oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, both), pf,
                                                                   oacc[dt], 0, 0, 0);
            }
        }
        __builtin_amdgcn_wave_barrier();               // this stage's LDS reads precede the next stage's writes

        // ---- leaving the (sequence, head group): final rows, or a partial for the merge -----------
        if (pair_ends) {
            float l_tot = l_run + __shfl_xor(l_run, 16, 64);
            l_tot += __shfl_xor(l_tot, 32, 64);
            const int cur_g = cur_hg * hw + jh;
            const int64_t pair_lo = sh_pref[cur_b] + static_cast<int64_t>(cur_hg) * cur_nqp;   // first quad of the head group
            const int64_t pair_hi = pair_lo + cur_nqp;
            if (ps == 1 && lo <= pair_lo && pair_hi <= hi) {      // this wavefront saw the whole pair
                if (r16 < G) {
                    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
                    bf16_t *op = a.out + (static_cast<int64_t>(cur_b) * a.num_heads + cur_g * G + r16) * kHeadDim + 4 * grp;
#pragma unroll
                    for (int dt = 0; dt < 8; ++dt) {
                        const u32x2_t o2 = {pack_bf16x2(oacc[dt][0] * inv, oacc[dt][1] * inv),
                                            pack_bf16x2(oacc[dt][2] * inv, oacc[dt][3] * inv)};
                        *reinterpret_cast<u32x2_t *>(op + 16 * dt) = o2;
                    }
                }
            } else {
                // (workgroup + head group) is unique per (workgroup, head group) along the quad list; its four wavefronts' rows are neighbours
                const int64_t slot = (blockIdx.x + (static_cast<int64_t>(cur_b) * hgroups + cur_hg)) * kDecWaves + wave;
                if (r16 < G) {
                    float *po = a.part_o + (slot * G + r16) * kHeadDim + 4 * grp;
#pragma unroll
                    for (int dt = 0; dt < 8; ++dt) *reinterpret_cast<f32x4_t *>(po + 16 * dt) = oacc[dt];
                    if (grp == 0) {
                        a.part_ml[(slot * G + r16) * 2 + 0] = m_run;
                        a.part_ml[(slot * G + r16) * 2 + 1] = l_tot;
                    }
                }
            }
            reset_state();
        }
    }
}

// Merges the partials of every (sequence, kv head) pair that was split over several wavefronts.
// One workgroup of G wavefronts per pair: wavefront h merges query head g*G + h, lane = 2 dims.
// Which workgroups met the pair's head group follows from the quad-count prefix sums the streaming
// kernel left in the workspace; a pair seen by a single wavefront was already written.  The partials
// of the pair are the rows ((slot0 + i) * 4 + j) * G + h for the 4 / HW wavefront indices j that
// carry its kv head and i = 0 .. workgroups - 1.  The building call also leaves (slot0, workgroups)
// per pair in the workspace, so that a call that reuses the work split starts from one 8-byte read
// instead of three dependent ones.  The partials are fetched eight at a time, all loads of a round
// in flight together.
template <int G, bool kReuse>
__global__ __launch_bounds__(G * kWave) void decode_merge_kernel(const DecodeArgs a) {
    const int pair = blockIdx.x;
    const int b = pair / a.num_kv_heads;
    const int g = pair % a.num_kv_heads;
    const int h = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int hw = a.hw, ps = 4 >> a.hw_shift, hgroups = a.hgroups;
    int64_t slot0;
    int n_wgs;
    if constexpr (kReuse) {
        const int2 info = reinterpret_cast<const int2 *>(a.pair_out)[pair];
        slot0 = info.x;
        n_wgs = info.y;
    } else {
        const int64_t n_total = a.pref_out[a.batch];
        const int pb = a.pref_out[b];
        const int nqp = (a.pref_out[b + 1] - pb) / hgroups;
        n_wgs = 0;                                     // no keys: the zero rows are already there
        slot0 = 0;
        if (nqp > 0) {
            const int64_t grid = n_total < kDecGrid ? n_total : kDecGrid;
            const int hg = g >> a.hw_shift;
            const int64_t pair_lo = pb + static_cast<int64_t>(hg) * nqp;
            const int x_first = worker_of(pair_lo, n_total, grid);
            n_wgs = worker_of(pair_lo + nqp - 1, n_total, grid) - x_first + 1;
            slot0 = static_cast<int64_t>(x_first) + static_cast<int64_t>(b) * hgroups + hg;   // slots of consecutive workgroups are consecutive
        }
        if (threadIdx.x == 0) reinterpret_cast<int2 *>(a.pair_out)[pair] = int2{static_cast<int>(slot0), n_wgs};
    }
    const int n_parts = n_wgs * ps;
    if (n_parts <= 1) return;                          // one wavefront saw the whole pair and wrote it
    const int jh = g & (hw - 1);
    // partial t of the pair: wavefront index jh + hw * (t / n_wgs), workgroup t % n_wgs of the pair's run
    const int64_t row_first = (slot0 * kDecWaves + jh) * G + h;               // partial 0; consecutive workgroups are 4 G rows apart
    auto part_row = [&](int t) __attribute__((always_inline)) -> int64_t {
        if (ps == 1) return row_first + static_cast<int64_t>(t) * (kDecWaves * G);   // (the usual case: kv heads a multiple of 4)
        const int js = (t >= n_wgs) + (t >= 2 * n_wgs) + (t >= 3 * n_wgs);     // t / n_wgs, which is below 4
        return row_first + (static_cast<int64_t>(t - js * n_wgs) * kDecWaves + hw * js) * G;
    };
    float mx = -INFINITY, lsum = 0.f, acc0 = 0.f, acc1 = 0.f;
    for (int base = 0; base < n_parts; base += 8) {
        float pm[8], pl[8];
        float2 po[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int64_t at = part_row(min(base + j, n_parts - 1));
            const float2 ml = *reinterpret_cast<const float2 *>(a.part_ml + at * 2);
            po[j] = *reinterpret_cast<const float2 *>(a.part_o + at * kHeadDim + 2 * lane);
            pm[j] = base + j < n_parts ? ml.x : -INFINITY;
            pl[j] = ml.y;
        }
        float m_new = mx;
#pragma unroll
        for (int j = 0; j < 8; ++j) m_new = fmaxf(m_new, pm[j]);
        if (m_new > -INFINITY) {
            const float keep = exp2f(mx - m_new);      // 0 in the first round
            lsum *= keep;
            acc0 *= keep;
            acc1 *= keep;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float f = exp2f(pm[j] - m_new);  // 0 for slots past the last partial and for partials without keys
                lsum = fmaf(f, pl[j], lsum);
                acc0 = fmaf(f, po[j].x, acc0);
                acc1 = fmaf(f, po[j].y, acc1);
            }
            mx = m_new;
        }
    }
    const float inv = lsum > 0.f ? 1.f / lsum : 0.f;
    *reinterpret_cast<uint32_t *>(a.out + (static_cast<int64_t>(b) * a.num_heads + g * G + h) * kHeadDim + 2 * lane) =
        pack_bf16x2(acc0 * inv, acc1 * inv);
}

template <int G>
static int launch_decode(const DecodeArgs &a, bool reuse, hipStream_t stream) {
    if (reuse)
        hipLaunchKernelGGL((decode_stream_kernel<G, true>), dim3(kDecGrid), dim3(kDecThreads), 0, stream, a);
    else
        hipLaunchKernelGGL((decode_stream_kernel<G, false>), dim3(kDecGrid), dim3(kDecThreads), 0, stream, a);
    if (launch_status() != NVA_OK) return NVA_ERR_LAUNCH_FAILED;
    if (reuse)
        hipLaunchKernelGGL((decode_merge_kernel<G, true>), dim3(a.batch * a.num_kv_heads), dim3(G * kWave), 0, stream, a);
    else
        hipLaunchKernelGGL((decode_merge_kernel<G, false>), dim3(a.batch * a.num_kv_heads), dim3(G * kWave), 0, stream, a);
    return launch_status();
}

static inline size_t align_up(size_t v, size_t to) { return (v + to - 1) / to * to; }

struct DecodeWorkspace {
    size_t pref_bytes, ctx_bytes, rec_bytes, pair_bytes, rows, total;
};
static DecodeWorkspace decode_workspace(int32_t batch, int32_t num_heads, int32_t num_kv_heads, int32_t head_dim) {
    DecodeWorkspace ws;
    const size_t per_launch = static_cast<size_t>(batch < kDecMaxBatch ? batch : kDecMaxBatch);
    ws.pref_bytes = align_up((per_launch + 1) * sizeof(int32_t), 256);
    // partial rows: one per query head of every (wavefront, head group) met along the quad list;
    // row index = ((workgroup + sequence * head groups + head group) * 4 + j) * G + head
    // with j < 4, i.e. below 2048 * G + 4 * batch * num_heads / HW; G <= 8 and HW >= 1 (the size does not depend on
    // the number of kv heads: the caller sizes the workspace without it)
    ws.rows = static_cast<size_t>(kDecWorkers) * (num_heads < 8 ? num_heads : 8) + 4 * per_launch * num_heads;
    ws.ctx_bytes = align_up(per_launch * sizeof(int32_t), 256);
    ws.rec_bytes = static_cast<size_t>(kDecWorkers) * 8 * sizeof(int32_t);
    ws.pair_bytes = align_up(per_launch * static_cast<size_t>(num_kv_heads) * 2 * sizeof(int32_t), 256);
    ws.total = ws.pref_bytes + ws.ctx_bytes + ws.rec_bytes + ws.pair_bytes +
               ws.rows * (static_cast<size_t>(head_dim) + 2) * sizeof(float);
    return ws;
}

}  // namespace nva

extern "C" size_t nva_paged_decode_workspace_bytes(int32_t batch, int32_t num_heads, int32_t head_dim,
                                                   int32_t max_blocks) {
    (void)max_blocks;
    if (batch <= 0 || num_heads <= 0 || head_dim <= 0) return 0;
    // (the number of kv heads is not an argument: sized for the most there can be, one per query head)
    return nva::decode_workspace(batch, num_heads, num_heads, head_dim).total;
}

extern "C" int nva_paged_decode_attn(const void *q, int64_t q_row_stride, const void *k_cache,
                                     const void *v_cache, const int32_t *block_tables,
                                     int32_t bt_row_stride, int32_t max_blocks,
                                     const int32_t *context_lens, void *out, void *workspace,
                                     size_t workspace_bytes, int32_t batch, int32_t num_heads,
                                     int32_t num_kv_heads, int32_t head_dim, int32_t block_size,
                                     int32_t num_blocks, float scale, void *stream) {
    return nva_paged_decode_attn_planned(q, q_row_stride, k_cache, v_cache, block_tables, bt_row_stride,
                                         max_blocks, context_lens, out, workspace, workspace_bytes, batch,
                                         num_heads, num_kv_heads, head_dim, block_size, num_blocks, scale,
                                         NVA_PLAN_BUILD, stream);
}

extern "C" int nva_paged_decode_attn_planned(const void *q, int64_t q_row_stride, const void *k_cache,
                                             const void *v_cache, const int32_t *block_tables,
                                             int32_t bt_row_stride, int32_t max_blocks,
                                             const int32_t *context_lens, void *out, void *workspace,
                                             size_t workspace_bytes, int32_t batch, int32_t num_heads,
                                             int32_t num_kv_heads, int32_t head_dim, int32_t block_size,
                                             int32_t num_blocks, float scale, int32_t plan, void *stream) {
    using namespace nva;
    if (plan != NVA_PLAN_BUILD && plan != NVA_PLAN_REUSE) return NVA_ERR_BAD_SHAPE;
    if (batch < 0 || num_heads <= 0 || num_kv_heads <= 0 || max_blocks < 0 || num_blocks < 0)
        return NVA_ERR_BAD_SHAPE;
    const int block_shift = block_shift_of(block_size);
    if (head_dim != kHeadDim || block_shift < 0) return NVA_ERR_UNSUPPORTED_GEOMETRY;
    if (num_heads % num_kv_heads != 0) return NVA_ERR_UNSUPPORTED_GEOMETRY;
    const int group = num_heads / num_kv_heads;
    if (group > 8) return NVA_ERR_UNSUPPORTED_GEOMETRY;                       // (every group from 1 to 8 is built)
    if (batch == 0) return NVA_OK;
    if (static_cast<int64_t>(max_blocks) * (block_size / kStageTok) * num_kv_heads * kDecMaxBatch > 0x7fffffffLL)
        return NVA_ERR_BAD_SHAPE;                                             // stage counts are int32
    if (!q || !k_cache || !v_cache || !context_lens || !out || !workspace) return NVA_ERR_NULL_POINTER;
    if (max_blocks > 0 && !block_tables) return NVA_ERR_NULL_POINTER;
    if (q_row_stride < static_cast<int64_t>(num_heads) * head_dim || q_row_stride % 8 != 0)
        return NVA_ERR_BAD_STRIDE;
    if (bt_row_stride < max_blocks) return NVA_ERR_BAD_STRIDE;
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(workspace) || !aligned16(out))
        return NVA_ERR_MISALIGNED;
    if (workspace_bytes < nva_paged_decode_workspace_bytes(batch, num_heads, head_dim, max_blocks)) return NVA_ERR_WORKSPACE_TOO_SMALL;
    const DecodeWorkspace ws = decode_workspace(batch, num_heads, num_kv_heads, head_dim);

    hipStream_t s = static_cast<hipStream_t>(stream);
    DecodeArgs a;
    a.k_cache = static_cast<const bf16_t *>(k_cache);
    a.v_cache = static_cast<const bf16_t *>(v_cache);
    a.bt_row_stride = bt_row_stride;
    a.q_row_stride = q_row_stride;
    a.pref_out = static_cast<int32_t *>(workspace);
    a.ctx_out = reinterpret_cast<int32_t *>(static_cast<char *>(workspace) + ws.pref_bytes);
    a.rec_out = reinterpret_cast<int32_t *>(static_cast<char *>(workspace) + ws.pref_bytes + ws.ctx_bytes);
    a.pair_out = reinterpret_cast<int32_t *>(static_cast<char *>(workspace) + ws.pref_bytes + ws.ctx_bytes + ws.rec_bytes);
    a.part_ml = reinterpret_cast<float *>(static_cast<char *>(workspace) + ws.pref_bytes + ws.ctx_bytes + ws.rec_bytes + ws.pair_bytes);
    // every launch of a split batch overwrites the stored work split, so only a single launch can reuse it
    const bool reuse = plan == NVA_PLAN_REUSE && batch <= kDecMaxBatch;
    a.part_o = a.part_ml + ws.rows * 2;
    a.max_blocks = max_blocks;
    a.num_heads = num_heads;
    a.num_kv_heads = num_kv_heads;
    a.num_blocks = num_blocks;
    a.block_shift = block_shift;
    a.hw = heads_abreast(num_kv_heads);
    a.hw_shift = a.hw == 4 ? 2 : (a.hw == 2 ? 1 : 0);
    a.hgroups = num_kv_heads / a.hw;
    a.scale_log2e = scale * 1.4426950408889634f;
    // launches of at most kDecMaxBatch sequences each, back to back on the stream
    for (int32_t b0 = 0; b0 < batch; b0 += kDecMaxBatch) {
        a.batch = batch - b0 < kDecMaxBatch ? batch - b0 : kDecMaxBatch;
        a.q = static_cast<const bf16_t *>(q) + static_cast<int64_t>(b0) * q_row_stride;
        a.block_tables = block_tables + static_cast<int64_t>(b0) * bt_row_stride;
        a.context_lens = context_lens + b0;
        a.out = static_cast<bf16_t *>(out) + static_cast<int64_t>(b0) * num_heads * head_dim;
        int rc;
        switch (group) {
            case 1: rc = launch_decode<1>(a, reuse, s); break;
            case 2: rc = launch_decode<2>(a, reuse, s); break;
            case 3: rc = launch_decode<3>(a, reuse, s); break;
            case 4: rc = launch_decode<4>(a, reuse, s); break;
            case 5: rc = launch_decode<5>(a, reuse, s); break;
            case 6: rc = launch_decode<6>(a, reuse, s); break;
            case 7: rc = launch_decode<7>(a, reuse, s); break;
            default: rc = launch_decode<8>(a, reuse, s); break;
        }
        if (rc != NVA_OK) return rc;
    }
    return NVA_OK;
}
