// Causal variable-length prefill attention for gfx950 (MFMA bf16, fp32 accumulate).
//
// Replaces flash_attn_varlen_func as called by nanovllm/layers/attention.py:64-70, including
// the prefix-cache case where K/V of every sequence are read through the block table.
//
// One workgroup of 4 wavefronts per (128-query tile, query head, sequence); wavefront w owns
// 32 query rows.  Keys are walked in tiles of 64.  The K and V tiles ([64][128] bf16 each) are
// double-buffered in LDS and travel global -> LDS directly (global_load_lds_dwordx4, 16 bytes per
// lane, no vector register in between): the loads of tile t+1 are issued before the arithmetic of
// tile t and waited for just before the one barrier per tile.  Rows keep their 256-byte pitch;
// the 16-byte chunk index is XOR-swizzled per key (K: by key%16, V: by 4*(key%4)) -- on the
// global side, since the LDS side of such a load is fixed -- so that the operand reads below are
// spread over all banks.
// Everything is computed transposed so that a query is a LANE (lane % 32) and keys / output
// dims live in that lane's registers:
//     S^T = K * Q^T      v_mfma_f32_32x32x16_bf16, A = K rows from LDS, B = Q^T (registers)
//     O^T = V^T * P^T    A = V^T through ds_read_b64_tr_b16 (LDS transpose read: 4 keys x 16
//                        dims -> lane = dim, registers = keys), B = P^T from the S^T registers
// The softmax state (running max, running sum) is therefore per lane, reductions over keys
// are in-register, and the only cross-lane step is one exchange between lanes l and l^32,
// which hold the two key halves of the same query.  The S^T accumulator layout (register i
// of lane l = key 8*(i/4) + 4*(l/32) + i%4) is also a legal k-ordering for the B operand of
// the second product as long as V^T uses the same key order, so P never leaves registers.
//
// The causal mask is aligned to the end of the keys: query i sees keys j <= i + (Lk - Lq).
// Work: 4 * 128 flop per (query, visible key, head).
#include "nva_common.h"

#include <math.h>

namespace nva {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));   // plain vectors: stay in registers
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef s16x4_t __attribute__((address_space(3))) * lds_s16x4_ptr;
typedef __attribute__((address_space(3))) void *lds_void_ptr;

constexpr int kPfThreads = 256;
constexpr int kPfBM = 128;            // queries per workgroup
constexpr int kPfBN = 64;             // keys per LDS tile
constexpr int kPfTileChunks = kPfBN * 16;   // 16-byte chunks per K (or V) tile
constexpr float kPfLazyLog2 = 8.f;    // how far (in powers of two) the running maximum may run ahead of the exponent base

struct PrefillArgs {
    const bf16_t *q; int64_t q_row_stride;
    const bf16_t *k; int64_t k_row_stride;
    const bf16_t *v; int64_t v_row_stride;
    const bf16_t *k_cache; const bf16_t *v_cache;
    const int32_t *block_tables; int32_t bt_row_stride;
    const int32_t *cu_seqlens_q; const int32_t *cu_seqlens_k;
    bf16_t *out;
    int32_t num_heads, num_kv_heads, num_blocks, num_q_tiles;
    float scale_log2e;
};

__device__ __forceinline__ bf16x8_t as_bf16x8(const u32x4_t &u) { return __builtin_bit_cast(bf16x8_t, u); }

// max of three in one instruction.  (fmaxf on accumulator registers costs three: the compiler
// first canonicalises both operands, because it cannot know that they hold no signalling NaN.)
__device__ __forceinline__ float max3(float x, float y, float z) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(y), "v"(z));
    return r;
}

// global -> LDS without a register in between: lane l's 16 bytes at base + voff land at LDS byte
// address lds_addr + 16 l.  Written as inline assembly on purpose: the compiler would make every
// LDS read that follows its own builtin wait for the load (it cannot tell the two LDS buffers
// apart), which would serialise the prefetch of the next tile with the arithmetic of this one.
// The caller waits with s_waitcnt vmcnt(0) before the barrier that publishes the tile.
// (s_nop 3: the load needs one wait state after the write of m0, and five after a vector
// instruction wrote one of its scalar operands -- v_readfirstlane does -- which the compiler
// cannot provide for an instruction it does not see.)
__device__ __forceinline__ void load_to_lds_16(const void *base, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(voff), "s"(base), "s"(lds_addr) : "memory", "m0");
}

// The same, for operands that a matrix instruction has just written.  A vector instruction may
// read the result registers of a v_mfma_f32_32x32x16_bf16 (8 passes) no sooner than 11 cycles
// after its issue, and the hardware does not check: the compiler pads its own instructions with
// s_nop, but it does not look inside inline assembly, so the padding is part of the statement.
__device__ __forceinline__ float max3_after_mfma(float x, float y, float z) {
    float r;
    asm volatile("s_nop 7\n\ts_nop 2\n\tv_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(y), "v"(z));
    return r;
}

template <bool kPaged>
__global__ __launch_bounds__(kPfThreads, 2) void prefill_attn_kernel(const PrefillArgs a) {
    // Workgroups go to the 8 XCDs round-robin by linear id and every XCD has an L2 of its own, so
    // the kv head is the fastest index: with 8 kv heads all workgroups that read the K/V of one
    // (sequence, kv head) -- every query tile of the query heads sharing it -- run on the same XCD
    // and find those rows in its L2.  Every XCD still gets the same mix of tiles however ragged
    // the sequences are.  Query tiles run from the last one (most keys, longest) to the first.
    const int group = a.num_heads / a.num_kv_heads;
    const int hkv = blockIdx.x % a.num_kv_heads;
    int rest = blockIdx.x / a.num_kv_heads;
    const int h = hkv * group + rest % group;
    rest /= group;
    const int mt = a.num_q_tiles - 1 - rest % a.num_q_tiles;
    const int b = rest / a.num_q_tiles;
    const int q0 = a.cu_seqlens_q[b], k0 = a.cu_seqlens_k[b];
    const int lq = a.cu_seqlens_q[b + 1] - q0;
    const int lk = a.cu_seqlens_k[b + 1] - k0;
    const int row0 = mt * kPfBM;
    if (row0 >= lq) return;                              // also covers empty query spans
    const int off = lk - lq;                             // bottom-right causal alignment

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int qi = lane & 31, hh = lane >> 5;
    const int qrow = row0 + wave * 32 + qi;              // query index inside the sequence
    const bool q_valid = qrow < lq;
    const int qrow_c = min(qrow, lq - 1);

    // Q^T fragments: B operand, column = this lane's query, k = dims 16*s + 8*hh + [0,8)
    bf16x8_t qfrag[8];
    {
        const bf16_t *qp = a.q + static_cast<int64_t>(q0 + qrow_c) * a.q_row_stride + h * kHeadDim + 8 * hh;
#pragma unroll
        for (int s = 0; s < 8; ++s) qfrag[s] = as_bf16x8(*reinterpret_cast<const u32x4_t *>(qp + 16 * s));
    }

    f32x16_t oacc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.f;
    float m_run = -INFINITY;      // shared by lanes l and l^32
    float l_run = 0.f;            // partial over this lane's key half

    __shared__ __attribute__((aligned(16))) u32x4_t sK[2][kPfTileChunks];
    __shared__ __attribute__((aligned(16))) u32x4_t sV[2][kPfTileChunks];

    const int q_hi = min(row0 + kPfBM, lq) - 1;          // last query row of the tile
    const int kv_end = min(lk, q_hi + off + 1);          // keys [0, kv_end) are visible to the tile
    const int ntiles = kv_end > 0 ? (kv_end + kPfBN - 1) / kPfBN : 0;
    const int wave_qmin = row0 + __builtin_amdgcn_readfirstlane(wave) * 32;   // (in a scalar register: branches on it stay scalar)

    // global -> registers for key tile kt: thread t moves chunks t, t+256, t+512, t+768 of the tile
    // (chunk c = key c/16, 16 bytes c%16); keys past the end are clamped and masked later
    // A tile of 64 keys starts at a multiple of 64 and so lies in one 256-token block: its block
    // id is the same for every lane, and it is fetched one tile ahead of the tile's own loads so
    // that no load of the loop waits for an address.
    // (The id is kept in a vector register until it is used: were the compiler to see that it is
    // uniform it would move it to a scalar register at once, and wait for every load issued before.)
    int lane_zero;
    asm volatile("v_mov_b32 %0, 0" : "=v"(lane_zero));
    auto fetch_block = [&](int kt) __attribute__((always_inline)) -> int32_t {
        // (the column is clamped to the row: cu_seqlens_k is device data the host could not check)
        return kPaged ? a.block_tables[static_cast<int64_t>(b) * a.bt_row_stride + min((kt * kPfBN) >> 8, a.bt_row_stride - 1) + lane_zero] : 0;
    };
    // K/V tiles go from global memory straight into LDS (global_load_lds_dwordx4: every lane
    // moves 16 bytes, the 64 lanes of one instruction fill 1 KB of LDS in lane order -- four key
    // rows -- and no vector register or LDS store instruction is spent on staging).  The LDS side
    // of such a load cannot be permuted, so the XOR swizzle is applied on the global side: the lane
    // that fills slot `lane % 16` of key row `key` fetches chunk slot ^ swizzle(key) of that row.
    // Instruction r of wavefront w covers keys 16r + 4w + [0, 4): this lane's key is tid/16 + 16r.
    // Addressing: a tile's first row has a wave-uniform address; this lane's chunk sits a fixed
    // 32-bit byte offset behind it, so a load needs no per-lane 64-bit arithmetic.  Only the last,
    // partial tile clamps its rows to the last key.
    const int lkey = tid >> 4;
    const int lch_k = (tid & 15) ^ (lkey & 15), lch_v = (tid & 15) ^ (4 * (lkey & 3));
    const int64_t kstride = kPaged ? static_cast<int64_t>(a.num_kv_heads) * kHeadDim : a.k_row_stride;
    const int64_t vstride = kPaged ? kstride : a.v_row_stride;
    const uint32_t koff0 = static_cast<uint32_t>((lkey * kstride + lch_k * 8) * 2);
    const uint32_t voff0 = static_cast<uint32_t>((lkey * vstride + lch_v * 8) * 2);
    const uint32_t kstep = static_cast<uint32_t>(16 * kstride * 2), vstep = static_cast<uint32_t>(16 * vstride * 2);
    // LDS byte addresses of this wavefront's first 1 KB span in buffer 0 of each tensor
    const uint32_t lds_k0 = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_ptr)&sK[0][wave * 64])));
    const uint32_t lds_v0 = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_ptr)&sV[0][wave * 64])));
    // Issues the loads of key tile kt into LDS buffer `buf`; returns false when the tile's block
    // table entry is out of range (the loads then read block 0 and the tile is masked out).
    auto load_tile = [&](int kt, int32_t blk_v, int buf) __attribute__((always_inline)) {
        const int32_t blk = kPaged ? __builtin_amdgcn_readfirstlane(blk_v) : 0;
        const bool ok = !kPaged || static_cast<uint32_t>(blk) < static_cast<uint32_t>(a.num_blocks);
        const int key0 = kt * kPfBN;
        const char *kb, *vb;
        if (kPaged) {
            const int64_t e = ((static_cast<int64_t>(ok ? blk : 0) * kBlockSize + (key0 & 255)) * a.num_kv_heads + hkv) *
                              kHeadDim * 2;
            kb = reinterpret_cast<const char *>(a.k_cache) + e;
            vb = reinterpret_cast<const char *>(a.v_cache) + e;
        } else {
            kb = reinterpret_cast<const char *>(a.k) + (static_cast<int64_t>(k0 + key0) * kstride + hkv * kHeadDim) * 2;
            vb = reinterpret_cast<const char *>(a.v) + (static_cast<int64_t>(k0 + key0) * vstride + hkv * kHeadDim) * 2;
        }
        const uint32_t dk = lds_k0 + buf * (kPfTileChunks * 16), dv = lds_v0 + buf * (kPfTileChunks * 16);
        if (key0 + kPfBN <= lk) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                load_to_lds_16(kb, r * kstep + koff0, dk + r * 4096);
                load_to_lds_16(vb, r * vstep + voff0, dv + r * 4096);
            }
        } else {
            const int last = lk - 1 - key0;              // >= 0: rows past it repeat it and are masked later
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = min(lkey + 16 * r, last);
                load_to_lds_16(kb, static_cast<uint32_t>((key * kstride + lch_k * 8) * 2), dk + r * 4096);
                load_to_lds_16(vb, static_cast<uint32_t>((key * vstride + lch_v * 8) * 2), dv + r * 4096);
            }
        }
        return ok;
    };

    bool tile_ok = true;                                 // of the tile computed next
    int32_t blk_next = 0;                                // block id of the tile loaded next
    if (ntiles > 0) tile_ok = load_tile(0, fetch_block(0), 0);
    if (ntiles > 1) blk_next = fetch_block(1);
    // Everything loaded so far (Q above all) is waited for here, and the Q fragments are then
    // passed through an empty asm.  Without this the compiler keeps treating them as in flight
    // inside the loop and makes each product wait for the loads issued just before it -- the
    // next tile's prefetch -- which put a full memory round trip into every tile.
    __builtin_amdgcn_s_waitcnt(0x0F70);                  // vmcnt(0): also the first tile has landed in LDS
#pragma unroll
    for (int s = 0; s < 8; ++s) asm volatile("" : "+v"(qfrag[s]));
    __syncthreads();

    for (int kt = 0; kt < ntiles; ++kt) {
        const int buf = kt & 1;
        const bool more = kt + 1 < ntiles;
        const bool cur_ok = tile_ok;
        if (more) {                                      // lands in the other buffer during this tile's arithmetic
            tile_ok = load_tile(kt + 1, blk_next, buf ^ 1);   // (that buffer was last read before the previous barrier)
            if (kt + 2 < ntiles) blk_next = fetch_block(kt + 2);
        }

        // A wavefront skips the arithmetic of a tile that lies wholly beyond the diagonal for all
        // of its 32 queries (the tile exists because later wavefronts of the workgroup see it).
        if (kt * kPfBN <= wave_qmin + 31 + off) {
        // ---- S^T = K Q^T for two 32-key sub-tiles ----------------------------------------
        f32x16_t sacc[2];
        // (the two wavefronts that share a SIMD belong to different workgroups; the one in a matrix
        // phase is given priority over the one in its softmax phase, so that the matrix pipe is fed
        // first: measured 3 % faster)
        __builtin_amdgcn_s_setprio(2);
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
#pragma unroll
            for (int i = 0; i < 16; ++i) sacc[t2][i] = 0.f;
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const int key = t2 * 32 + qi;
                const u32x4_t kf = sK[buf][key * 16 + ((2 * s + hh) ^ (key & 15))];
                sacc[t2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(kf), qfrag[s], sacc[t2], 0, 0, 0);
            }
        }

        __builtin_amdgcn_s_setprio(0);
        // ---- causal mask, running softmax (base 2; the scale is folded into the exponent) -------
        const int limit = cur_ok ? qrow + off : -1;      // last key this query may see
        if ((kt * kPfBN + kPfBN - 1) > (wave_qmin + off) || !cur_ok) {   // only tiles that cross the diagonal
            const int key_base = kt * kPfBN + 4 * hh;
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    if (key_base + t2 * 32 + 8 * (i >> 2) + (i & 3) > limit) sacc[t2][i] = -INFINITY;
        }
        // one dependent chain per sub-tile, so that every read of an accumulator follows the padded first one
        float mloc0 = max3_after_mfma(sacc[0][0], sacc[0][1], sacc[0][2]);
        float mloc1 = max3_after_mfma(sacc[1][0], sacc[1][1], sacc[1][2]);
#pragma unroll
        for (int i = 3; i < 15; i += 2) {
            mloc0 = max3(mloc0, sacc[0][i], sacc[0][i + 1]);
            mloc1 = max3(mloc1, sacc[1][i], sacc[1][i + 1]);
        }
        mloc1 = max3(mloc1, sacc[1][15], sacc[0][15]);   // (behind both padded reads)
        const float mloc = max3(mloc0, mloc1, mloc1);
        // m_run is the reference point of the exponentials, p = exp2(scale*log2e * (s - m_run)).  It
        // follows the true running maximum lazily: only when the maximum has moved more than
        // kPfLazyLog2 powers of two past it are the sums rescaled (p stays below 2^kPfLazyLog2, far
        // inside fp32 / bf16 range, and the final division by the row sum cancels the common
        // factor exactly).  With an eager update nearly every tile of a short sequence moves the
        // maximum of some query of the wavefront, and every move costs 64 multiplications per lane.
        const float m_true = max3(m_run, mloc, __shfl_xor(mloc, 32, 64));
        const bool lift = (m_true - m_run) * a.scale_log2e > kPfLazyLog2;   // -inf - -inf = NaN: false
        if (__builtin_amdgcn_ballot_w64(lift) != 0) {
            const float m_to = lift ? m_true : m_run;
            const float alpha = lift ? __builtin_amdgcn_exp2f((m_run - m_to) * a.scale_log2e) : 1.f;   // 0 on first use
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[dt][i] *= alpha;
            m_run = m_to;
        }
        const float m_safe = (m_run == -INFINITY) ? 0.f : m_run;    // no key seen yet: p = 0
        const float neg_ms = -m_safe * a.scale_log2e;
        float ps[4] = {0.f, 0.f, 0.f, 0.f};              // four short chains instead of one of 32 adds
        u32x4_t pfrag[2][2];                             // [sub-tile][k-step of 16 keys]
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            float p[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                p[i] = __builtin_amdgcn_exp2f(fmaf(sacc[t2][i], a.scale_log2e, neg_ms));   // exp2(-inf) = 0
                ps[i & 3] += p[i];
            }
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2)
                pfrag[t2][s2] = u32x4_t{pack_bf16x2(p[8 * s2 + 0], p[8 * s2 + 1]), pack_bf16x2(p[8 * s2 + 2], p[8 * s2 + 3]),
                                        pack_bf16x2(p[8 * s2 + 4], p[8 * s2 + 5]), pack_bf16x2(p[8 * s2 + 6], p[8 * s2 + 7])};
        }
        l_run += (ps[0] + ps[1]) + (ps[2] + ps[3]);

        // ---- O^T += V^T P^T ----------------------------------------------------------------
        // A operand: row = output dim (dt*32 + lane%32), k slot (hh, i) = key 16*s2 + 8*(i/4) + 4*hh + i%4.
        // Transpose read: the 16 lanes of a group fetch [4 keys][16 dims]; lane r16 supplies the address
        // of key r16/4, dims 4*(r16%4)..+3 and receives dim r16 of the four keys.
        {
            __builtin_amdgcn_s_setprio(2);
            const int r16 = lane & 15;
            const int dsub = (lane >> 4) & 1;            // which 16-dim half of the 32-dim tile
            const int kq = r16 >> 2;                     // key within the group of four
            const int cin = dsub * 2 + ((r16 >> 1) & 1); // 16-byte chunk within the tile's 64-byte dim span
            const char *vbase = reinterpret_cast<const char *>(&sV[buf][0]) + (r16 & 1) * 8;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
                    for (int s2 = 0; s2 < 2; ++s2) {
                        const int k_lo = t2 * 32 + 16 * s2 + 4 * hh + kq;     // k slots 0..3
                        const int k_hi = k_lo + 8;                            // k slots 4..7
                        const int c = dt * 4 + cin;
                        const s16x4_t vlo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (lds_s16x4_ptr)(vbase + k_lo * 256 + ((c ^ (4 * (k_lo & 3))) * 16)));
                        const s16x4_t vhi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (lds_s16x4_ptr)(vbase + k_hi * 256 + ((c ^ (4 * (k_hi & 3))) * 16)));
                        const s16x8_t both = __builtin_shufflevector(vlo, vhi, 0, 1, 2, 3, 4, 5, 6, 7);
                        oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, both),
                                                                           as_bf16x8(pfrag[t2][s2]), oacc[dt], 0, 0, 0);
                    }
            __builtin_amdgcn_s_setprio(0);
        }

        }
        __builtin_amdgcn_s_waitcnt(0x0F70);              // vmcnt(0): this wavefront's part of the next tile is in LDS
        __syncthreads();
    }

    // ---- normalise and store: register i of tile dt = dim dt*32 + 8*(i/4) + 4*hh + i%4 ----
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (q_valid) {
        bf16_t *op = a.out + (static_cast<int64_t>(q0 + qrow) * a.num_heads + h) * kHeadDim + 4 * hh;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                uint2 w;
                w.x = pack_bf16x2(oacc[dt][4 * g4 + 0] * inv, oacc[dt][4 * g4 + 1] * inv);
                w.y = pack_bf16x2(oacc[dt][4 * g4 + 2] * inv, oacc[dt][4 * g4 + 3] * inv);
                *reinterpret_cast<uint2 *>(op + dt * 32 + 8 * g4) = w;
            }
    }
}

}  // namespace nva

extern "C" int nva_varlen_prefill_attn(const void *q, int64_t q_row_stride, const void *k, int64_t k_row_stride,
                                       const void *v, int64_t v_row_stride, const void *k_cache,
                                       const void *v_cache, const int32_t *block_tables, int32_t bt_row_stride,
                                       int32_t max_blocks, const int32_t *cu_seqlens_q,
                                       const int32_t *cu_seqlens_k, int32_t batch, int32_t max_seqlen_q,
                                       int32_t max_seqlen_k, void *out, int32_t num_heads, int32_t num_kv_heads,
                                       int32_t head_dim, int32_t block_size, int32_t num_blocks, float scale,
                                       void *stream) {
    using namespace nva;
    if (batch < 0 || max_seqlen_q < 0 || max_seqlen_k < 0 || num_heads <= 0 || num_kv_heads <= 0)
        return NVA_ERR_BAD_SHAPE;
    if (head_dim != kHeadDim) return NVA_ERR_UNSUPPORTED_GEOMETRY;
    if (num_heads % num_kv_heads != 0) return NVA_ERR_UNSUPPORTED_GEOMETRY;
    if (batch == 0 || max_seqlen_q == 0) return NVA_OK;
    if (batch > 65535 || num_heads > 65535) return NVA_ERR_BAD_SHAPE;
    if (!q || !cu_seqlens_q || !cu_seqlens_k || !out) return NVA_ERR_NULL_POINTER;
    const bool paged = block_tables != nullptr;
    const int64_t dkv = static_cast<int64_t>(num_kv_heads) * head_dim;
    if (paged) {
        if (block_size != kBlockSize) return NVA_ERR_UNSUPPORTED_GEOMETRY;
        if (!k_cache || !v_cache) return NVA_ERR_NULL_POINTER;
        if (max_blocks <= 0 || num_blocks <= 0) return NVA_ERR_BAD_SHAPE;
        if (bt_row_stride < max_blocks) return NVA_ERR_BAD_STRIDE;
        if (static_cast<int64_t>(max_blocks) * kBlockSize < max_seqlen_k) return NVA_ERR_BAD_SHAPE;
        if (!aligned16(k_cache) || !aligned16(v_cache)) return NVA_ERR_MISALIGNED;
    } else {
        if (!k || !v) return NVA_ERR_NULL_POINTER;
        if (k_row_stride < dkv || v_row_stride < dkv || k_row_stride % 8 != 0 || v_row_stride % 8 != 0)
            return NVA_ERR_BAD_STRIDE;
        if (!aligned16(k) || !aligned16(v)) return NVA_ERR_MISALIGNED;
    }
    if (q_row_stride < static_cast<int64_t>(num_heads) * head_dim || q_row_stride % 8 != 0)
        return NVA_ERR_BAD_STRIDE;
    if (!aligned16(q) || !aligned16(out)) return NVA_ERR_MISALIGNED;

    PrefillArgs a;
    a.q = static_cast<const bf16_t *>(q); a.q_row_stride = q_row_stride;
    a.k = static_cast<const bf16_t *>(k); a.k_row_stride = k_row_stride;
    a.v = static_cast<const bf16_t *>(v); a.v_row_stride = v_row_stride;
    a.k_cache = static_cast<const bf16_t *>(k_cache); a.v_cache = static_cast<const bf16_t *>(v_cache);
    a.block_tables = block_tables; a.bt_row_stride = bt_row_stride;
    a.cu_seqlens_q = cu_seqlens_q; a.cu_seqlens_k = cu_seqlens_k;
    a.out = static_cast<bf16_t *>(out);
    a.num_heads = num_heads; a.num_kv_heads = num_kv_heads; a.num_blocks = num_blocks;
    a.scale_log2e = scale * 1.4426950408889634f;
    a.num_q_tiles = (max_seqlen_q + kPfBM - 1) / kPfBM;
    if (static_cast<int64_t>(a.num_q_tiles) * num_heads * batch > 0x7fffffffLL) return NVA_ERR_BAD_SHAPE;
    const dim3 grid(static_cast<uint32_t>(a.num_q_tiles) * num_heads * batch);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (paged)
        hipLaunchKernelGGL(prefill_attn_kernel<true>, grid, dim3(kPfThreads), 0, s, a);
    else
        hipLaunchKernelGGL(prefill_attn_kernel<false>, grid, dim3(kPfThreads), 0, s, a);
    return launch_status();
}
