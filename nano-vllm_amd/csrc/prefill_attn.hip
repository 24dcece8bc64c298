// Causal variable-length prefill attention for gfx950 (MFMA bf16, fp32 accumulate).
//
// Replaces flash_attn_varlen_func as called by nanovllm/layers/attention.py:64-70, including
// the prefix-cache case where K/V of every sequence are read through the block table.
//
// One workgroup of 4 wavefronts per (128-query tile, query head, sequence); wavefront w owns
// 32 query rows, as two groups of 16.  Keys are walked in tiles of 64.  Everything is computed
// transposed with v_mfma_f32_16x16x32_bf16 (on this part it sustains 98 % of the matrix peak,
// the 32x32x16 form 71-87 %), so that a query is a lane column (lane % 16) and keys / output
// dims live in registers and across the four 16-lane groups:
//     S^T = K * Q^T      A = 16 keys x 32 dims from LDS (one ds_read_b128), B = Q^T (registers)
//     O^T = V^T * P^T    A = 16 dims x 32 keys through two ds_read_b64_tr_b16 (LDS transpose
//                        read), B = P^T straight from the S^T accumulators
// The S^T accumulator layout (register i of lane l = key 4*(l/16) + i of a 16-key block) taken
// over two key blocks is a legal k-ordering for the B operand of the second product as long as
// V^T is fetched in the same key order, so P never leaves registers.
//
// LDS.  The K and V tiles are double-buffered and travel global -> LDS directly
// (global_load_lds_dwordx4, 16 bytes per lane, no vector register in between).  Such a load
// writes its 64 lanes' 16-byte pieces to consecutive LDS addresses, but which piece of global
// memory a lane fetches is free, so the LDS image is laid out fragment by fragment: one load
// instruction fetches 64 bytes (32 dims) of 16 key rows and fills the 1 KB block that one
// matrix operand is read from.  Within a block the four 16-byte pieces of a key are permuted
// so that every operand read is spread over all banks, and every read address is one lane
// constant plus an immediate offset: no address arithmetic in the loop.
//
// Softmax.  p = exp2(scale*log2e * s - ref) with ONE exponent reference per query for the whole
// pass: the largest score among the first 32 keys of the row.  Any reference cancels in the final
// division by the row sum; it only has to keep every p inside fp32 range (which bf16 shares).  The
// common path therefore computes no maximum, rescales nothing and exchanges nothing between lanes.
// If a row sum of the workgroup ends beyond 2^100 or is not a number, some score exceeded the
// first keys' maximum by hundreds: the workgroup then computes the exact row maxima in a pass of
// their own (scores only) and repeats its query tile with them.  Row sums are accumulated on the
// matrix pipe (P^T times a block of ones), over the bf16 values of P that the second product uses.
// Per score that leaves one fma, one exp2 and half a bf16 pack on the vector pipe.
//
// Schedule.  A tile is processed in two halves of 32 keys, written out in execution order and
// fenced step by step: the scores of the second half are multiplied while the first half goes
// through the softmax, and the first half's P*V runs while the second half goes through the
// softmax; the eight loads of the next tile are spread over the products.  One barrier per tile.
//
// The causal mask is aligned to the end of the keys: query i sees keys j <= i + (Lk - Lq).
// Work: 4 * 128 flop per (query, visible key, head).
#include "nva_common.h"

#include <math.h>

#include <type_traits>

namespace nva {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));   // plain vectors: stay in registers
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) char *lds_char_ptr;
typedef __attribute__((address_space(3))) u32x4_t *lds_u32x4_ptr;
typedef __attribute__((address_space(3))) s16x4_t *lds_s16x4_ptr;

constexpr int kPfThreads = 256;
constexpr int kPfBM = 128;            // queries per workgroup
constexpr int kPfBN = 64;             // keys per LDS tile
constexpr int kPfTileBytes = kPfBN * kHeadDim * 2;      // one K (or V) tile: 16 KB = 16 blocks of 1 KB
constexpr float kPfLiftLimit = 1.2676506e30f;           // 2^100: a row sum beyond it makes the workgroup repeat its work with exact maxima

struct PrefillArgs {
    const bf16_t *q; int64_t q_row_stride;
    const bf16_t *k; int64_t k_row_stride;
    const bf16_t *v; int64_t v_row_stride;
    const bf16_t *k_cache; const bf16_t *v_cache;
    const int32_t *block_tables; int32_t bt_row_stride;
    const int32_t *cu_seqlens_q; const int32_t *cu_seqlens_k;
    bf16_t *out;
    int32_t num_heads, num_kv_heads, num_blocks, num_q_tiles;
    int32_t block_shift;     // log2 of the tokens per KV block
    float scale_log2e;
};

__device__ __forceinline__ bf16x8_t as_bf16x8(const u32x4_t &u) { return __builtin_bit_cast(bf16x8_t, u); }

// global -> LDS without a register in between: lane l's 16 bytes at base + voff land at LDS byte
// address lds_addr + 16 l.  Written as inline assembly on purpose: the compiler would make every
// LDS read that follows its own builtin wait for the load (it cannot tell the two LDS buffers
// apart), which would serialise the prefetch of the next tile with the arithmetic of this one.
// The caller waits with s_waitcnt vmcnt(0) before the barrier that publishes the tile.
// (s_nop 0: the load needs one wait state after the write of m0, which the compiler cannot provide
// for an instruction it does not see.  Its scalar operands are always results of scalar
// arithmetic; one written by a vector instruction -- v_readfirstlane -- would need five.)
__device__ __forceinline__ void load_to_lds_16(const void *base, uint32_t &voff, uint32_t lds_addr) {
    // Not volatile, and the offset register is declared as written although it keeps its value: the
    // statement is then an ordinary instruction that the scheduler may place anywhere between the
    // computation of its operands and the next use of the offset (a volatile statement is a fence
    // for every LDS read and cuts the block into separately scheduled pieces).  The loads of one
    // tensor form a chain through the offset; loads_issued() ends the chains before the wait.
    asm("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
        : "+v"(voff) : "s"(base), "s"(lds_addr) : "m0");
}
__device__ __forceinline__ void loads_issued(uint32_t koff, uint32_t voff) { asm volatile("" :: "v"(koff), "v"(voff)); }

template <bool kPaged>
__global__ __launch_bounds__(kPfThreads, 2) void prefill_attn_kernel(const PrefillArgs a) {
    // Workgroups go to the 8 XCDs round-robin by linear id and every XCD has an L2 of its own, so
    // the kv head is the fastest index: with 8 kv heads all workgroups that read the K/V of one
    // (sequence, kv head) -- every query tile of the query heads sharing it -- run on the same XCD
    // and find those rows in its L2.  Every XCD still gets the same mix of tiles however ragged
    // the sequences are.  Query tiles run from the last one (most keys, longest) to the first, sequence
    // by sequence: the tiles of one sequence run close together in time and share its K/V in L2
    // (handing out the last tiles of ALL sequences first, then the ones before them, takes as long
    // and fetches twice as much from memory: 7 MB of K/V per kv head do not stay in a 4 MB L2).
    const int group = a.num_heads / a.num_kv_heads;
    const int hkv = blockIdx.x % a.num_kv_heads;
    int rest = blockIdx.x / a.num_kv_heads;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // (in a scalar register: branches on it stay scalar)
    const int h = hkv * group + rest % group;
    rest /= group;
    const int mt = a.num_q_tiles - 1 - rest % a.num_q_tiles;
    const int b = rest / a.num_q_tiles;
    // A tile of 64 keys starts at a multiple of 64 and so lies in one KV block (256 * 2^k tokens): its block
    // id is the same for every lane, and it is fetched one tile ahead of the tile's own loads so
    // that no load of the loop waits for an address.
    // (The id is kept in a vector register until it is used: were the compiler to see that it is
    // uniform it would move it to a scalar register at once, and wait for every load issued before.)
    int lane_zero;
    asm volatile("v_mov_b32 %0, 0" : "=v"(lane_zero));
    auto fetch_block = [&](int kt) __attribute__((always_inline)) -> int32_t {
        // (the column is clamped to the row: cu_seqlens_k is device data the host could not check)
        return kPaged ? a.block_tables[static_cast<int64_t>(b) * a.bt_row_stride + min((kt * kPfBN) >> a.block_shift, a.bt_row_stride - 1) + lane_zero] : 0;
    };
    // (the ids of the first tiles depend on the sequence only: asked for together with its bounds, one trip
    // to memory instead of two in a row)
    const int32_t blk_first = fetch_block(0), blk_second = fetch_block(1);

    const int q0 = a.cu_seqlens_q[b], k0 = a.cu_seqlens_k[b];
    const int lq = a.cu_seqlens_q[b + 1] - q0;
    const int lk = a.cu_seqlens_k[b + 1] - k0;
    const int row0 = mt * kPfBM;
    if (row0 >= lq) return;                              // also covers empty query spans
    const int off = lk - lq;                             // bottom-right causal alignment

    const int r = lane & 15, g = lane >> 4;              // column of the 16x16 products, 16-lane group
    const float c = a.scale_log2e;

    // Q^T fragments: B operand, column = this lane's query of group qa, k = dims 32 ks + 8 g + [0, 8)
    int qrow[2];                                         // query index inside the sequence
    bf16x8_t qfrag[2][4];
#pragma unroll
    for (int qa = 0; qa < 2; ++qa) {
        qrow[qa] = row0 + wave * 32 + 16 * qa + r;
        const bf16_t *qp = a.q + static_cast<int64_t>(q0 + min(qrow[qa], lq - 1)) * a.q_row_stride + h * kHeadDim + 8 * g;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) qfrag[qa][ks] = as_bf16x8(*reinterpret_cast<const u32x4_t *>(qp + 32 * ks));
    }

    f32x4_t oacc[8][2];                                  // [16-dim block][query group]: dim 16 db + 4 g + i
    // Exponent reference per query group, shared by the four lanes of a query: neg_ref = -c * (the
    // raw score that maps to p = 1).
    float neg_ref[2] = {0.f, 0.f};
    // Row sums: accumulated by the matrix pipe as a product of P^T with a block of ones (every row of
    // the 16x16 result is the sum over all 32 keys of the step), which costs 4 products per tile where
    // 32 additions per lane would compete with the exponentials for the vector pipe.  The sums are
    // thus taken over the bf16 values of P that the second product uses.
    f32x4_t lacc[2];

    // K tiles 0/1, then V tiles 0/1; a tile is 16 blocks of 1 KB, block (16-key group kb, 32-dim slice x)
    __shared__ __attribute__((aligned(1024))) unsigned char smem[4 * kPfTileBytes];
    __shared__ int retry_flag;
    const lds_char_ptr lds = (lds_char_ptr)(&smem[0]);

    const int q_hi = min(row0 + kPfBM, lq) - 1;          // last query row of the tile
    const int kv_end = min(lk, q_hi + off + 1);          // keys [0, kv_end) are visible to the tile
    const int ntiles = kv_end > 0 ? (kv_end + kPfBN - 1) / kPfBN : 0;
    const int wave_qmin = row0 + wave * 32;

    // ---- loads.  Wavefront w fetches key rows 16 w .. 16 w + 15 of a tile with four K and four V
    // instructions; instruction x covers bytes 64 x .. 64 x + 63 of those rows (4 lanes per row) and
    // fills block (w, x).  Lane 4 k + j of it fetches, for key k of the group, piece
    //     K: j ^ (-(k >> 2) & 3)   V: j ^ 2 ((k >> 2) & 1)
    // of the row's four 16-byte pieces.
    const int lk16 = lane >> 2, lj = lane & 3;
    const int lrow = wave * 16 + lk16;                   // this lane's key row within a tile
    const int kpiece = lj ^ ((0 - (lk16 >> 2)) & 3), vpiece = lj ^ (2 * ((lk16 >> 2) & 1));
    const int64_t kstride = kPaged ? static_cast<int64_t>(a.num_kv_heads) * kHeadDim : a.k_row_stride;
    const int64_t vstride = kPaged ? kstride : a.v_row_stride;
    const uint32_t lds_k0 = __builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + wave * 4096);
    struct NextTile { const char *kb, *vb; uint32_t ko, vo, dk, dv; };
    // Prepares the loads of key tile kt into LDS buffer `buf`; `ok` is false when the tile's block
    // table entry is out of range (the loads then read block 0 and the tile is masked out).
    auto plan_tile = [&](int kt, int32_t blk_v, int buf, bool &ok) __attribute__((always_inline)) -> NextTile {
        const int32_t blk = kPaged ? __builtin_amdgcn_readfirstlane(blk_v) : 0;
        ok = !kPaged || static_cast<uint32_t>(blk) < static_cast<uint32_t>(a.num_blocks);
        const int key0 = kt * kPfBN;
        NextTile t;
        if (kPaged) {
            const int64_t e = (((static_cast<int64_t>(ok ? blk : 0) << a.block_shift) + (key0 & ((1 << a.block_shift) - 1))) * a.num_kv_heads + hkv) *
                              kHeadDim * 2;
            t.kb = reinterpret_cast<const char *>(a.k_cache) + e;
            t.vb = reinterpret_cast<const char *>(a.v_cache) + e;
        } else {
            t.kb = reinterpret_cast<const char *>(a.k) + (static_cast<int64_t>(k0 + key0) * kstride + hkv * kHeadDim) * 2;
            t.vb = reinterpret_cast<const char *>(a.v) + (static_cast<int64_t>(k0 + key0) * vstride + hkv * kHeadDim) * 2;
        }
        const int row = min(lrow, lk - 1 - key0);        // rows past the last key repeat it and are masked later
        t.ko = static_cast<uint32_t>((row * kstride + kpiece * 8) * 2);
        t.vo = static_cast<uint32_t>((row * vstride + vpiece * 8) * 2);
        t.dk = lds_k0 + buf * kPfTileBytes;
        t.dv = t.dk + 2 * kPfTileBytes;
        return t;
    };
    auto issue_k = [&](NextTile &t, int x) __attribute__((always_inline)) { load_to_lds_16(t.kb + 64 * x, t.ko, t.dk + 1024 * x); };
    auto issue_v = [&](NextTile &t, int x) __attribute__((always_inline)) { load_to_lds_16(t.vb + 64 * x, t.vo, t.dv + 1024 * x); };

    // ---- operand reads.  K block (kb, ks): the piece of key k holding dims 32 ks + 8 g' + [0, 8) sits at
    // 16-byte slot 4 k + (g' ^ (-(k >> 2) & 3)).  V block (kb, x): key k owns 64 bytes, its two 32-byte
    // halves (16 dims each) swapped when (k >> 2) is odd.  A transpose read of a 16-lane group covers
    // 4 keys x 16 dims: lane r supplies the address of key r / 4, dims 4 (r % 4) .. + 3 and
    // receives dim r of the four keys.
    // Which lanes have to fall into different banks was measured: a 64-bit read serves lanes 0-31 in one
    // LDS cycle and 32-63 in the next; a 128-bit read serves 16 lanes per cycle, and they are not 16
    // neighbours but four aligned groups of four lanes: of the eight such groups of each half of the
    // wavefront, the ones numbered 0, 3, 5, 6 in one cycle and 1, 2, 4, 7 in the other.  The K
    // permutation above puts the four groups of a cycle on the four residues of the slot number
    // modulo 4 (with k >> 2 in place of -(k >> 2) & 3 groups 0 and 5 collide and every K read takes
    // twice as long).
    const uint32_t kread0 = 16 * (4 * r + (g ^ ((0 - (r >> 2)) & 3)));
    const uint32_t vread0 = 2 * kPfTileBytes + 64 * (4 * g + (r >> 2)) + 8 * (r & 3);
    const uint32_t vread_y0 = vread0 + 32 * (g & 1), vread_y1 = vread0 + 32 * ((g & 1) ^ 1);

    const std::integral_constant<int, 0> h0;
    const std::integral_constant<int, 1> h1;
    f32x4_t sacc[4][2];                                  // [16-key block][query group]: key 16 kb + 4 g + i
    u32x4_t pfrag[2][2];                                 // [32-key half][query group]

    // S^T = K Q^T for the two 16-key blocks of half H
    auto scores = [&](auto hc, lds_char_ptr kl) __attribute__((always_inline)) {
        constexpr int H = decltype(hc)::value;
#pragma unroll
        for (int kb = 2 * H; kb < 2 * H + 2; ++kb)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const u32x4_t kf = *(lds_u32x4_ptr)(kl + (kb * 4 + ks) * 1024);
#pragma unroll
                for (int qa = 0; qa < 2; ++qa)
                    sacc[kb][qa] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        as_bf16x8(kf), qfrag[qa][ks], ks == 0 ? f32x4_t{0.f, 0.f, 0.f, 0.f} : sacc[kb][qa], 0, 0, 0);
            }
    };
    // score of register e (0..7) of half H, masked: key index kt*64 + 32 H + 16 (e/4) + 4 g + e%4
    auto masked_score = [&](auto hc, auto dc, int qa, int e, int key_base, int limit) __attribute__((always_inline)) -> float {
        constexpr int H = decltype(hc)::value;
        constexpr bool kDiag = decltype(dc)::value;
        const float s = sacc[2 * H + (e >> 2)][qa][e & 3];
        return (kDiag && key_base + 32 * H + 16 * (e >> 2) + (e & 3) > limit) ? -INFINITY : s;
    };
    // running maximum of the (masked) scores of half H, per lane
    auto row_max = [&](auto hc, int key_base, bool cur_ok, float (&m)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int qa = 0; qa < 2; ++qa) {
            const int limit = cur_ok ? qrow[qa] + off : -1;
#pragma unroll
            for (int e = 0; e < 8; ++e) m[qa] = fmaxf(m[qa], masked_score(hc, std::true_type{}, qa, e, key_base, limit));
        }
    };
    // One tile of the attention proper, written out in the order it is to execute and fenced step by
    // step (left to itself the scheduler issues every LDS read right before its use and keeps each
    // softmax in one piece, so that reads, exponentials and products wait for one another):
    //   1  the 8 K reads of the first half
    //   2  its 16 products, the 8 K reads of the second half and the next tile's K loads between them
    //   3  the second half's 16 products, each followed by one score of the first half going through
    //      the softmax and one V read of the first half
    //   4  the first half's 16 P V products, each followed by one score of the second half going
    //      through the softmax and one V read of the second half
    //   5  the second half's 16 P V products, the next tile's V loads between them
    // A read is thus issued 8 to 16 products before its use, and the exponentials run beside products.
    auto attend = [&](auto dc, auto lc, lds_char_ptr kl, lds_char_ptr vl0, lds_char_ptr vl1, int key_base, bool cur_ok,
                      NextTile &nxt) __attribute__((always_inline)) {
        constexpr bool kLoads = decltype(lc)::value;       // false for the last tile of the pass: nothing follows it
        const int limit[2] = {cur_ok ? qrow[0] + off : -1, cur_ok ? qrow[1] + off : -1};   // last key a query may see
        const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
        const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};     // eight bf16 1.0
        u32x4_t kfa[8], kfb[8];
        s16x4_t vta[16], vtb[16];
        float pprev = 0.f;
        // one score of half H through the softmax: j = 8 qa + e
        auto slice = [&](auto hc, int j) __attribute__((always_inline)) {
            constexpr int H = decltype(hc)::value;
            const int qa = j >> 3, e = j & 7;
            const float p = __builtin_amdgcn_exp2f(fmaf(masked_score(hc, dc, qa, e, key_base, limit[qa]), c, neg_ref[qa]));   // exp2(-inf) = 0
            if (e & 1) pfrag[H][qa][e >> 1] = pack_bf16x2(pprev, p);
            else pprev = p;
        };
        auto vread = [&](auto hc, int j) __attribute__((always_inline)) -> s16x4_t {    // j = 2 db + (0: keys 0..15, 1: keys 16..31 of the half)
            constexpr int H = decltype(hc)::value;
            const int db = j >> 1;
            const lds_char_ptr vl = (db & 1) ? vl1 : vl0;
            return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(vl + ((2 * H + (j & 1)) * 4 + (db >> 1)) * 1024));
        };
#pragma unroll
        for (int i = 0; i < 8; ++i) kfa[i] = *(lds_u32x4_ptr)(kl + i * 1024);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int kb = i >> 2, ks = i & 3;
#pragma unroll
            for (int qa = 0; qa < 2; ++qa)
                sacc[kb][qa] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kfa[i]), qfrag[qa][ks], ks == 0 ? zero : sacc[kb][qa], 0, 0, 0);
            kfb[i] = *(lds_u32x4_ptr)(kl + (8 + i) * 1024);
            if (kLoads && (i & 1) == 0) issue_k(nxt, i >> 1);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int i = j >> 1, qa = j & 1, kb = 2 + (i >> 2), ks = i & 3;
            sacc[kb][qa] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kfb[i]), qfrag[qa][ks], ks == 0 ? zero : sacc[kb][qa], 0, 0, 0);
            slice(h0, j);
            vta[j] = vread(h0, j);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int qa = 0; qa < 2; ++qa)
            lacc[qa] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(ones), as_bf16x8(pfrag[0][qa]), lacc[qa], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int db = j >> 1, qa = j & 1;
            const s16x8_t both = __builtin_shufflevector(vta[2 * db], vta[2 * db + 1], 0, 1, 2, 3, 4, 5, 6, 7);
            oacc[db][qa] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, both), as_bf16x8(pfrag[0][qa]), oacc[db][qa], 0, 0, 0);
            slice(h1, j);
            vtb[j] = vread(h1, j);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int qa = 0; qa < 2; ++qa)
            lacc[qa] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(ones), as_bf16x8(pfrag[1][qa]), lacc[qa], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int db = j >> 1, qa = j & 1;
            const s16x8_t both = __builtin_shufflevector(vtb[2 * db], vtb[2 * db + 1], 0, 1, 2, 3, 4, 5, 6, 7);
            oacc[db][qa] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, both), as_bf16x8(pfrag[1][qa]), oacc[db][qa], 0, 0, 0);
            if (kLoads && (j & 3) == 0) issue_v(nxt, j >> 2);
            if (j & 1) __builtin_amdgcn_sched_barrier(0);
        }
    };
    int retry_pending = 0;

    // One pass over the key tiles.  kExact = false: the attention itself, with the exponent reference
    // taken from the first 32 keys.  kExact = true: only the scores, for the exact row maxima.
    auto pass = [&](auto xc) __attribute__((always_inline)) {
        constexpr bool kExact = decltype(xc)::value;
        float m_exact[2] = {-INFINITY, -INFINITY};
        bool tile_ok = true;                             // of the tile computed next
        int32_t blk_next = 0;                            // block id of the tile loaded next
        if (ntiles > 0) {
            NextTile t = plan_tile(0, blk_first, 0, tile_ok);
#pragma unroll
            for (int x = 0; x < 4; ++x) { issue_k(t, x); issue_v(t, x); }
            loads_issued(t.ko, t.vo);
        }
        if (ntiles > 1) blk_next = blk_second;
        // Everything loaded so far (Q above all) is waited for here, and the Q fragments are then
        // passed through an empty asm.  Without this the compiler keeps treating them as in flight
        // inside the loop and makes each product wait for the loads issued just before it -- the
        // next tile's prefetch -- which put a full memory round trip into every tile.
        __builtin_amdgcn_s_waitcnt(0x0F70);              // vmcnt(0): also the first tile has landed in LDS
#pragma unroll
        for (int qa = 0; qa < 2; ++qa)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) asm volatile("" : "+v"(qfrag[qa][ks]));
        __syncthreads();

        if (!kExact) {
#pragma unroll
            for (int db = 0; db < 8; ++db)
#pragma unroll
                for (int qa = 0; qa < 2; ++qa) oacc[db][qa] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            lacc[0] = lacc[1] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            if (retry_pending == 0 && ntiles > 0 && wave_qmin < lq) {
                // exponent reference: the largest score among the first 32 keys of the row.  Whatever it
                // is cancels in the final division; it only has to keep every p inside fp32 range.
                float m[2] = {-INFINITY, -INFINITY};
                scores(h0, lds + kread0);
                row_max(h0, 4 * g, tile_ok, m);
#pragma unroll
                for (int qa = 0; qa < 2; ++qa) {
                    m[qa] = fmaxf(m[qa], __shfl_xor(m[qa], 16, 64));
                    m[qa] = fmaxf(m[qa], __shfl_xor(m[qa], 32, 64));
                    neg_ref[qa] = m[qa] == -INFINITY ? 0.f : -m[qa] * c;
                }
            }
        }

        // Per wavefront the tiles come in three runs: those wholly below the diagonal for all of its 32
        // queries (no mask), those that cross it, and those wholly beyond it, of which only the loads
        // are this wavefront's business (they exist because later wavefronts of the workgroup see
        // them).  One loop per run, so that each loop has a single body.
        // (a wavefront whose 32 rows all lie past the end of the sequence only helps with the loads)
        const int n_active = wave_qmin >= lq ? 0 : min(ntiles, (wave_qmin + 31 + off) / kPfBN + 1);   // wave_qmin + 31 + off >= 0 or no tile at all
        const int n_plain = wave_qmin + off + 1 >= kPfBN ? min(n_active, (wave_qmin + off + 1) / kPfBN) : 0;
        // lc = false: the last tile of the pass.  Nothing is loaded during it and nobody waits after it.
        auto step = [&](int kt, auto dc, auto cc, auto lc) __attribute__((always_inline)) {
            constexpr bool kCompute = decltype(cc)::value;
            constexpr bool kLoads = decltype(lc)::value;
            const int buf = kt & 1;
            const bool cur_ok = tile_ok;
            // the next tile lands in the other buffer during this tile's arithmetic (that buffer was last
            // read before the previous barrier)
            NextTile nxt = {};
            if (kLoads) {
                nxt = plan_tile(kt + 1, blk_next, buf ^ 1, tile_ok);
                if (kt + 2 < ntiles) blk_next = fetch_block(kt + 2);
            }
            if (kCompute) {
                const lds_char_ptr kl = lds + (kread0 + buf * kPfTileBytes);
                const lds_char_ptr vl0 = lds + (vread_y0 + buf * kPfTileBytes), vl1 = lds + (vread_y1 + buf * kPfTileBytes);
                const int key_base = kt * kPfBN + 4 * g; // key of register 0 of block 0
                if (kExact) {
                    if (kLoads) {
#pragma unroll
                        for (int x = 0; x < 4; ++x) issue_k(nxt, x);
                    }
                    scores(h0, kl);
                    scores(h1, kl);
                    row_max(h0, key_base, cur_ok, m_exact);
                    row_max(h1, key_base, cur_ok, m_exact);
                } else {
                    attend(dc, lc, kl, vl0, vl1, key_base, cur_ok, nxt);
                }
            } else if (kLoads) {
#pragma unroll
                for (int x = 0; x < 4; ++x) { issue_k(nxt, x); if (!kExact) issue_v(nxt, x); }
            }
            if (kLoads) {
                loads_issued(nxt.ko, nxt.vo);
                __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): this wavefront's part of the next tile is in LDS
                __syncthreads();
            }
        };
        const std::true_type yes;
        const std::false_type no;
        const int last = ntiles - 1;
        int kt = 0;
        for (; kt < min(n_plain, last); ++kt) {
            if (kPaged && !tile_ok) step(kt, yes, no, yes);     // (a tile behind a bad block id is masked out: nothing to add)
            else step(kt, no, yes, yes);
        }
        for (; kt < min(n_active, last); ++kt) {
            // (behind a bad block id the loads were pointed at block 0, which may never have been written:
            // with every score masked the products would still be 0 x its contents, and 0 x NaN is NaN)
            if (kPaged && !tile_ok) step(kt, yes, no, yes);
            else step(kt, yes, yes, yes);
        }
        for (; kt < last; ++kt) step(kt, yes, no, yes);
        if (last >= 0 && last < n_active && !(kPaged && !tile_ok)) step(last, yes, yes, no);    // (with the mask, needed or not: one body fewer)
        if (kExact) {
#pragma unroll
            for (int qa = 0; qa < 2; ++qa) {
                m_exact[qa] = fmaxf(m_exact[qa], __shfl_xor(m_exact[qa], 16, 64));
                m_exact[qa] = fmaxf(m_exact[qa], __shfl_xor(m_exact[qa], 32, 64));
                neg_ref[qa] = m_exact[qa] == -INFINITY ? 0.f : -m_exact[qa] * c;
            }
        }
    };

    // First with the cheap reference.  If a row sum of the workgroup then lies beyond 2^100 (or is not a
    // number), some score exceeded the first 32 keys' maximum by hundreds: the workgroup computes the
    // exact row maxima in a pass of their own and repeats the attention with them (p <= 1).
    float l_tot[2];
    for (;;) {
        pass(std::false_type{});
        bool beyond = false;
#pragma unroll
        for (int qa = 0; qa < 2; ++qa) {
            l_tot[qa] = lacc[qa][0];
            beyond |= !(l_tot[qa] <= kPfLiftLimit);
        }
        if (retry_pending) {
            __syncthreads();                             // (the output tiles go through the LDS the last tile is read from)
            break;
        }
        if (tid == 0) retry_flag = 0;
        __syncthreads();
        if (beyond) retry_flag = 1;
        __syncthreads();
        if (retry_flag == 0) break;
        retry_pending = 1;
        pass(std::true_type{});
        __syncthreads();                                 // (its last tile is still being read while a faster wavefront would already load tile 0 again)
    }

    // ---- normalise and store.  Register i of block db is dim 16 db + 4 g + i of one query: stored from
    // there a lane would write 8 bytes here and 8 bytes 32 bytes further on.  Each wavefront passes its
    // 32 x 128 tile through LDS instead (the K/V tiles are done with; rows 272 bytes apart, so that the
    // 64-bit writes of 32 lanes fall into 32 different bank pairs) and stores whole rows, 16 bytes per lane.
    constexpr int kOutPitch = 2 * kHeadDim + 16;
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(3))) u32x2_t *lds_u32x2_ptr;
    const lds_char_ptr ow = lds + wave * (32 * kOutPitch);
#pragma unroll
    for (int qa = 0; qa < 2; ++qa) {
        const float inv = l_tot[qa] > 0.f ? 1.f / l_tot[qa] : 0.f;
#pragma unroll
        for (int db = 0; db < 8; ++db) {
            const u32x2_t w = {pack_bf16x2(oacc[db][qa][0] * inv, oacc[db][qa][1] * inv),
                               pack_bf16x2(oacc[db][qa][2] * inv, oacc[db][qa][3] * inv)};
            *(lds_u32x2_ptr)(ow + (16 * qa + r) * kOutPitch + (16 * db + 4 * g) * 2) = w;
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int orow = 4 * i + (lane >> 4);
        const u32x4_t w = *(lds_u32x4_ptr)(ow + orow * kOutPitch + (lane & 15) * 16);
        const int qr = row0 + wave * 32 + orow;
        if (qr < lq)
            *reinterpret_cast<u32x4_t *>(a.out + (static_cast<int64_t>(q0 + qr) * a.num_heads + h) * kHeadDim + (lane & 15) * 8) = w;
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
        if (block_shift_of(block_size) < 0) return NVA_ERR_UNSUPPORTED_GEOMETRY;
        if (!k_cache || !v_cache) return NVA_ERR_NULL_POINTER;
        if (max_blocks <= 0 || num_blocks <= 0) return NVA_ERR_BAD_SHAPE;
        if (bt_row_stride < max_blocks) return NVA_ERR_BAD_STRIDE;
        if (static_cast<int64_t>(max_blocks) * block_size < max_seqlen_k) return NVA_ERR_BAD_SHAPE;
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
    a.block_shift = paged ? block_shift_of(block_size) : 8;
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
