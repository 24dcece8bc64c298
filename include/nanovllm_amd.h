/*
 * nanovllm_amd -- C ABI of the MI355X (gfx950) attention hot path for nano-vllm.
 *
 * Every entry point borrows raw device pointers for the duration of one asynchronous
 * launch on the HIP stream it is given.  The library never allocates or frees device
 * memory, never synchronises and never reads device data on the host, so all calls are
 * legal under stream capture.  Scratch memory is supplied by the caller (query its size
 * with the *_workspace_bytes functions).  Arguments are validated on the host before any
 * launch; a non-zero return means nothing was enqueued.
 *
 * Dtypes / geometry: bf16 tensors, int32 index tensors, head_dim 128, KV blocks of 256, 512,
 * 1024, 2048 or 4096 tokens, num_heads / num_kv_heads from 1 to 8 (decode; prefill takes any
 * multiple).  Anything else is rejected with
 * NVA_ERR_UNSUPPORTED_GEOMETRY rather than served by a slow path.
 *
 * File:line citations name the reference (nano-vllm) interface each entry point replaces.
 */
#ifndef NANOVLLM_AMD_H
#define NANOVLLM_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum nva_status {
    NVA_OK = 0,
    NVA_ERR_NULL_POINTER = 1,         /* a required pointer is NULL                         */
    NVA_ERR_BAD_SHAPE = 2,            /* negative / inconsistent counts                     */
    NVA_ERR_UNSUPPORTED_GEOMETRY = 3, /* head_dim, block_size or GQA group not built        */
    NVA_ERR_BAD_STRIDE = 4,           /* row stride smaller than a row, or not 16-byte      */
    NVA_ERR_MISALIGNED = 5,           /* base pointer not 16-byte aligned                   */
    NVA_ERR_WORKSPACE_TOO_SMALL = 6,  /* workspace_bytes below *_workspace_bytes()          */
    NVA_ERR_LAUNCH_FAILED = 7,        /* hipGetLastError() after the launch was not success */
    NVA_ERR_NO_DEVICE = 8,            /* no HIP device visible                              */
    NVA_ERR_SCRATCH_TOO_SMALL = 9     /* problem exceeds the library's built-in scratch array */
};

/* Library version, (major << 16) | minor. */
int nva_version(void);

/* Static, human-readable name of a status code (never NULL). */
const char *nva_status_string(int status);

/* Number of visible HIP devices; NVA_ERR_NO_DEVICE (and *count = 0) when there is none. */
int nva_device_count(int *count);

/*
 * KV-cache slot scatter.  Replaces store_kvcache / store_kvcache_kernel
 * (nanovllm/layers/attention.py:10-40).
 *
 * key/value: bf16 [n_tokens, num_kv_heads, head_dim], innermost two dims dense, row
 * strides in ELEMENTS (value is a strided view of the fused qkv buffer in the model).
 * k_cache/v_cache: bf16, addressed flat as [num_slots, num_kv_heads*head_dim].
 * slot_mapping: int32 [n_tokens]; row i goes to cache row slot_mapping[i]; -1 skips the
 * row.  Slots outside [0, num_slots) are skipped as well instead of written out of
 * bounds.  Duplicate slots are safe; which row wins is unspecified (as in the reference).
 * The copy is bit-exact.  n_tokens == 0 is a no-op.
 */
int nva_store_kvcache(const void *key, int64_t key_row_stride,
                      const void *value, int64_t value_row_stride,
                      void *k_cache, void *v_cache,
                      const int32_t *slot_mapping,
                      int32_t n_tokens, int32_t num_kv_heads, int32_t head_dim,
                      int64_t num_slots, void *stream);

/*
 * Paged single-query (decode) attention.  Replaces the flash_attn_with_kvcache call of
 * Attention.forward (nanovllm/layers/attention.py:71-74).
 *
 * q: bf16 [batch, num_heads, head_dim], row stride q_row_stride elements, heads dense.
 * k_cache/v_cache: bf16 [num_blocks, block_size, num_kv_heads, head_dim], dense.
 * block_tables: int32 [batch, max_blocks] with row stride bt_row_stride; only entries
 * j < ceil(context_lens[b] / block_size) are dereferenced (the rest may be -1 or stale);
 * an entry outside [0, num_blocks) contributes nothing instead of faulting.
 * context_lens: int32 [batch]; 0 yields an all-zero output row.
 * out: bf16 [batch, num_heads, head_dim] dense (the reference's [B,1,Hq,Dh]).
 * workspace: at least nva_paged_decode_workspace_bytes() bytes, 16-byte aligned; holds
 * split partials, contents need no initialisation.  Calls that overlap in time need
 * separate workspaces; calls ordered on one stream (every layer of a model) can share one.
 * Launch geometry depends only on (batch, heads), never on device data, so a call can be
 * captured in a HIP graph and replayed with new contents.
 */
size_t nva_paged_decode_workspace_bytes(int32_t batch, int32_t num_heads, int32_t head_dim,
                                        int32_t max_blocks);

int nva_paged_decode_attn(const void *q, int64_t q_row_stride,
                          const void *k_cache, const void *v_cache,
                          const int32_t *block_tables, int32_t bt_row_stride, int32_t max_blocks,
                          const int32_t *context_lens,
                          void *out, void *workspace, size_t workspace_bytes,
                          int32_t batch, int32_t num_heads, int32_t num_kv_heads,
                          int32_t head_dim, int32_t block_size, int32_t num_blocks,
                          float scale, void *stream);

/*
 * The same operation for a caller that makes several calls over the SAME context_lens and
 * block_tables contents, batch, head counts and workspace, ordered on one stream -- the
 * layers of one decode step (the loop over decoder layers around
 * nanovllm/layers/attention.py:71-74 changes only q and the cache pointers).
 *   plan == NVA_PLAN_BUILD: as nva_paged_decode_attn; the work split it derives from
 *     context_lens and block_tables stays in the workspace.
 *   plan == NVA_PLAN_REUSE: takes the split the last NVA_PLAN_BUILD call left in this
 *     workspace instead of deriving it again (saves a few microseconds per launch).  The caller
 *     guarantees that call had the same batch, head counts, num_blocks and table contents
 *     and that nothing else wrote the workspace since; otherwise the result is undefined
 *     (memory accesses stay inside the caches as long as the old block numbers were valid).
 * Batches above 1024 sequences are run as several launches and always rebuild.
 */
enum { NVA_PLAN_BUILD = 0, NVA_PLAN_REUSE = 1 };

int nva_paged_decode_attn_planned(const void *q, int64_t q_row_stride,
                                  const void *k_cache, const void *v_cache,
                                  const int32_t *block_tables, int32_t bt_row_stride,
                                  int32_t max_blocks, const int32_t *context_lens,
                                  void *out, void *workspace, size_t workspace_bytes,
                                  int32_t batch, int32_t num_heads, int32_t num_kv_heads,
                                  int32_t head_dim, int32_t block_size, int32_t num_blocks,
                                  float scale, int32_t plan, void *stream);

/*
 * Causal variable-length prefill attention, optionally reading K/V through the paged
 * cache.  Replaces the flash_attn_varlen_func call of Attention.forward
 * (nanovllm/layers/attention.py:64-70).
 *
 * q: bf16 [total_q, num_heads, head_dim], row stride q_row_stride elements.
 * block_tables == NULL: k/v are packed bf16 [total_k, num_kv_heads, head_dim] with their
 *   own row strides, sequence b owning rows cu_seqlens_k[b]..cu_seqlens_k[b+1].
 * block_tables != NULL: k/v are ignored (may be NULL) and every sequence reads its
 *   cu_seqlens_k[b+1]-cu_seqlens_k[b] logical positions from k_cache/v_cache through
 *   block_tables[b] (int32 [batch, max_blocks], row stride bt_row_stride, -1 padded).
 *   A table entry outside [0, num_blocks) that a sequence's keys reach contributes nothing
 *   (its 256 keys drop out) instead of faulting.
 * The causal mask is aligned to the END of the keys: query i of a sequence sees keys
 * j <= i + (Lk - Lq).  Empty query spans are no-ops.
 * out: bf16 [total_q, num_heads, head_dim] dense.  max_seqlen_q bounds the launch grid.
 */
int nva_varlen_prefill_attn(const void *q, int64_t q_row_stride,
                            const void *k, int64_t k_row_stride,
                            const void *v, int64_t v_row_stride,
                            const void *k_cache, const void *v_cache,
                            const int32_t *block_tables, int32_t bt_row_stride, int32_t max_blocks,
                            const int32_t *cu_seqlens_q, const int32_t *cu_seqlens_k,
                            int32_t batch, int32_t max_seqlen_q, int32_t max_seqlen_k,
                            void *out,
                            int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                            int32_t block_size, int32_t num_blocks,
                            float scale, void *stream);

/*
 * Temperature / exponential-race sampler.  Replaces Sampler.forward
 * (nanovllm/layers/sampler.py:10-15):
 *     token[b] = argmax_i softmax(float(logits[b]) / T[b])[i] / max(E[b,i], 1e-10)
 * with the first index winning ties.
 *
 * logits: bf16 [batch, vocab], row stride logits_row_stride elements.
 * temperatures: fp32 [batch].  T == 0 selects greedy argmax(logits) for that row (an
 * extension; the reference forbids T <= 1e-10, nanovllm/sampling_params.py:11).
 * noise: fp32 [batch, vocab] Exp(1) draws (row stride noise_row_stride): the formula above is
 * evaluated (scores relative to the maximum of each 4096-column chunk, rescaled to the row) and a
 * draw can be replayed; the argmax differs from the formula only between scores that agree to fp32
 * rounding.  NULL: the token is drawn from the same categorical distribution softmax(logits / T) by a
 * tree of inverse-CDF steps (row -> chunk of 8192 columns -> one of 4 column groups -> one of its 64
 * lanes -> one of the lane's 32 columns; at every level the first branch whose running sum of
 * weights exceeds u * total), each level with its own 32-bit uniform from Philox4x32-10 keyed by
 * (seed, offset, row, chunk); the same (seed, offset) reproduces the draw.  Sums are fp32 and a
 * conditional probability below 2^-32 at a level is not resolved.
 * out_tokens: int64 [batch].
 * workspace: at least nva_sample_workspace_bytes() bytes, 16-byte aligned.  Its size (and the limit
 * of nva_sample_static below) is counted in records of 2048 columns, the finest chunking any path
 * has used; the present chunkings (4096 columns with a noise tensor, 8192 without) need fewer.
 */
size_t nva_sample_workspace_bytes(int32_t batch, int32_t vocab);

int nva_sample(const void *logits, int64_t logits_row_stride,
               const float *temperatures,
               const float *noise, int64_t noise_row_stride,
               uint64_t seed, uint64_t offset,
               int64_t *out_tokens,
               void *workspace, size_t workspace_bytes,
               int32_t batch, int32_t vocab, void *stream);

/*
 * nva_sample without a workspace argument, for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments, kernels and results as nva_sample; the per-chunk
 * records live in a device array built into the library (2 MiB per GPU the library is used on, held
 * until the process ends), which bounds the problem size:
 *     batch * ceil(vocab / 2048) <= NVA_SAMPLE_STATIC_MAX_RECORDS      (1747 rows at vocab 151,936)
 * Larger problems return NVA_ERR_SCRATCH_TOO_SMALL and launch nothing.  The call allocates and frees
 * nothing; the first call on a device looks the array's address up (make that call outside stream
 * capture).  All calls on one GPU share the array: calls that overlap in time on one GPU race and
 * must be ordered by the caller (one stream, or events); nothing needs clearing between calls.
 */
#define NVA_SAMPLE_STATIC_MAX_RECORDS 131072

int nva_sample_static(const void *logits, int64_t logits_row_stride,
                      const float *temperatures,
                      const float *noise, int64_t noise_row_stride,
                      uint64_t seed, uint64_t offset,
                      int64_t *out_tokens,
                      int32_t batch, int32_t vocab, void *stream);

/*
 * ---- steps either side of the hot path (the callers' element-wise glue) ----------------
 */

/*
 * RMSNorm, optionally fused with the residual add.  Replaces RMSNorm.rms_forward /
 * add_rms_forward (nanovllm/layers/layernorm.py:16-40).
 *   residual == NULL: out = bf16(x * rsqrt(mean(x^2) + eps)) * weight
 *   otherwise:        s = x + residual (fp32); residual_out = bf16(s);
 *                     out = bf16(s * rsqrt(mean(s^2) + eps)) * weight
 * x / residual: bf16 [rows, hidden] with row strides in elements; weight bf16 [hidden];
 * out / residual_out: bf16 [rows, hidden] dense.  hidden % 8 == 0, hidden <= 4096.
 */
int nva_rms_norm(const void *x, int64_t x_row_stride,
                 const void *residual, int64_t residual_row_stride,
                 const void *weight, void *out, void *residual_out,
                 int32_t rows, int32_t hidden, float eps, void *stream);

/*
 * Final norm of a prefill step on the rows that feed the LM head only.  Replaces the pair
 * "hidden_states, _ = self.norm(hidden_states, residual)" (nanovllm/models/qwen3.py:176) +
 * "x = x[cu_seqlens_q[1:] - 1].contiguous()" (nanovllm/layers/embed_head.py:56-61): the reference
 * normalises all total_rows rows and then copies the last row of every sequence; this reads and
 * normalises those batch rows alone, bit-identical to the rows nva_rms_norm would have produced.
 *   i = cu_seqlens_q[b + 1] - 1  (a negative index wraps to total_rows + i, as torch indexing does;
 *                                 an empty query span picks the previous sequence's last row, as in
 *                                 the reference; indices are clamped to the tensor)
 *   out[b] = bf16(s * rsqrt(mean(s^2) + eps)) * weight,  s = x[i] (+ residual[i] when residual != NULL)
 * x / residual: bf16 [total_rows, hidden], row strides in elements; cu_seqlens_q: int32 [batch + 1];
 * out: bf16 [batch, hidden] dense.  hidden % 8 == 0, hidden <= 4096.
 */
int nva_gather_last_rms_norm(const void *x, int64_t x_row_stride,
                             const void *residual, int64_t residual_row_stride,
                             const int32_t *cu_seqlens_q, const void *weight, void *out,
                             int32_t batch, int32_t total_rows, int32_t hidden, float eps, void *stream);

/*
 * Per-head RMSNorm of q and k followed by the neox rotary embedding, optionally fused with the
 * KV-cache scatter.  Replaces the q_norm / k_norm / rotary_emb sequence of
 * Qwen3Attention.forward (nanovllm/models/qwen3.py:76-79; nanovllm/layers/rotary_embedding.py:6-48)
 * and, when a cache is given, the store_kvcache call of Attention.forward
 * (nanovllm/layers/attention.py:62-63) for the same rows.
 * qkv: bf16 [n_tokens, (num_heads + 2*num_kv_heads) * head_dim], row stride in elements
 * (q heads, then k heads, then v heads).  positions: int64 [n_tokens].
 * q_weight / k_weight: bf16 [head_dim].  rope_cache: fp32 [max_position, head_dim], cos in
 * the first half of a row, sin in the second; positions are clamped to [0, max_position).
 * q_out: bf16 [n_tokens, num_heads, head_dim], k_out: bf16 [n_tokens, num_kv_heads, head_dim],
 * both dense.  head_dim must be 128.
 * k_cache / v_cache / slot_mapping: all NULL (no scatter), or the flat caches
 * [num_slots, num_kv_heads * head_dim] and int32 [n_tokens] slots: the rotated key row and the
 * (unchanged) value row of token i are also written to cache row slot_mapping[i], bit-identical
 * to what nva_store_kvcache would write from k_out and the v view; -1 / out-of-range skips.
 * Every tensor pointer must be 16-byte aligned and qkv_row_stride a multiple of 8 elements
 * (NVA_ERR_MISALIGNED / NVA_ERR_BAD_STRIDE otherwise): all accesses are 16 bytes per lane.
 */
int nva_qk_norm_rope(const void *qkv, int64_t qkv_row_stride, const int64_t *positions,
                     const void *q_weight, const void *k_weight, const float *rope_cache,
                     int32_t max_position, void *q_out, void *k_out,
                     void *k_cache, void *v_cache, const int32_t *slot_mapping, int64_t num_slots,
                     int32_t n_tokens, int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                     float eps, void *stream);

/*
 * SwiGLU gate.  Replaces SiluAndMul.forward (nanovllm/layers/activation.py:11-14):
 * out[r, i] = bf16(silu(x[r, i])) * x[r, inter + i].
 * x: bf16 [rows, 2*inter] (row stride in elements), out: bf16 [rows, inter] dense, inter % 8 == 0.
 */
int nva_silu_and_mul(const void *x, int64_t x_row_stride, void *out,
                     int32_t rows, int32_t inter, void *stream);

/*
 * Brings the per-step decode inputs from a pinned host buffer into their device buffer with one
 * kernel (the device reads host memory directly; no copy engine, no second launch), and feeds the
 * tokens sampled by the previous step to this one without a trip through the host.  It stands
 * where the reference copies input_ids, positions, slot_mapping, context_lens and block_tables
 * from the host one by one (nanovllm/engine/model_runner.py:162-179,197-203).
 *   dst[0 .. nbytes) = src_host[0 .. nbytes)                        (nbytes % 16 == 0, both 16-byte aligned)
 *   then, with ids = (int64*)(dst + ids_offset) and idx = (int32*)(src_host + index_offset), for i < n:
 *   ids[i] = prev_tokens[idx[i]] where 0 <= idx[i] < n_prev         (other rows keep the host's value)
 * src_host must be device-accessible host memory (hipHostMalloc / a pinned torch tensor).
 * prev_tokens: int64 [n_prev], the sampler's output of the previous step; NULL with n_prev == 0.
 */
int nva_stage_decode_inputs(void *dst, const void *src_host, int64_t nbytes, int64_t ids_offset,
                            int64_t index_offset, int32_t n, const int64_t *prev_tokens, int32_t n_prev,
                            void *stream);

/*
 * Calibration, no counterpart in the reference: streams nbytes from src with the access discipline of
 * the decode kernel (2048 wavefront workers, contiguous slices, 16-byte non-temporal loads) and keeps
 * nothing.  Its duration is what any kernel that reads that many bytes needs at least on this GPU;
 * bench.py reports it next to the roofline fractions.  src 16-byte aligned, nbytes % 16 == 0; sink:
 * at least 4 writable bytes of device memory (practically never written).
 */
int nva_probe_stream_read(const void *src, int64_t nbytes, void *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* NANOVLLM_AMD_H */
