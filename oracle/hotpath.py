"""Eager-PyTorch CPU restatement of the reference's four hot-path device ops.

TEST INFRASTRUCTURE: imported only by tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg.  Each function cites the reference lines it follows.

Precision modes for the two attention functions
  "fp32"  q, K, V upcast to fp32, fp32 softmax and output -- the tolerance reference the
          device kernels are compared against (max-abs 2e-2 / mean-abs 2e-3 in bf16).
  "sdpa"  the reference semantics as a plain CPU path: bf16 tensors through
          torch.nn.functional.scaled_dot_product_attention (what bench.py times as the
          cpu_baseline).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

__all__ = [
    "store_kvcache",
    "gather_pages",
    "paged_decode_attention",
    "varlen_prefill_attention",
    "sample",
    "sample_scores",
]


# --------------------------------------------------------------------------------------
# KV-cache slot scatter
# --------------------------------------------------------------------------------------
def store_kvcache(key, value, k_cache, v_cache, slot_mapping):
    """Scatter token rows into the flat paged cache, in place.

    Follows nanovllm/layers/attention.py:10-40: program ``i`` reads ``slot_mapping[i]``,
    returns if it is ``-1`` (:22), otherwise copies the ``D = Hkv*Dh`` elements of key row
    ``i`` / value row ``i`` (each with its own row stride, :23-26) to cache row ``slot``
    (:27-29).  Caches are addressed flat as ``[num_slots, D]`` (:38).
    """
    n, hkv, dh = key.shape
    d = hkv * dh
    assert value.shape == key.shape
    assert slot_mapping.numel() == n                      # attention.py:39
    assert k_cache.numel() % d == 0 and v_cache.numel() % d == 0
    slots = slot_mapping.reshape(-1).to(torch.int64)
    keep = slots != -1
    idx = slots[keep]
    num_slots = k_cache.numel() // d
    assert idx.numel() == 0 or (int(idx.min()) >= 0 and int(idx.max()) < num_slots)
    k_cache.view(num_slots, d).index_copy_(0, idx, key.reshape(n, d)[keep])
    v_cache.view(num_slots, d).index_copy_(0, idx, value.reshape(n, d)[keep])
    return k_cache, v_cache


# --------------------------------------------------------------------------------------
# Block-table indexing
# --------------------------------------------------------------------------------------
def gather_pages(cache, block_table_row, num_tokens):
    """Dense ``[num_tokens, Hkv, Dh]`` view of one sequence's keys (or values).

    Logical position ``p`` of a sequence lives at ``cache[block_table[p // page], p % page]``
    -- the layout nanovllm/engine/model_runner.py:100-117 allocates
    (``[num_blocks, block_size, Hkv, Dh]`` per layer) and that the slot formula of
    model_runner.py:146-152,172 writes to (``slot = block_id * block_size + offset``).
    Only the first ``ceil(num_tokens / page)`` table entries are dereferenced.
    """
    page = cache.shape[1]
    nblk = (int(num_tokens) + page - 1) // page
    ids = block_table_row[:nblk].to(torch.int64)
    assert nblk == 0 or (int(ids.min()) >= 0 and int(ids.max()) < cache.shape[0])
    return cache[ids].reshape(nblk * page, *cache.shape[2:])[: int(num_tokens)]


def _attend(q, k, v, scale, q_offset, precision):
    """softmax(q k^T * scale + causal) v for one sequence.

    q [Lq, Hq, Dh], k/v [Lk, Hkv, Dh].  Query row i may see key j iff j <= i + q_offset
    (q_offset = Lk - Lq: bottom-right alignment, flash-attn >= 2.1 ``causal=True``).
    Query head h reads kv head ``h // (Hq // Hkv)``.
    """
    lq, hq, dh = q.shape
    lk, hkv, _ = k.shape
    group = hq // hkv
    i = torch.arange(lq).unsqueeze(1)
    j = torch.arange(lk).unsqueeze(0)
    allowed = j <= i + q_offset                                     # [Lq, Lk]
    if precision == "fp32":
        qf = q.float().permute(1, 0, 2)                             # [Hq, Lq, Dh]
        kf = k.float().permute(1, 0, 2).repeat_interleave(group, dim=0)
        vf = v.float().permute(1, 0, 2).repeat_interleave(group, dim=0)
        s = torch.matmul(qf, kf.transpose(1, 2)) * scale            # [Hq, Lq, Lk]
        s = s.masked_fill(~allowed, float("-inf"))
        p = torch.softmax(s, dim=-1)
        p = torch.nan_to_num(p, nan=0.0)                            # rows with no visible key -> 0
        return torch.matmul(p, vf).permute(1, 0, 2).contiguous()    # [Lq, Hq, Dh] fp32
    if precision == "sdpa":
        qh = q.permute(1, 0, 2).unsqueeze(0)                        # [1, Hq, Lq, Dh]
        kh = k.permute(1, 0, 2).repeat_interleave(group, dim=0).unsqueeze(0)
        vh = v.permute(1, 0, 2).repeat_interleave(group, dim=0).unsqueeze(0)
        o = F.scaled_dot_product_attention(qh, kh, vh, attn_mask=allowed, scale=scale)
        return o.squeeze(0).permute(1, 0, 2).contiguous()
    raise ValueError(precision)


# --------------------------------------------------------------------------------------
# Paged decode attention
# --------------------------------------------------------------------------------------
def paged_decode_attention(q, k_cache, v_cache, context_lens, block_tables, scale, precision="fp32"):
    """One query token per sequence against its paged keys.

    Follows nanovllm/layers/attention.py:71-74 (``flash_attn_with_kvcache(q.unsqueeze(1),
    k_cache, v_cache, cache_seqlens=context_lens, block_table=block_tables,
    softmax_scale=scale, causal=True)``): sequence ``b`` attends over its first
    ``context_lens[b]`` logical positions, which already include the token the scatter just
    wrote (model_runner.py:170-172).  ``causal`` is a no-op for one query.  Rows with
    ``context_lens == 0`` (graph padding, model_runner.py:199-202) produce zeros.
    Returns ``[B, 1, Hq, Dh]`` like the reference.
    """
    b, hq, dh = q.shape
    out_dtype = torch.float32 if precision == "fp32" else q.dtype
    out = torch.zeros(b, 1, hq, dh, dtype=out_dtype)
    for s in range(b):
        n = int(context_lens[s])
        if n <= 0:
            continue
        k = gather_pages(k_cache, block_tables[s], n)
        v = gather_pages(v_cache, block_tables[s], n)
        out[s, 0] = _attend(q[s : s + 1], k, v, scale, n - 1, precision)[0]
    return out


# --------------------------------------------------------------------------------------
# Causal varlen prefill (optionally reading K/V through pages)
# --------------------------------------------------------------------------------------
def varlen_prefill_attention(q, k, v, cu_seqlens_q, cu_seqlens_k, scale,
                             k_cache=None, v_cache=None, block_tables=None, precision="fp32"):
    """Packed variable-length causal attention.

    Follows nanovllm/layers/attention.py:64-70.  With ``block_tables is None`` keys/values
    are the packed ``k``/``v`` rows ``cu_seqlens_k[b]:cu_seqlens_k[b+1]``; otherwise they are
    read from the paged cache for *every* sequence of the batch (:65-66), sequence ``b``
    owning ``cu_seqlens_k[b+1]-cu_seqlens_k[b]`` logical positions, the last
    ``cu_seqlens_q[b+1]-cu_seqlens_q[b]`` of which are the queries
    (model_runner.py:136-141).  An empty query span is a no-op.
    Returns ``[total_q, Hq, Dh]``.
    """
    total_q, hq, dh = q.shape
    out_dtype = torch.float32 if precision == "fp32" else q.dtype
    out = torch.zeros(total_q, hq, dh, dtype=out_dtype)
    nseq = cu_seqlens_q.numel() - 1
    for s in range(nseq):
        q0, q1 = int(cu_seqlens_q[s]), int(cu_seqlens_q[s + 1])
        k0, k1 = int(cu_seqlens_k[s]), int(cu_seqlens_k[s + 1])
        lq, lk = q1 - q0, k1 - k0
        if lq <= 0:
            continue
        if block_tables is not None:
            ks = gather_pages(k_cache, block_tables[s], lk)
            vs = gather_pages(v_cache, block_tables[s], lk)
        else:
            ks, vs = k[k0:k1], v[k0:k1]
        out[q0:q1] = _attend(q[q0:q1], ks, vs, scale, lk - lq, precision)
    return out


# --------------------------------------------------------------------------------------
# Sampler
# --------------------------------------------------------------------------------------
def sample_scores(logits, temperatures, noise):
    """The quantity whose row-argmax is the sampled token.

    Follows nanovllm/layers/sampler.py:12-14 line by line, with the Exp(1) tensor that the
    reference draws inside the compiled function (:14) passed in as ``noise``:
    ``softmax(logits.float() / T[:, None]) / clamp_min(noise, 1e-10)``.
    The inputs are not modified.
    """
    x = logits.float().div_(temperatures.float().unsqueeze(1))
    probs = torch.softmax(x, dim=-1)
    return probs.div_(noise.float().clamp_min(1e-10))


def sample(logits, temperatures, noise):
    """Sampled token id per row, int64 ``[B]`` (nanovllm/layers/sampler.py:14 ``argmax``).

    torch's argmax returns the first index among equal maxima.  Rows whose temperature is
    exactly 0 are an extension the reference forbids (sampling_params.py:11): they return
    ``argmax(logits)`` (greedy), with no noise.
    """
    t = temperatures.float()
    greedy = t == 0
    safe_t = torch.where(greedy, torch.ones_like(t), t)
    tokens = sample_scores(logits, safe_t, noise).argmax(dim=-1)
    if bool(greedy.any()):
        tokens = torch.where(greedy, logits.float().argmax(dim=-1), tokens)
    return tokens


# ------------------------------------------------------------------ draws without a noise tensor
def philox4x32_10(counter, key):
    """Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3",
    SC'11): ``counter`` four and ``key`` two 32-bit words; returns the four output words.
    Pinned by the known-answer vectors of the authors' Random123 distribution."""
    m0, m1, w0, w1 = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85
    c = [int(x) & 0xFFFFFFFF for x in counter]
    k = [int(x) & 0xFFFFFFFF for x in key]
    for _ in range(10):
        p0, p1 = m0 * c[0], m1 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & 0xFFFFFFFF, (p0 >> 32) ^ c[3] ^ k[1], p0 & 0xFFFFFFFF]
        k = [(k[0] + w0) & 0xFFFFFFFF, (k[1] + w1) & 0xFFFFFFFF]
    return c


def _unit_uniform(word):
    """32 random bits -> uniform in (0, 1): ``(word + 1/2) * 2**-32`` (exact in float64)."""
    return (int(word) + 0.5) * 2.0 ** -32


def _philox_words(seed, offset, row, stream):
    return philox4x32_10((row, stream, offset & 0xFFFFFFFF, (offset >> 32) & 0xFFFFFFFF),
                         (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))


def row_uniforms(seed, offset, batch):
    """The uniform in (0, 1) that the library draws at the ROW level (which 8192-column chunk) for
    row ``b`` of a call keyed by ``(seed, offset)`` when no noise tensor is given: first output word
    of Philox4x32-10 with counter ``(b, 0x5a17, offset_lo, offset_hi)`` and key
    ``(seed_lo, seed_hi)``, plus one half, times 2**-32.  float64 ``[batch]``."""
    out = torch.empty(batch, dtype=torch.float64)
    for b in range(batch):
        out[b] = _unit_uniform(_philox_words(seed, offset, b, 0x5A17)[0])
    return out


def inverse_cdf_bounds(logits, temperatures):
    """float64 running sums of ``softmax(logits / T)`` per row, ``[B, V]``: the token drawn for a
    uniform ``u`` is the first column whose running sum exceeds ``u`` -- a draw from the same
    categorical distribution as the exponential race of nanovllm/layers/sampler.py:12-14."""
    p = torch.softmax(logits.double() / temperatures.double().unsqueeze(1), dim=-1)
    return p.cumsum(-1)


# The library's draw without a noise tensor is a tree of such inverse-CDF draws, each level with its
# own uniform: row -> chunk of 8192 columns -> one of 4 column groups -> one of its 64 lanes -> one of
# the lane's 32 columns.  Column ``2048 v + 512 g + 8 l + i`` of a chunk (v < 4, g < 4, l < 64, i < 8)
# belongs to lane ``l`` of group ``g``; a lane's columns are walked in (v, i) order.
TREE_CHUNK = 8192


def _pick(weights, u):
    """Inverse-CDF step over a float64 weight vector: first index of positive weight whose running
    sum exceeds ``u * total`` (the last index of positive weight if rounding leaves none).  Also
    returns how far ``u`` lies from the nearer edge of the chosen interval, as a probability."""
    total = float(weights.sum())
    live = (weights > 0).nonzero().flatten()
    if live.numel() == 0:
        return -1, float("inf")
    incl = weights.cumsum(0)
    t = u * total
    hit = ((weights > 0) & (incl > t)).nonzero().flatten()
    idx = int(hit[0]) if hit.numel() else int(live[-1])
    hi = float(incl[idx]) / total
    lo = hi - float(weights[idx]) / total
    return idx, min(abs(u - lo), abs(hi - u))


def tree_draw(logits, temperatures, seed, offset):
    """float64 restatement of the library's draw from ``softmax(logits / T)`` without a noise
    tensor -- the same distribution as nanovllm/layers/sampler.py:12-14, by other randomness.

    Row ``b`` picks a chunk of 8192 columns by the chunk weights with ``row_uniforms``; inside chunk
    ``c`` the first three output words of Philox counter ``(b, 0x10000 + c, offset)`` pick, in turn,
    one of the 4 column groups, one of its 64 lanes and one of the lane's 32 columns, each by its
    share of the level's weight.  Returns ``(tokens int64 [B], margins float64 [B])``: the margin is
    the smallest distance, over the levels, between a level's uniform and the edges of the interval
    it fell into -- where it is tiny, fp32 sums may legitimately pick the neighbour.
    A row without a finite logit yields token 0.
    """
    batch, vocab = logits.shape
    nchunks = -(-vocab // TREE_CHUNK)
    tokens = torch.zeros(batch, dtype=torch.int64)
    margins = torch.full((batch,), float("inf"), dtype=torch.float64)
    cols = torch.arange(TREE_CHUNK).view(4, 4, 64, 8)                 # [v, group, lane, i] -> column inside the chunk
    for b in range(batch):
        y = logits[b].double() / float(temperatures[b])
        top = float(y.max())
        if top == float("-inf"):
            continue
        w = torch.zeros(nchunks * TREE_CHUNK, dtype=torch.float64)
        w[:vocab] = torch.exp(y - top)
        c, margin = _pick(w.view(nchunks, -1).sum(-1), _unit_uniform(_philox_words(seed, offset, b, 0x5A17)[0]))
        words = _philox_words(seed, offset, b, 0x10000 + c)
        node = w[c * TREE_CHUNK:(c + 1) * TREE_CHUNK].view(4, 4, 64, 8)
        g, mg = _pick(node.sum(dim=(0, 2, 3)), _unit_uniform(words[0]))
        margin = min(margin, mg)
        l, mg = _pick(node[:, g].sum(dim=(0, 2)), _unit_uniform(words[1]))
        margin = min(margin, mg)
        i, mg = _pick(node[:, g, l].reshape(32), _unit_uniform(words[2]))
        margin = min(margin, mg)
        tokens[b] = c * TREE_CHUNK + int(cols[:, g, l].reshape(32)[i])
        margins[b] = margin
    return tokens, margins
