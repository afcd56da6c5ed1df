"""CPU oracle for the ringattention hot path.  TEST INFRASTRUCTURE ONLY.

This file restates, loop for loop, the algorithm of the reference's
``ringattention/ringattention_jax.py`` with torch-CPU tensors.  It exists to
check the HIP kernels; nothing in the shipped package may import it.  Only the
tests, the smoke entry and the ``cpu_baseline`` leg of the benchmark use it.

How the oracle itself is pinned (the reference ships no tests or golden
vectors, and JAX/flax are not importable where this was written):

* forward (``blockwise_attention_fwd`` / ``ring_attention_fwd``): checked in
  float64 against ``dense_attention`` below, an independent un-chunked softmax
  whose mask is built from global positions, on sweeps of chunk sizes, ring
  sizes, causal block sizes, segment ids, biases and cache_idx values.
* backward: checked against ``torch.autograd`` of ``dense_attention`` and
  against float64 finite differences.
* ``below_or_on_diag``: exhaustive integer tables against the brute-force
  "tile holds an unmasked pair" test where they must agree, and against the
  enumerated off-by-one cases where they must not.
* ``chunk_attention_bias``: case enumeration (bias / segment / causal / all),
  the ``min(bias, 0)`` clamp and the two ``finfo.min`` constants.
* ``blockwise_feedforward``: equals the un-chunked feed-forward; SwiGLU
  backward is torch autograd.
* ``ring_attention_inference_fwd`` / ``_bwd`` (ringattention_inference.py): checked in float64
  against ``dense_attention_inference`` (an un-chunked masked softmax) and its torch autograd, over
  ring sizes, broadcast mask shapes and rows with no attended key.

* ``rope_rotate`` / ``rope_kv_append`` / ``rmsnorm_residual`` (steps either side of the path; the reference
  repository has no code for them, the formulas are the LLaMA ones): rotation checked against complex
  multiplication, norm preservation, additivity in the position and the relative-position property of the
  rotated dot product; RMSNorm against its definition in float64, unit RMS of the result, scale invariance and
  torch autograd / finite differences for the backward formula.

* attention dropout (ringattention_jax.py:119-123, :206-208, :311-321): the arithmetic given a mask
  (``finfo.min`` ADDED to the tile bias, slices taken with ``dynamic_slice`` at global offsets of a mask
  of local shape) is restated and checked against ``dense_attention`` with the same mask, against the
  exact-zero weight of dropped keys and against a hand-enumerated row whose every allowed key is dropped.
  The mask BITS are not the reference's: ``jax.random`` (threefry) is not restated; ``dropout_mask``
  draws 16 bits a position from Philox4x32-10, pinned by the known-answer vectors of the Random123 distribution.

Parity unpinned (would need the reference's own runtime): the dropout mask
bits of the ``jax.random`` stream (replaced by the documented Philox stream above) and XLA-CPU's exact
summation order / its bf16 rounding of intermediate einsum results, both far
below the stated tolerances.

Layout: q/k/v/out/grads ``(B, S, H, D)``; softmax statistics ``(B, H, S)``.
"""
import math

import numpy as np
import torch

_FINFO_MIN = {
    torch.float32: torch.finfo(torch.float32).min,    # -3.4028235e38
    torch.bfloat16: torch.finfo(torch.bfloat16).min,  # -3.3895314e38
    torch.float16: torch.finfo(torch.float16).min,    # -65504
    torch.float64: torch.finfo(torch.float64).min,
}


def finfo_min(dtype):
    return _FINFO_MIN[dtype]


def below_or_on_diag(r, r_blk_size, c, c_blk_size, causal_block_size):
    """ringattention_jax.py:324-331.  Pure integer predicate on global chunk indices."""
    cq = max(causal_block_size, r_blk_size)
    ck = max(causal_block_size, c_blk_size)
    r = r // (cq // r_blk_size)
    c = c // (ck // c_blk_size)
    return ((r + 1) * cq - 1) > (c * ck)


def _dynamic_slice_start(start, size, dim):
    # lax.dynamic_slice clamps the start so the slice stays in range.
    return max(0, min(start, dim - size))


def philox4x32_10(counter, key):
    """Philox4x32-10 of Salmon, Moraes, Dror and Shaw (SC'11), vectorised: counter (..., 4) and key (..., 2)
    uint32 arrays -> (..., 4) uint32.  Ten rounds; the key is bumped by the Weyl constants between rounds."""
    c = [np.asarray(counter[..., i], dtype=np.uint64) for i in range(4)]
    k0 = np.asarray(key[..., 0], dtype=np.uint64)
    k1 = np.asarray(key[..., 1], dtype=np.uint64)
    m32 = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0 = np.uint64(0xD2511F53) * c[0]
        p1 = np.uint64(0xCD9E8D57) * c[2]
        c = [(p1 >> np.uint64(32)) ^ c[1] ^ k0, p1 & m32, (p0 >> np.uint64(32)) ^ c[3] ^ k1, p0 & m32]
        k0 = (k0 + np.uint64(0x9E3779B9)) & m32
        k1 = (k1 + np.uint64(0xBB67AE85)) & m32
    return np.stack(c, axis=-1).astype(np.uint32)


def dropout_mask(seed, attn_pdrop, shape):
    """The boolean mask of ringattention_jax.py:120-121 / :207-208 (True = dropped, probability attn_pdrop)
    of shape (batch, heads, q_len, kv_len), from the documented Philox stream instead of jax.random:
    position e of the dense mask takes 16 bits, half-word e % 8 of block e // 8 (word (e % 8) // 2, low half
    first), keyed by the 64-bit seed; dropped iff they are below floor(float32(attn_pdrop) * 2^16)."""
    n = int(np.prod(shape))
    assert shape[-1] % 8 == 0
    blk = np.arange(n // 8, dtype=np.uint64)
    counter = np.stack([blk & np.uint64(0xFFFFFFFF), blk >> np.uint64(32), np.zeros_like(blk), np.zeros_like(blk)],
                       axis=-1)
    key = np.array([seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF], dtype=np.uint64)
    words = philox4x32_10(counter, np.broadcast_to(key, (n // 8, 2)))                 # (n / 8, 4)
    halves = np.stack([words & np.uint32(0xFFFF), words >> np.uint32(16)], axis=-1).reshape(n)
    threshold = int(float(np.float32(attn_pdrop)) * 65536.0)
    return torch.from_numpy((halves < np.uint32(threshold)).reshape(shape))


def chunk_attention_bias(query_chunk_size, key_chunk_size, bias, segment_ids,
                         causal_block_size, dtype, query_chunk_idx, key_chunk_idx,
                         work_dtype=torch.float32, attn_dropout=None):
    """ringattention_jax.py:272-322; ``attn_dropout`` is the boolean mask of :120-121 (True = dropped) or None.

    Returns the additive tile, broadcastable to (B, H, qc, kc), holding values
    representable in ``dtype`` but stored in ``work_dtype``.
    """
    query_offset = query_chunk_idx * query_chunk_size
    key_offset = key_chunk_idx * key_chunk_size
    fmin = finfo_min(dtype)
    chunk_bias = torch.zeros((1, 1, 1, 1), dtype=work_dtype)
    if bias is not None:                                                   # :278-283
        qs = min(bias.shape[-2], query_chunk_size)
        ks = min(bias.shape[-1], key_chunk_size)
        k0 = _dynamic_slice_start(key_offset, ks, bias.shape[-1])
        chunk_bias = bias[:, :, 0:qs, k0:k0 + ks].to(work_dtype)
    if segment_ids is not None:                                            # :285-299
        q0 = _dynamic_slice_start(query_offset, query_chunk_size, segment_ids.shape[1])
        k0 = _dynamic_slice_start(key_offset, key_chunk_size, segment_ids.shape[1])
        q_seg = segment_ids[:, q0:q0 + query_chunk_size]
        k_seg = segment_ids[:, k0:k0 + key_chunk_size]
        neq = ~torch.eq(q_seg[:, :, None], k_seg[:, None, :])
        seg_bias = neq[:, None].to(work_dtype) * fmin
        chunk_bias = torch.minimum(chunk_bias, seg_bias)
    if causal_block_size is not None:                                      # :301-309
        q_idx = (torch.arange(query_chunk_size).reshape(-1, 1) + query_offset) // causal_block_size
        k_idx = (torch.arange(key_chunk_size).reshape(1, -1) + key_offset) // causal_block_size
        causal = (q_idx < k_idx).to(work_dtype) * fmin
        chunk_bias = torch.minimum(chunk_bias, causal.reshape(1, 1, *causal.shape))
    if attn_dropout is not None:                                           # :311-321
        qs = min(attn_dropout.shape[-2], query_chunk_size)
        ks = min(attn_dropout.shape[-1], key_chunk_size)
        q0 = _dynamic_slice_start(query_offset, qs, attn_dropout.shape[-2])
        k0 = _dynamic_slice_start(key_offset, ks, attn_dropout.shape[-1])
        chunk_bias = chunk_bias + attn_dropout[:, :, q0:q0 + qs, k0:k0 + ks].to(work_dtype) * fmin
        # twice finfo.min overflows to -inf in ``dtype``; once plus a finite bias rounds back to finfo.min
        chunk_bias = chunk_bias.to(dtype).to(work_dtype)
    # :322  .astype(dtype): round to the kwargs dtype, then carry on in work_dtype
    if dtype in (torch.bfloat16, torch.float16):
        chunk_bias = chunk_bias.to(dtype).to(work_dtype)
    return chunk_bias


def _attn_dropout(deterministic, attn_pdrop, dropout_rng, shape):
    """:119-123 / :206-210: one mask of the LOCAL shape (batch, heads, q_len, kv_len) per call, the same in
    the forward and the backward pass; ``dropout_rng`` is the integer seed of ``dropout_mask``."""
    if deterministic or not attn_pdrop > 0.0:
        return None
    return dropout_mask(int(dropout_rng), attn_pdrop, shape)


def blockwise_attention_fwd(q, k, v, carry, q_chunk_idx_start, k_chunk_idx_start, bias, segment_ids,
                            causal_block_size, query_chunk_size, key_chunk_size, deterministic=True,
                            dropout_rng=None, attn_pdrop=0.0, dtype=torch.float32, policy=None,
                            precision=None, prevent_cse=True, cache_idx=None):
    """ringattention_jax.py:99-179.  q/k/v already in the working dtype; returns the new carry."""
    batch, q_len, num_heads, dim = q.shape
    kv_len = k.shape[1]
    num_q = q_len // query_chunk_size
    num_kv = kv_len // key_chunk_size
    wd = q.dtype
    attn_dropout = _attn_dropout(deterministic, attn_pdrop, dropout_rng, (batch, num_heads, q_len, kv_len))
    numerator, denominator, max_score = (x.clone() for x in carry)
    scale = math.sqrt(dim)                                                  # :118
    for qi in range(num_q):                                                 # :171
        qs = slice(qi * query_chunk_size, (qi + 1) * query_chunk_size)
        q_chunk = q[:, qs]
        num_c = numerator[:, qs]
        den_c = denominator[:, :, qs]
        max_c = max_score[:, :, qs]
        for ki in range(num_kv):                                            # :166-168
            if causal_block_size is not None and not below_or_on_diag(
                    q_chunk_idx_start + qi, query_chunk_size,
                    k_chunk_idx_start + ki, key_chunk_size, causal_block_size):
                continue                                                    # :158-164 identity
            ks = slice(ki * key_chunk_size, (ki + 1) * key_chunk_size)
            k_chunk, v_chunk = k[:, ks], v[:, ks].to(wd)
            w = torch.einsum('bqhd,bkhd->bhqk', q_chunk, k_chunk) / scale   # :134
            w = w + chunk_attention_bias(query_chunk_size, key_chunk_size, bias, segment_ids,
                                         causal_block_size, dtype, q_chunk_idx_start + qi,
                                         k_chunk_idx_start + ki, work_dtype=wd,
                                         attn_dropout=attn_dropout)         # :135-136
            new_max = torch.maximum(max_c, w.max(dim=-1).values)            # :138
            e = torch.exp(w - new_max[..., None])                           # :140
            ev = torch.einsum('bhqk,bkhd->bqhd', e, v_chunk)                # :141
            corr = torch.exp(max_c - new_max)                               # :142
            num_c = num_c * corr.permute(0, 2, 1)[..., None] + ev           # :143
            den_c = den_c * corr + e.sum(dim=-1)                            # :144
            max_c = new_max
        numerator[:, qs] = num_c
        denominator[:, :, qs] = den_c
        max_score[:, :, qs] = max_c
    return numerator, denominator, max_score


def blockwise_attention_bwd(q, k, v, g, carry, q_chunk_idx_start, k_chunk_idx_start, bias, segment_ids,
                            causal_block_size, query_chunk_size, key_chunk_size, deterministic=True,
                            dropout_rng=None, attn_pdrop=0.0, dtype=torch.float32, policy=None,
                            precision=None, prevent_cse=True, cache_idx=None):
    """ringattention_jax.py:181-270.  Adds this block's gradients into the incoming dq/dk/dv."""
    batch, q_len, num_heads, dim = q.shape
    kv_len = k.shape[1]
    num_q = q_len // query_chunk_size
    num_kv = kv_len // key_chunk_size
    wd = q.dtype
    attn_dropout = _attn_dropout(deterministic, attn_pdrop, dropout_rng, (batch, num_heads, q_len, kv_len))
    dq, dk, dv, output, denominator, max_score = carry
    dq, dk, dv = dq.clone(), dk.clone(), dv.clone()
    g = g.to(wd)
    scale = math.sqrt(dim)
    for qi in range(num_q):                                                 # :263
        qs = slice(qi * query_chunk_size, (qi + 1) * query_chunk_size)
        q_chunk, g_chunk = q[:, qs], g[:, qs]
        den_c, max_c = denominator[:, :, qs], max_score[:, :, qs]
        dl_part = torch.einsum('bqhd,bqhd->bhq', g_chunk, output[:, qs].to(wd))[..., None]  # :218
        dq_c = dq[:, qs]
        for ki in range(num_kv):                                            # :259-261
            if causal_block_size is not None and not below_or_on_diag(
                    q_chunk_idx_start + qi, query_chunk_size,
                    k_chunk_idx_start + ki, key_chunk_size, causal_block_size):
                continue                                                    # :246-257 zero dk/dv part
            ks = slice(ki * key_chunk_size, (ki + 1) * key_chunk_size)
            k_chunk, v_chunk = k[:, ks], v[:, ks].to(wd)
            w = torch.einsum('bqhd,bkhd->bhqk', q_chunk, k_chunk) / scale   # :223
            w = w + chunk_attention_bias(query_chunk_size, key_chunk_size, bias, segment_ids,
                                         causal_block_size, dtype, q_chunk_idx_start + qi,
                                         k_chunk_idx_start + ki, work_dtype=wd,
                                         attn_dropout=attn_dropout)         # :224-225
            p = torch.exp(w - max_c[..., None]) / den_c[..., None]          # :226
            ds = torch.einsum('bqhd,bkhd->bhqk', g_chunk, v_chunk)          # :228
            dl = (ds - dl_part) * p                                         # :229
            dq_c = dq_c + torch.einsum('bhqk,bkhd->bqhd', dl, k_chunk) / scale      # :230
            dk[:, ks] += torch.einsum('bqhd,bhqk->bkhd', q_chunk, dl) / scale       # :231,:262
            dv[:, ks] += torch.einsum('bhqk,bqhd->bkhd', p, g_chunk)                # :232,:262
        dq[:, qs] = dq_c
    return dq, dk, dv


def _work_dtype(q, float32_logits, compute_dtype):
    if compute_dtype is not None:
        return compute_dtype
    # :18-19: q and k are cast to float32 only when float32_logits is set; otherwise logits, softmax statistics and
    # the carry all live in the dtype of q (:22-23)
    return torch.float32 if (float32_logits or q.dtype == torch.float32) else q.dtype


def ring_attention_fwd(q, k, v, attn_bias, segment_ids, cache_idx, axis_size, float32_logits,
                       blockwise_kwargs, compute_dtype=None):
    """ringattention_jax.py:17-53 executed for every device of a ring of ``axis_size``.

    q/k/v are the *global* arrays (what the caller of shard_map holds); device i
    owns the i-th contiguous slice of the sequence axis.  ``attn_bias`` and
    ``segment_ids`` are replicated.  The ppermute (:47) is replaced by indexing
    the shard that would have arrived at step idx, which is (i - idx) % N (:36).
    Returns (out in v.dtype, residuals) with residuals in the working dtype.
    """
    wd = _work_dtype(q, float32_logits, compute_dtype)
    n = axis_size
    qw, kw = q.to(wd), k.to(wd)                                            # :18-19
    batch, q_total, num_heads, dim = q.shape
    kv_total = k.shape[1]
    q_len, kv_len = q_total // n, kv_total // n
    qc, kc = blockwise_kwargs["query_chunk_size"], blockwise_kwargs["key_chunk_size"]
    outs, dens, maxs = [], [], []
    for dev in range(n):
        q_d = qw[:, dev * q_len:(dev + 1) * q_len]
        num = torch.zeros((batch, q_len, num_heads, dim), dtype=wd)         # :22
        den = torch.zeros((batch, num_heads, q_len), dtype=wd)              # :23
        mx = torch.full((batch, num_heads, q_len), -math.inf, dtype=wd)     # :49
        for idx in range(n):                                                # :50-51
            if cache_idx is None:
                q_start = dev * (q_len // qc)                               # :32-33
            else:
                q_start = cache_idx // qc                                   # :35
            k_blk = (dev - idx) % n                                         # :36
            k_start = k_blk * (kv_len // kc)                                # :37
            ksl = slice(k_blk * kv_len, (k_blk + 1) * kv_len)
            num, den, mx = blockwise_attention_fwd(
                q_d, kw[:, ksl], v[:, ksl], (num, den, mx), q_start, k_start,
                bias=attn_bias, segment_ids=segment_ids, cache_idx=cache_idx, **blockwise_kwargs)
        outs.append(num / den.permute(0, 2, 1)[..., None])                  # :52
        dens.append(den)
        maxs.append(mx)
    output = torch.cat(outs, dim=1)
    denominator = torch.cat(dens, dim=2)
    max_score = torch.cat(maxs, dim=2)
    res = (output, qw, kw, v, attn_bias, segment_ids, cache_idx, denominator, max_score)
    return output.to(v.dtype), res


def ring_attention_bwd(axis_size, float32_logits, blockwise_kwargs, res, g):
    """ringattention_jax.py:55-90 for every device of the ring; returns global dq, dk, dv."""
    output, q, k, v, attn_bias, segment_ids, cache_idx, denominator, max_score = res
    wd = q.dtype
    n = axis_size
    batch, q_total, num_heads, dim = q.shape
    kv_total = k.shape[1]
    q_len, kv_len = q_total // n, kv_total // n
    qc, kc = blockwise_kwargs["query_chunk_size"], blockwise_kwargs["key_chunk_size"]
    dq = torch.zeros_like(q)                                               # :61
    dk = torch.zeros_like(k)                                               # :62
    dv = torch.zeros(v.shape, dtype=wd)                                    # :63
    for dev in range(n):
        qsl = slice(dev * q_len, (dev + 1) * q_len)
        for idx in range(n):                                                # :88
            q_start = dev * (q_len // qc) if cache_idx is None else cache_idx // qc   # :69-73
            k_blk = (dev - idx) % n                                         # :74
            k_start = k_blk * (kv_len // kc)                                # :75
            ksl = slice(k_blk * kv_len, (k_blk + 1) * kv_len)
            # dk/dv partials travel with their K/V shard (:85-86): accumulate at the shard's home.
            dq_d, dk_s, dv_s = blockwise_attention_bwd(
                q[:, qsl], k[:, ksl], v[:, ksl], g[:, qsl],
                (dq[:, qsl], dk[:, ksl], dv[:, ksl], output[:, qsl], denominator[:, :, qsl],
                 max_score[:, :, qsl]),
                q_start, k_start, bias=attn_bias, segment_ids=segment_ids, cache_idx=cache_idx,
                **blockwise_kwargs)
            dq[:, qsl], dk[:, ksl], dv[:, ksl] = dq_d, dk_s, dv_s
    return dq, dk, dv


def ring_attention(q, k, v, attn_bias, segment_ids, cache_idx, axis_size, float32_logits,
                   blockwise_kwargs, compute_dtype=None):
    """Forward value only (ringattention_jax.py:92-95)."""
    return ring_attention_fwd(q, k, v, attn_bias, segment_ids, cache_idx, axis_size, float32_logits,
                              blockwise_kwargs, compute_dtype)[0]


def dense_attention(q, k, v, attn_bias, segment_ids, cache_idx, axis_size, blockwise_kwargs,
                    compute_dtype=torch.float64):
    """Independent closed form: softmax(Q K^T / sqrt(D) + B_eff) V on the global arrays.

    B_eff is built from global positions, not chunk by chunk: pairs in tiles the
    skip predicate drops are -inf; pairs masked by segment/causal inside a tile
    that runs are finfo(dtype).min; the rest get the bias, clamped to <= 0
    whenever a mask feature is on (the minimum() of ringattention_jax.py:299,309).
    Differentiable with torch.autograd.
    """
    wd = compute_dtype
    qc, kc = blockwise_kwargs["query_chunk_size"], blockwise_kwargs["key_chunk_size"]
    cbs = blockwise_kwargs["causal_block_size"]
    dtype = blockwise_kwargs.get("dtype", torch.float32)
    fmin = finfo_min(dtype)
    batch, q_total, num_heads, dim = q.shape
    kv_total = k.shape[1]
    n = axis_size
    q_len = q_total // n
    # global positions of every local query row / key column
    loc_q = torch.arange(q_total) % q_len
    dev_q = torch.arange(q_total) // q_len
    if cache_idx is None:
        q_chunk = dev_q * (q_len // qc) + loc_q // qc
    else:
        q_chunk = cache_idx // qc + loc_q // qc
    g_q = q_chunk * qc + loc_q % qc
    g_k = torch.arange(kv_total)
    k_chunk = g_k // kc
    logits = torch.einsum('bqhd,bkhd->bhqk', q.to(wd), k.to(wd)) / math.sqrt(dim)
    any_mask = (segment_ids is not None) or (cbs is not None)
    add = torch.zeros((1, 1, 1, 1), dtype=wd)
    if attn_bias is not None:
        b = attn_bias.to(wd)
        if b.shape[-2] != 1:
            # the reference always slices query rows 0:qc of the bias (:281)
            b = b[:, :, (loc_q % qc), :]
        if b.shape[-1] == 1:
            b = b.expand(*b.shape[:3], kv_total)
        add = b
        if any_mask:
            add = torch.clamp(add, max=0.0)
    add = add.expand(-1, -1, q_total if add.shape[2] != 1 else 1, kv_total if add.shape[3] != 1 else 1)
    if dtype in (torch.bfloat16, torch.float16):
        add = add.to(dtype).to(wd)
    masked = torch.zeros((1, 1, q_total, kv_total), dtype=torch.bool)
    if segment_ids is not None:
        masked = masked | (segment_ids[:, g_q][:, None, :, None] != segment_ids[:, g_k][:, None, None, :])
    if cbs is not None:
        masked = masked | ((g_q // cbs)[:, None] < (g_k // cbs)[None, :])[None, None]
    logits = logits + add
    logits = torch.where(masked, torch.full((), fmin, dtype=wd), logits)
    if (not blockwise_kwargs.get("deterministic", True)) and blockwise_kwargs.get("attn_pdrop", 0.0) > 0.0:
        # the mask has the LOCAL shape and is sliced at GLOBAL chunk offsets, clamped (:312-320)
        kv_len = kv_total // n
        drop = dropout_mask(int(blockwise_kwargs["dropout_rng"]), blockwise_kwargs["attn_pdrop"],
                            (batch, num_heads, q_len, kv_len))
        row = torch.clamp(q_chunk * qc, max=q_len - qc) + loc_q % qc
        col = torch.clamp(k_chunk * kc, max=kv_len - kc) + g_k % kc
        dropped = drop[:, :, row][:, :, :, col]
        # finfo.min is added: once -> finfo.min (logit and bias are absorbed), twice -> -inf
        logits = torch.where(dropped, torch.where(masked, torch.full((), -math.inf, dtype=wd),
                                                  torch.full((), fmin, dtype=wd)), logits)
    if cbs is not None:
        cq, ck = max(cbs, qc), max(cbs, kc)
        r = q_chunk // (cq // qc)
        c = k_chunk // (ck // kc)
        run = ((r[:, None] + 1) * cq - 1) > (c[None, :] * ck)
        logits = torch.where(run[None, None], logits, torch.full((), -math.inf, dtype=wd))
    p = torch.softmax(logits, dim=-1)      # all -inf rows -> NaN, as 0/0 in the reference (:52)
    return torch.einsum('bhqk,bkhd->bqhd', p, v.to(wd))


# --------------------------------------------------------------------------- mask-based inference ring
def _mask_rows(attn_mask, dev, q_len, q_total):
    """The device's view of the global boolean mask (B|1, H|1, Q_total|1, K_total): its own query rows
    when the mask has a query axis (the mask is sharded like q), the broadcast row otherwise."""
    if attn_mask.shape[2] == 1:
        return attn_mask
    assert attn_mask.shape[2] == q_total
    return attn_mask[:, :, dev * q_len:(dev + 1) * q_len]


def ring_attention_inference_fwd(q, k, v, attn_mask, axis_size, float32_logits=True, compute_dtype=None):
    """ringattention_inference.py:8-36 for every device of a ring of ``axis_size`` (global arrays, as in
    ring_attention_fwd above): un-chunked online softmax per ring step, boolean mask sliced along its key
    axis at the block that would have arrived at that step (:19-20), masked logits set to finfo.min of the
    logits' dtype (:22)."""
    wd = compute_dtype or (torch.float32 if (float32_logits or q.dtype == torch.float32) else q.dtype)
    n = axis_size
    qw, kw = q.to(wd), k.to(wd)                                            # :9-10
    batch, q_total, num_heads, dim = q.shape
    kv_total = k.shape[1]
    q_len, kv_len = q_total // n, kv_total // n
    scale = math.sqrt(dim)                                                  # :16
    neg = finfo_min(wd)
    outs, nums, dens, maxs = [], [], [], []
    for dev in range(n):
        q_d = qw[:, dev * q_len:(dev + 1) * q_len]
        m_d = _mask_rows(attn_mask, dev, q_len, q_total)
        num = torch.zeros((batch, q_len, num_heads, dim), dtype=wd)         # :13
        den = torch.zeros((batch, num_heads, q_len), dtype=wd)              # :14
        prev = torch.full((batch, num_heads, q_len), -math.inf, dtype=wd)   # :31
        for idx in range(n):                                                # :32-33
            k_blk = (dev - idx) % n                                         # :20
            ksl = slice(k_blk * kv_len, (k_blk + 1) * kv_len)
            mask = m_d[..., ksl]                                            # :19-20
            w = torch.einsum("bqhd,bkhd->bhqk", q_d, kw[:, ksl]) / scale    # :21
            w = torch.where(mask, w, torch.full_like(w, neg))               # :22
            mx = torch.maximum(prev, w.max(dim=-1).values)                  # :23
            e = torch.exp(w - mx[..., None])                                # :24
            corr = torch.exp(prev - mx)                                     # :25
            num = num * corr.permute(0, 2, 1)[..., None] + torch.einsum("bhqk,bkhd->bqhd", e, v[:, ksl].to(wd))   # :26
            den = den * corr + e.sum(dim=-1)                                # :27
            prev = mx
        outs.append(num / den.permute(0, 2, 1)[..., None])                  # :34
        nums.append(num); dens.append(den); maxs.append(prev)
    output = torch.cat(outs, dim=1)
    res = (output, qw, kw, v, attn_mask, torch.cat(nums, dim=1), torch.cat(dens, dim=2), torch.cat(maxs, dim=2))
    return output.to(v.dtype), res                                          # :35


def ring_attention_inference_bwd(axis_size, res, g):
    """ringattention_inference.py:38-64 for every device of the ring; returns global fp32 dq, dk, dv cast to
    the residual dtypes (:62)."""
    output, q, k, v, attn_mask, _num, denominator, max_score = res
    n = axis_size
    batch, q_total, num_heads, dim = q.shape
    kv_total = k.shape[1]
    q_len, kv_len = q_total // n, kv_total // n
    scale = math.sqrt(dim)                                                  # :46
    neg = finfo_min(q.dtype)
    acc = torch.float64 if q.dtype == torch.float64 else torch.float32   # fp32 in the reference
    dq = torch.zeros(q.shape, dtype=acc)                                    # :42
    dk = torch.zeros(k.shape, dtype=acc)                                    # :43
    dv = torch.zeros(v.shape, dtype=acc)                                    # :44
    gf = g.to(acc)
    for dev in range(n):
        qsl = slice(dev * q_len, (dev + 1) * q_len)
        m_d = _mask_rows(attn_mask, dev, q_len, q_total)
        for idx in range(n):
            k_blk = (dev - idx) % n                                         # :50
            ksl = slice(k_blk * kv_len, (k_blk + 1) * kv_len)
            mask = m_d[..., ksl]
            w = torch.einsum("bqhd,bkhd->bhqk", q[:, qsl], k[:, ksl]) / scale              # :51
            w = torch.where(mask, w, torch.full_like(w, neg))                              # :52
            p = torch.exp(w - max_score[:, :, qsl, None]) / denominator[:, :, qsl, None]   # :53
            ds = torch.einsum("bqhd,bkhd->bhqk", gf[:, qsl], v[:, ksl].to(acc))  # :54
            dl = (ds - torch.einsum("bqhd,bqhd->bhq", gf[:, qsl], output[:, qsl].to(acc))[..., None]) * p   # :55
            dq[:, qsl] += torch.einsum("bhqk,bkhd->bqhd", dl, k[:, ksl].to(acc)) / scale   # :56
            dk[:, ksl] += torch.einsum("bqhd,bhqk->bkhd", q[:, qsl].to(acc), dl) / scale   # :57
            dv[:, ksl] += torch.einsum("bhqk,bqhd->bkhd", p.to(acc), gf[:, qsl])           # :58
    return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype)                   # :62


def dense_attention_inference(q, k, v, attn_mask, dtype=torch.float64):
    """Independent closed form for ring_attention_inference: softmax over all keys of
    where(mask, Q K^T / sqrt(D), -inf) times V.  A row with no attended key is the mean of V over all keys:
    the reference's finfo.min logits are all equal there and softmax of a constant is uniform."""
    qd, kd, vd = q.to(dtype), k.to(dtype), v.to(dtype)
    w = torch.einsum("bqhd,bkhd->bhqk", qd, kd) / math.sqrt(q.shape[-1])
    mask = attn_mask.expand(w.shape[0], w.shape[1], w.shape[2], w.shape[3])
    none = ~mask.any(dim=-1, keepdim=True)
    w = torch.where(mask | none, w, torch.full_like(w, -math.inf))
    w = torch.where(none, torch.zeros_like(w), w)
    p = torch.softmax(w, dim=-1)
    return torch.einsum("bhqk,bkhd->bqhd", p, vd)


def swiglu(x, w1, w2, w3):
    """The caller-side SwiGLU MLP the reference's blockwise_feedforward is used with:
    w2( silu(x w1) * (x w3) ), weights stored (in, out)."""
    a = x @ w1
    b = x @ w3
    return (torch.nn.functional.silu(a) * b) @ w2


def blockwise_feedforward(feedforward, inputs, chunk_size, static_argnums=(1,), policy=None, pre_remat=True):
    """ringattention_jax.py:333-352.  'b (c n) d -> b c n d' with c=chunk_size, scanned over n:
    each step feeds chunk_size tokens {ci*n + j : ci} to ``feedforward``."""
    b, s, d = inputs.shape
    n = s // chunk_size
    x = inputs.reshape(b, chunk_size, n, d)                                 # :339
    outs = [feedforward(x[:, :, j, :]) for j in range(n)]                   # :340-350
    out = torch.stack(outs, dim=2)
    return out.reshape(b, s, out.shape[-1])                                 # :351


# ----------------------------------------------------------------------------- steps either side of the path

def rope_rotate(x, pos, theta=10000.0, style="adjacent"):
    """Rotary position embedding of x (..., D) at integer position ``pos``: the pair (x0, x1) of frequency index
    j = 0 .. D/2-1 turns by the angle pos * theta^(-2j/D).  ``style`` "adjacent" pairs elements (2j, 2j+1),
    "half" pairs (j, j + D/2).  Angles in float64; the result has x's dtype."""
    D = x.shape[-1]
    j = torch.arange(D // 2, dtype=torch.float64)
    ang = float(pos) * torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * j / D)
    cs, sn = torch.cos(ang).to(x.dtype), torch.sin(ang).to(x.dtype)
    if style == "adjacent":
        x0, x1 = x[..., 0::2], x[..., 1::2]
    else:
        x0, x1 = x[..., : D // 2], x[..., D // 2:]
    y0, y1 = x0 * cs - x1 * sn, x0 * sn + x1 * cs
    if style == "adjacent":
        return torch.stack((y0, y1), dim=-1).reshape(x.shape)
    return torch.cat((y0, y1), dim=-1)


def rope_kv_append(q, k_new, v_new, k_cache, v_cache, cache_idx, theta=10000.0, style="adjacent"):
    """The decode step's prologue: returns (q rotated, k_cache, v_cache) with the rotated new key and the new value
    written at position cache_idx of copies of the caches.  theta None or 0: no rotation."""
    rot = (lambda t: rope_rotate(t, cache_idx, theta, style)) if theta else (lambda t: t)
    kc, vc = k_cache.clone(), v_cache.clone()
    kc[:, cache_idx] = rot(k_new)[:, 0]
    vc[:, cache_idx] = v_new[:, 0]
    return rot(q), kc, vc


def rmsnorm_residual(x, residual, weight, eps=1e-6, stream_dtype=None):
    """y = x + residual (residual may be None); normed = y / sqrt(mean(y^2) + eps) * weight.  ``stream_dtype`` rounds
    y to the dtype the residual stream is stored in before the norm is taken of it (what a bf16 model does)."""
    y = x if residual is None else x + residual
    if stream_dtype is not None:
        y = y.to(stream_dtype).to(x.dtype)
    rstd = torch.rsqrt((y * y).mean(dim=-1, keepdim=True) + eps)
    return y, y * rstd * weight
