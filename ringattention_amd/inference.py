"""ring_attention_inference (ringattention/ringattention_inference.py:8-73): the ring with a boolean
attention mask and no chunking inside a ring step.  bf16 / fp32 / fp16 inputs with head sizes up to 128 run on
the MFMA kernels, which read the mask in a packed form (ra_keep_pack): shard lengths that are no multiple of 128
are padded to one (_pad_lengths) unless some row of the mask attends to nothing; that case and head sizes
above 128 run on the fp32 vector-ALU kernels."""
import torch

from . import _lib as L
from .ringattention_hip import (_Config, _MaskInputs, _blockwise_attention_bwd, _blockwise_attention_fwd, _bwd_delta,
                                _check_qkv, _row_dense, _save_residuals, _saved_residuals, axis_size)


def _inference_cfg(q, q_len, kv_len, float32_logits, logit_dim=0):
    # one "chunk" per ring step (:21 is a single einsum over the shard); finfo.min of the logits' dtype (:22)
    logits_dtype = torch.float32 if (float32_logits or q.dtype == torch.float32) else q.dtype
    cfg = _Config(dict(causal_block_size=None, query_chunk_size=q_len, key_chunk_size=kv_len, deterministic=True,
                       attn_pdrop=0.0, dtype=logits_dtype, impl="auto", skip_masked_tiles=False))
    cfg.logit_dim = logit_dim       # q, k, v zero-padded along D: the head size that scales the logits (:18)
    return cfg


def _fwd(q, k, v, attn_mask, axis_name, float32_logits, logit_dim=0):
    _check_qkv(q, k, v)
    q = q.contiguous()                             # the cotangent arrives dense and shares q's strides
    k, v = (t if _row_dense(t) else t.contiguous() for t in (k, v))            # other views are copied once
    if k.stride(0) != v.stride(0):
        k, v = k.contiguous(), v.contiguous()
    n = axis_size(axis_name)                                                     # :15
    B, q_total, H, D = q.shape
    kv_total = k.shape[1]
    if q_total % n or kv_total % n:
        raise ValueError("sequence lengths must divide by the ring size %d" % n)
    q_len, kv_len = q_total // n, kv_total // n
    if attn_mask.dim() != 4 or attn_mask.shape[3] != kv_total or attn_mask.shape[2] not in (1, q_total) or \
            attn_mask.shape[0] not in (1, B) or attn_mask.shape[1] not in (1, H):
        raise ValueError("attn_mask must be (B|1, H|1, Q|1, K) with Q = %d and K = %d" % (q_total, kv_total))
    cfg = _inference_cfg(q, q_len, kv_len, float32_logits, logit_dim)
    mi = _MaskInputs(cfg, None, None, None, B, q.device, kv_total)
    mi.set_keep(attn_mask, q.device, q_total, kv_total)
    if q_len % 64 or kv_len % 64:
        mi.keep_packed = None                        # shards not aligned to the 64 x 64 packing: generic kernels
    # tiles without a kept pair may be skipped unless some row attends to nothing at all (its logits stay
    # equal at finfo.min and its weights uniform, ringattention_inference.py:22-24)
    cfg.skip_masked_tiles = not mi.keep_has_empty_row
    # the numerator (:13) lives between the steps of a device only: the first step starts it, the last one writes
    # out = numerator / denominator (:34) instead
    num = torch.empty((B, q_total, H, D), dtype=torch.float32, device=q.device) if n > 1 else None
    den = torch.empty((B, H, q_total), dtype=torch.float32, device=q.device)      # :14
    mx = torch.empty((B, H, q_total), dtype=torch.float32, device=q.device)       # :31
    out = torch.empty((B, q_total, H, D), dtype=v.dtype, device=q.device)
    # the residual `output` of :35 is the quotient before it is rounded to v's dtype (it meets the cotangent at :55)
    out32 = None
    if out.dtype != torch.float32:
        out32 = torch.empty((B, q_total, H, D), dtype=torch.float32, device=q.device)
    for dev in range(n):
        qs = slice(dev * q_len, (dev + 1) * q_len)
        mi.keep_row0 = dev * q_len                  # the device's rows of a mask that is sharded like q
        carry = (num[:, qs] if num is not None else None, den[:, :, qs], mx[:, :, qs])
        for idx in range(n):                                                      # :32-33
            k_blk = (dev - idx) % n                                               # :20
            ks = slice(k_blk * kv_len, (k_blk + 1) * kv_len)
            _blockwise_attention_fwd(q[:, qs], k[:, ks], v[:, ks], carry, dev, k_blk, None, None,
                                     None, q_len, kv_len, _mask_inputs=mi, _cfg=cfg, _carry_is_initial=(idx == 0),
                                     _out=out[:, qs] if idx == n - 1 else None,
                                     _out_f32=out32[:, qs] if out32 is not None and idx == n - 1 else None)
    return out, (out if out32 is None else out32, q, k, v, mi, cfg, n, den, mx)


def _bwd(res, g):
    out, q, k, v, mi, cfg, n, den, mx = res
    B, q_total, H, D = q.shape
    kv_total = k.shape[1]
    q_len, kv_len = q_total // n, kv_total // n
    g = g.to(q.dtype).contiguous()
    delta = _bwd_delta(g, out)                                                    # :55
    # fp32 accumulators (:42-44) between the calls that add into a gradient only: every device adds into its dq
    # n times (first idx 0, last idx n - 1) and into every K/V shard once (first device 0, last device n - 1)
    mk = lambda t: torch.empty(t.shape, dtype=torch.float32, device=q.device) if n > 1 else None
    dq, dk, dv = mk(q), mk(k), mk(v)
    dq_out, dk_out, dv_out = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    part = lambda t, sl: t[:, sl] if t is not None else None
    for dev in range(n):
        qs = slice(dev * q_len, (dev + 1) * q_len)
        mi.keep_row0 = dev * q_len
        for idx in range(n):
            k_blk = (dev - idx) % n                                               # :50
            ks = slice(k_blk * kv_len, (k_blk + 1) * kv_len)
            initial = (L.RA_GRAD_INIT_DQ if idx == 0 else 0) | (L.RA_GRAD_INIT_DKV if dev == 0 else 0)
            _blockwise_attention_bwd(q[:, qs], k[:, ks], v[:, ks], g[:, qs],
                                     (part(dq, qs), part(dk, ks), part(dv, ks), out[:, qs], den[:, :, qs],
                                      mx[:, :, qs]),
                                     dev, k_blk, None, None, None, q_len, kv_len,
                                     _mask_inputs=mi, _cfg=cfg, _delta=delta[:, :, qs], _grads_initial=initial,
                                     _dq_out=dq_out[:, qs] if idx == n - 1 else None,
                                     _dkv_out=(dk_out[:, ks], dv_out[:, ks]) if dev == n - 1 else None)
    return dq_out, dk_out, dv_out                                                 # :62


class _RingAttentionInferenceFn(torch.autograd.Function):
    """custom_vjp of ringattention_inference.py:67-73: cotangents for q, k, v; None for the mask (:64)."""

    @staticmethod
    def forward(ctx, q, k, v, attn_mask, axis_name, float32_logits, logit_dim=0):
        out, res = _fwd(q, k, v, attn_mask, axis_name, float32_logits, logit_dim)
        _save_residuals(ctx, res)
        return out

    @staticmethod
    def backward(ctx, g):
        dq, dk, dv = _bwd(_saved_residuals(ctx), g)
        return dq, dk, dv, None, None, None, None


def _pad_lengths(q, k, v, attn_mask, axis_name, float32_logits, n, grid=128):
    """Lengths whose shards are no multiple of 128 (a prompt of 1000 tokens): the matrix-core kernels tile 128
    positions and read the mask packed in words of 64, so such a call would take the vector kernels.  The mask says
    who attends to whom and positions mean nothing else here, so q, k, v and the mask are padded at the end to the
    next multiple of 128 per device and the result is cut back: the new keys are attended to by no real row, the new
    rows - whose output is dropped and which get no cotangent - attend to the new keys (or to key 0 when only rows
    were added), so no row is left without a key.  A real row that attends to nothing averages over all keys
    (ringattention_inference.py:22-24), padded ones included: a mask with such a row is left as it is.  Returns the
    result, or None."""
    B, Q, H, D = q.shape
    K = k.shape[1]
    step = grid * n
    if (Q % step == 0 and K % step == 0) or q.dtype not in (torch.bfloat16, torch.float32) or D > 128:
        return None
    if attn_mask.dim() != 4 or attn_mask.shape[3] != K or attn_mask.shape[2] not in (1, Q):
        return None                    # refused further down, with the message for it
    m = attn_mask if attn_mask.dtype == torch.bool else attn_mask != 0
    if not bool(m.any(dim=-1).all()):
        return None
    pq, pk = -Q % step, -K % step
    rows = m.shape[2] > 1
    mp = torch.nn.functional.pad(m, (0, pk, 0, pq if rows else 0), value=False)
    if rows and pq:
        if pk:
            mp[:, :, Q:, K:] = True
        else:
            mp[:, :, Q:, 0] = True
    qp = torch.nn.functional.pad(q, (0, 0, 0, 0, 0, pq))
    kp, vp = (torch.nn.functional.pad(t, (0, 0, 0, 0, 0, pk)) for t in (k, v))
    return ring_attention_inference(qp, kp, vp, mp, axis_name, float32_logits)[:, :Q].contiguous()


def ring_attention_inference(q, k, v, attn_mask, axis_name, float32_logits=True):
    """ringattention_inference.py:67-70.  q, k, v are the global (B, S, H, D) arrays of the virtual ring
    declared with ``ring_axis``; attn_mask is the global boolean mask (B|1, H|1, Q|1, K), True = attend.
    bf16, fp32 or fp16 (computed on fp32 copies, as ring_attention does); a head size no kernel tiles (they take 64
    and 128 on the matrix cores, 32, 64, 128 and 256 otherwise) is zero-padded to the next one that is, with the
    logits still divided by the square root of the original head size."""
    if q.dtype == torch.float16 and k.dtype == torch.float16 and v.dtype == torch.float16:
        return ring_attention_inference(q.float(), k.float(), v.float(), attn_mask, axis_name,
                                        float32_logits).to(torch.float16)
    if q.numel() == 0 or k.numel() == 0:          # nothing to launch (as in ring_attention)
        _check_qkv(q, k, v)
        fill = float("nan") if q.numel() else 0.0
        return torch.full_like(q, fill) + 0.0 * (q.sum() + k.sum() + v.sum()).to(q.dtype)
    D = q.shape[-1]
    if D > 256:
        raise NotImplementedError("head size %d: the kernels take head sizes up to 256" % D)
    n = axis_size(axis_name)
    padded = _pad_lengths(q, k, v, attn_mask, axis_name, float32_logits, n)
    if padded is not None:
        return padded
    on_grid = q.shape[1] % (64 * n) == 0 and k.shape[1] % (64 * n) == 0 and D <= 128
    if on_grid:
        to = 64 if D <= 64 else 128
    elif q.dtype == torch.bfloat16:
        to = 128 if D <= 128 else 256           # the matrix-core kernels that evaluate the mask element by element
    else:
        to = next(s for s in (32, 64, 128, 256) if D <= s)
    if to == D:
        return _RingAttentionInferenceFn.apply(q, k, v, attn_mask, axis_name, float32_logits)
    q, k, v = (torch.nn.functional.pad(t, (0, to - D)) for t in (q, k, v))
    return _RingAttentionInferenceFn.apply(q, k, v, attn_mask, axis_name, float32_logits, D)[..., :D].contiguous()
