"""Decode through cache_idx (ringattention_jax.py:31-35 with one query token): host wrapper of the
streaming kernels ra_decode_fwd / ra_decode_fwd_static."""
import ctypes

import torch

from . import _lib as L
from .ringattention_hip import _Config, _MaskInputs, _check_qkv, _ra_dtype, _rows, _stream


def decode_workspace(q, k, num_splits=0):
    """A workspace for ``decode_attention(..., workspace=...)``: what ra_decode_workspace_bytes asks for the
    shapes of q (B,1,H,D) and the cache k (B,L,H,D).  A caller that captures decode steps into a HIP graph, or
    that decodes on several streams, owns one such buffer per graph / stream and keeps it alive as long as
    the graph may replay."""
    B, _, H, D = q.shape
    lib = L.load()
    if num_splits == 0:         # what the automatic choice needs, not the 256-split upper bound
        num_splits = lib.ra_decode_auto_splits(B, k.shape[1], H, D, _ra_dtype(q))
    nbytes = lib.ra_decode_workspace_bytes(B, k.shape[1], H, D, num_splits)
    return torch.empty(nbytes, dtype=torch.uint8, device=q.device)


def decode_attention(q, k, v, attn_bias, segment_ids, cache_idx, blockwise_kwargs, out=None, num_splits=0,
                     workspace=None, static_scratch=False, carry=None, carry_is_initial=False, k_chunk_idx_start=0,
                     write_out=True, _mask_inputs=None):
    """q (B,1,H,D) against the cache buffers k, v (B,L,H,D); cache_idx is a Python int or a device
    int32 scalar (read by the kernel, so the call can sit in a captured graph or a tight loop).
    blockwise_kwargs must carry query_chunk_size == 1, as q_len // query_chunk_size demands.

    The split-KV partials go to ``workspace`` (see decode_workspace) when one is given; otherwise to a buffer
    allocated for this call from torch's stream-aware caching allocator, which is safe for eager calls on any
    stream but must not be captured into a graph (the graph would keep writing to a block torch hands out again).
    ``static_scratch=True`` takes ra_decode_fwd_static instead: no allocation at all, the partials go to the
    library's built-in 16 MiB buffer of the GPU; calls that overlap in time on one GPU must not use it (make one
    eager call per GPU before capturing it into a graph: the first call looks the buffer's address up).

    ``carry = (numerator (B,1,H,D), denominator (B,H,1), max_score (B,H,1))``, fp32, makes the call one step of a
    ring whose cache is sharded over the sequence axis (:31-37 with an axis size above one): k, v are the shard that
    has arrived, ``k_chunk_idx_start`` its first key chunk (:37); the carry is updated in place and ``out`` is only
    written when ``write_out`` (the device's last step, :52)."""
    cfg = _Config(blockwise_kwargs)
    if cfg.pdrop > 0.0:
        raise NotImplementedError("attention dropout together with cache_idx is not supported")
    _check_qkv(q, k, v)
    B, Sq, H, D = q.shape
    if Sq != 1:
        raise ValueError("decode_attention takes one query token per batch row")
    if cfg.qc != 1:
        raise ValueError("query_chunk_size must be 1 when q_len is 1")
    L_buf = k.shape[1]
    if L_buf % cfg.kc:
        raise ValueError("cache length %d must divide by key_chunk_size %d" % (L_buf, cfg.kc))
    mi = _mask_inputs or _MaskInputs(cfg, attn_bias, segment_ids, cache_idx, B, q.device,
                                     k_chunk_idx_start * cfg.kc + L_buf, q.shape[2])
    if out is None and (write_out or carry is None):
        out = torch.empty_like(q)
    lib = L.load()
    p = L.RaDecodeParams()
    p.q, p.k, p.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    if carry is not None:
        num, den, mx = carry
        if not (num.dtype == den.dtype == mx.dtype == torch.float32) or num.shape != q.shape \
                or den.shape != (B, H, 1) or mx.shape != (B, H, 1) or den.stride() != mx.stride() \
                or den.stride(1) != 1:
            raise ValueError("carry: fp32 numerator (B,1,H,D), denominator and max_score (B,H,1) with equal strides")
        p.carry_numerator, p.carry_denominator, p.carry_max_score = num.data_ptr(), den.data_ptr(), mx.data_ptr()
        p.carry_num_stride_b, p.carry_stat_stride_b = _rows(num)[0], den.stride(0)
        p.carry_is_initial = 1 if carry_is_initial else 0
        if not write_out:
            out = None
    if out is not None:
        p.out = out.data_ptr()
    p.dtype = _ra_dtype(q)
    p.B, p.L, p.H, p.D = B, L_buf, H, D
    p.q_stride_b = _rows(q)[0]
    p.kv_stride_b, p.kv_stride_s = _rows(k)
    if _rows(v) != _rows(k):
        raise ValueError("k and v caches must share strides")
    if out is not None:
        p.out_stride_b = _rows(out)[0]
    q_start = mi.cache_idx_host if mi.cache_idx_host is not None else 0
    p.mask = mi.fill(cfg, q_start, k_chunk_idx_start, False)
    p.num_splits = num_splits
    if static_scratch:
        if workspace is not None:
            raise ValueError("static_scratch and workspace exclude each other")
        L.check(lib.ra_decode_fwd_static(ctypes.byref(p), _stream()), "ra_decode_fwd_static")
        return out
    if workspace is None:
        workspace = decode_workspace(q, k, num_splits)
    elif workspace.device != q.device or workspace.dtype != torch.uint8 or not workspace.is_contiguous():
        raise ValueError("workspace must be a contiguous uint8 tensor on the device of q")
    p.workspace, p.workspace_bytes = workspace.data_ptr(), workspace.numel()
    L.check(lib.ra_decode_fwd(ctypes.byref(p), _stream()), "ra_decode_fwd")
    return out


def decode_attention_ring(q, k, v, attn_bias, segment_ids, cache_idx, blockwise_kwargs, n):
    """cache_idx with a ring of n virtual devices (ringattention_jax.py:29-51 with :34-35): q (B,n,H,D) holds one
    query token per device, all at position cache_idx; the cache buffers k, v (B,L,H,D) are sharded over the
    sequence axis, device d holding positions [d L/n, (d+1) L/n).  In scan step idx device d streams the shard
    (d - idx) mod n (:36) with the split kernel and merges the result into its carry; the last step writes
    out = numerator / denominator (:52).  Returns out (B,n,H,D)."""
    cfg = _Config(blockwise_kwargs)
    _check_qkv(q, k, v)
    B, n_q, H, D = q.shape
    if n_q != n:
        raise ValueError("one query token per virtual device: q must be (B, %d, H, D)" % n)
    L_buf = k.shape[1]
    if L_buf % n or (L_buf // n) % cfg.kc:
        raise ValueError("cache length %d must divide into %d shards of whole key chunks (%d)" % (L_buf, n, cfg.kc))
    kv_len = L_buf // n
    mi = _MaskInputs(cfg, attn_bias, segment_ids, cache_idx, B, q.device, L_buf, H)
    out = torch.empty_like(q)
    num = torch.empty((B, n, H, D), dtype=torch.float32, device=q.device)
    den = torch.empty((B, n, H, 1), dtype=torch.float32, device=q.device)
    mx = torch.empty((B, n, H, 1), dtype=torch.float32, device=q.device)
    ws = decode_workspace(q[:, :1], k[:, :kv_len])
    for idx in range(n):                    # the scan of :29-51; the devices of a step one after the other
        for dev in range(n):
            shard = (dev - idx) % n
            ks = slice(shard * kv_len, (shard + 1) * kv_len)
            decode_attention(q[:, dev:dev + 1], k[:, ks], v[:, ks], None, None, cache_idx, blockwise_kwargs,
                             out=out[:, dev:dev + 1], workspace=ws,
                             carry=(num[:, dev:dev + 1], den[:, dev], mx[:, dev]), carry_is_initial=idx == 0,
                             k_chunk_idx_start=shard * (kv_len // cfg.kc), write_out=idx == n - 1, _mask_inputs=mi)
    return out
