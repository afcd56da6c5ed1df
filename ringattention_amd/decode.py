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
    nbytes = L.load().ra_decode_workspace_bytes(B, k.shape[1], H, D, num_splits)
    return torch.empty(nbytes, dtype=torch.uint8, device=q.device)


def decode_attention(q, k, v, attn_bias, segment_ids, cache_idx, blockwise_kwargs, out=None, num_splits=0,
                     workspace=None, static_scratch=False):
    """q (B,1,H,D) against the cache buffers k, v (B,L,H,D); cache_idx is a Python int or a device
    int32 scalar (read by the kernel, so the call can sit in a captured graph or a tight loop).
    blockwise_kwargs must carry query_chunk_size == 1, as q_len // query_chunk_size demands.

    The split-KV partials go to ``workspace`` (see decode_workspace) when one is given; otherwise to a buffer
    allocated for this call from torch's stream-aware caching allocator, which is safe for eager calls on any
    stream but must not be captured into a graph (the graph would keep writing to a block torch hands out again).
    ``static_scratch=True`` takes ra_decode_fwd_static instead: no allocation at all, the partials go to the
    library's built-in 16 MiB buffer of the GPU; calls that overlap in time on one GPU must not use it."""
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
    mi = _MaskInputs(cfg, attn_bias, segment_ids, cache_idx, B, q.device, L_buf)
    if out is None:
        out = torch.empty_like(q)
    lib = L.load()
    p = L.RaDecodeParams()
    p.q, p.k, p.v, p.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    p.dtype = _ra_dtype(q)
    p.B, p.L, p.H, p.D = B, L_buf, H, D
    p.q_stride_b = _rows(q)[0]
    p.kv_stride_b, p.kv_stride_s = _rows(k)
    if _rows(v) != _rows(k):
        raise ValueError("k and v caches must share strides")
    p.out_stride_b = _rows(out)[0]
    q_start = mi.cache_idx_host if mi.cache_idx_host is not None else 0
    p.mask = mi.fill(cfg, q_start, 0, False)
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
