"""The steps a model runs either side of the hot path, over the bandwidth-bound kernels of libringattn_hip.so:
``rope_kv_append`` before a decode step (rotary embedding of the new token's query / key at ``cache_idx`` and the
write of the new key / value into the cache buffers that ``ringattention(..., cache_idx)`` reads,
ringattention_jax.py:31-35) and ``rmsnorm_residual`` around ``blockwise_feedforward`` (:333-352).  The reference
repository has neither (its README points at the LWM model code); the formulas are the LLaMA ones."""
import ctypes

import torch

from . import _lib as L
from .ringattention_hip import _ra_dtype, _stream

ROPE_STYLES = {"adjacent": 0, "half": 1}


def rope_kv_append(q, k_new, v_new, k_cache, v_cache, cache_idx, rope_theta=10000.0, rope_style="adjacent",
                   q_out=None):
    """q, k_new, v_new (B,1,H,D); k_cache, v_cache (B,L,H,D), written in place at position ``cache_idx`` (a Python
    int or a device int32 scalar) of every batch row.  Returns the rotated query.  ``rope_style`` "adjacent" pairs
    elements (2j, 2j+1) (the complex-number form of LLaMA / LWM), "half" pairs (j, j + D/2);
    ``rope_theta`` None or 0 appends without rotating."""
    for t in (q, k_new, v_new, k_cache, v_cache):
        if not t.is_cuda:
            raise RuntimeError("ringattention_amd runs on the GPU only")
    B, one, H, D = q.shape
    if one != 1 or k_new.shape != q.shape or v_new.shape != q.shape:
        raise ValueError("q, k_new and v_new must be (B, 1, H, D)")
    if k_cache.shape != v_cache.shape or k_cache.shape[0] != B or tuple(k_cache.shape[2:]) != (H, D):
        raise ValueError("k_cache and v_cache must be (B, L, H, D) with the batch, heads and head size of q")
    if not (q.dtype == k_new.dtype == v_new.dtype == k_cache.dtype == v_cache.dtype):
        raise ValueError("q, k_new, v_new and the caches must share a dtype")
    if rope_style not in ROPE_STYLES:
        raise ValueError("rope_style must be 'adjacent' or 'half'")
    for t in (q, k_new, v_new, k_cache, v_cache):
        if t.stride(3) != 1 or t.stride(2) != D:
            raise ValueError("the head axis must be dense (stride D) and the last axis contiguous")
    if k_cache.stride() != v_cache.stride() or k_new.stride(0) != v_new.stride(0):
        raise ValueError("k / v buffers must share strides")
    if q_out is None:
        q_out = torch.empty_like(q)
    p = L.RaRopeAppendParams()
    p.q, p.q_out, p.k_new, p.v_new = q.data_ptr(), q_out.data_ptr(), k_new.data_ptr(), v_new.data_ptr()
    p.k_cache, p.v_cache = k_cache.data_ptr(), v_cache.data_ptr()
    if isinstance(cache_idx, torch.Tensor):
        if cache_idx.dtype != torch.int32 or cache_idx.numel() != 1 or not cache_idx.is_cuda:
            raise ValueError("a tensor cache_idx must be one int32 on the device")
        p.cache_idx, p.cache_idx_host = cache_idx.data_ptr(), 0
    else:
        p.cache_idx, p.cache_idx_host = None, int(cache_idx)
    p.dtype = _ra_dtype(q)
    p.B, p.L, p.H, p.D = B, k_cache.shape[1], H, D
    p.q_stride_b, p.q_out_stride_b, p.new_stride_b = q.stride(0), q_out.stride(0), k_new.stride(0)
    p.cache_stride_b, p.cache_stride_s = k_cache.stride(0), k_cache.stride(1)
    p.rope_theta = float(rope_theta or 0.0)
    p.rope_style = ROPE_STYLES[rope_style]
    L.check(L.load().ra_rope_kv_append(ctypes.byref(p), _stream()), "ra_rope_kv_append")
    return q_out


class _RMSNormResidualFn(torch.autograd.Function):
    """y = x + residual, normed = y * rsqrt(mean(y^2) + eps) * weight; returns (y, normed).  With residual None,
    y is x itself."""

    @staticmethod
    def forward(ctx, x, residual, weight, eps):
        T, d = x.shape
        normed = torch.empty_like(x)
        y = torch.empty_like(x) if residual is not None else x
        rstd = torch.empty(T, dtype=torch.float32, device=x.device)
        p = L.RaRmsnormParams()
        p.T, p.d, p.eps = T, d, eps
        p.x, p.residual, p.weight = x.data_ptr(), (residual.data_ptr() if residual is not None else None), weight.data_ptr()
        p.y, p.normed, p.rstd = (y.data_ptr() if residual is not None else None), normed.data_ptr(), rstd.data_ptr()
        L.check(L.load().ra_rmsnorm_fwd(ctypes.byref(p), _stream()), "ra_rmsnorm_fwd")
        ctx.save_for_backward(y, weight, rstd)
        ctx.has_residual = residual is not None
        ctx.mark_non_differentiable(rstd)
        return y, normed

    @staticmethod
    def backward(ctx, d_y_in, d_normed):
        y, weight, rstd = ctx.saved_tensors
        T, d = y.shape
        lib = L.load()
        d_normed = (torch.zeros_like(y) if d_normed is None else d_normed.to(torch.bfloat16).contiguous())
        d_res = d_y_in.to(torch.bfloat16).contiguous() if d_y_in is not None else None
        d_y = torch.empty_like(y)
        d_w = torch.zeros(d, dtype=torch.float32, device=y.device)
        nbytes = lib.ra_rmsnorm_workspace_bytes(T, d)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=y.device)
        p = L.RaRmsnormParams()
        p.T, p.d = T, d
        p.weight, p.y, p.rstd = weight.data_ptr(), y.data_ptr(), rstd.data_ptr()
        p.d_normed, p.d_residual = d_normed.data_ptr(), (d_res.data_ptr() if d_res is not None else None)
        p.d_y, p.d_weight, p.dw_workspace, p.dw_workspace_bytes = d_y.data_ptr(), d_w.data_ptr(), ws.data_ptr(), nbytes
        L.check(lib.ra_rmsnorm_bwd(ctypes.byref(p), _stream()), "ra_rmsnorm_bwd")
        return d_y, (d_y if ctx.has_residual else None), d_w.to(weight.dtype), None


def rmsnorm_residual(x, residual, weight, eps=1e-6):
    """x, residual (..., d) bf16 (residual may be None), weight (d,) bf16.  Returns (y, normed) with y = x + residual
    (the residual stream, rounded to bf16 as it is stored) and normed = RMSNorm(y) * weight."""
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise NotImplementedError("the RMSNorm kernels are bf16")
    if not x.is_cuda:
        raise RuntimeError("ringattention_amd runs on the GPU only")
    shp = x.shape
    d = shp[-1]
    if weight.shape != (d,):
        raise ValueError("weight must be (%d,)" % d)
    if residual is not None and (residual.shape != shp or residual.dtype != x.dtype):
        raise ValueError("residual must match x")
    x2 = x.reshape(-1, d).contiguous()
    r2 = residual.reshape(-1, d).contiguous() if residual is not None else None
    y, normed = _RMSNormResidualFn.apply(x2, r2, weight.contiguous(), float(eps))
    return y.reshape(shp), normed.reshape(shp)
