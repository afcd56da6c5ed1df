"""Shared helpers of the parity tests: seeded inputs, oracle calls, error measures."""
import math

import torch

from oracle import ringattention_oracle as O


def kwargs(qc, kc, cbs=1, dtype=torch.float32, **extra):
    kw = dict(causal_block_size=cbs, deterministic=True, dropout_rng=None, attn_pdrop=0.0,
              query_chunk_size=qc, key_chunk_size=kc, dtype=dtype, policy=None, precision=None,
              prevent_cse=True)
    kw.update(extra)
    return kw


def oracle_kwargs(kw):
    return {k: v for k, v in kw.items() if k not in ("impl", "skip_masked_tiles", "bwd_only", "ring_launch", "output_residual",
                                                          "cache_segment_ids", "segment_hull_table")}


def make_qkv(B, S, H, D, dtype=torch.float32, seed=0, Skv=None, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    Skv = S if Skv is None else Skv
    q = (torch.randn(B, S, H, D, generator=g) * scale).to(dtype)
    k = (torch.randn(B, Skv, H, D, generator=g) * scale).to(dtype)
    v = torch.randn(B, Skv, H, D, generator=g).to(dtype)
    do = torch.randn(B, S, H, D, generator=g).to(dtype)
    return q, k, v, do


def packed_segment_ids(B, S, mean_len, seed=1):
    """Document ids of packed sequences: lengths ~ Geometric(1/mean_len), truncated to fill S."""
    g = torch.Generator().manual_seed(seed)
    out = torch.zeros(B, S, dtype=torch.int32)
    for b in range(B):
        pos, doc = 0, 0
        while pos < S:
            u = float(torch.rand(1, generator=g))
            ln = max(1, int(math.ceil(math.log(max(1.0 - u, 1e-12)) / math.log(1.0 - 1.0 / mean_len))))
            out[b, pos:pos + ln] = doc
            pos += ln
            doc += 1
    return out


def errors(got, ref):
    """(max-abs, relative L2) with NaN positions required to coincide."""
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    nan_g, nan_r = torch.isnan(got), torch.isnan(ref)
    assert torch.equal(nan_g, nan_r), "NaN positions differ"
    got = torch.where(nan_g, torch.zeros_like(got), got)
    ref = torch.where(nan_r, torch.zeros_like(ref), ref)
    max_abs = float((got - ref).abs().max()) if got.numel() else 0.0
    rel = float((got - ref).norm() / ref.norm().clamp_min(1e-30))
    return max_abs, rel


def tolerances(dtype):
    """The parity bar: max-abs 1e-4 (fp32) / 2e-2 (bf16), relative L2 1e-2."""
    return (1e-4, 1e-2) if dtype == torch.float32 else (2e-2, 1e-2)


def assert_close(got, ref, dtype, what=""):
    ma, rl = errors(got, ref)
    tol_abs, tol_rel = tolerances(dtype)
    assert ma <= tol_abs and rl <= tol_rel, "%s: max-abs %.3e (tol %.0e), rel-L2 %.3e (tol %.0e)" % (
        what, ma, tol_abs, rl, tol_rel)
    return ma, rl


def assert_close_scaled(got, ref, dtype, what=""):
    """assert_close for results that may be large (sharp softmax rows, q and k of standard deviation 3: gradients
    of 10 - 60).  The max-abs bars of 2e-2 / 1e-4 are meant for results of order one; beyond that they scale with the
    largest reference element: for the 16-bit types three bf16 units in the last place of it (one is what two
    roundings a boundary apart differ by, 3.1e-2 for a value in [4, 8); the weights P and dS are themselves rounded
    to bf16 before their second product, 2^-9 relative each on the terms that dominate a sharp row, and the result is
    rounded once more), for fp32 3e-5 of it
    (a logit of 40 carries 40 fp32 roundings' worth of error into its exponential, on either side).
    The relative L2 bar stays as it is."""
    ma, rl = errors(got, ref)
    tol_abs, tol_rel = tolerances(dtype)
    finite = ref.detach().float()
    finite = finite[torch.isfinite(finite)]
    top = float(finite.abs().max()) if finite.numel() else 0.0
    if top > 0.0:
        if dtype != torch.float32:
            tol_abs = max(tol_abs, 3.0 * 2.0 ** (math.floor(math.log2(top)) - 7))
        else:
            tol_abs = max(tol_abs, 3e-5 * top)
    if ma <= 1e-5:
        rl = 0.0            # a result that is zero but for rounding noise (one kept key per row: dq = 0) has no relative error
    assert ma <= tol_abs and rl <= tol_rel, "%s: max-abs %.3e (tol %.1e), rel-L2 %.3e (tol %.0e)" % (
        what, ma, tol_abs, rl, tol_rel)
    return ma, rl


def oracle_fwd_bwd(q, k, v, do, bias, seg, cache_idx, n, kw):
    """Oracle forward and backward on CPU in fp32 from the (possibly bf16) inputs."""
    okw = oracle_kwargs(kw)
    out, res = O.ring_attention_fwd(q, k, v, bias, seg, cache_idx, n, True, okw)
    grads = O.ring_attention_bwd(n, True, okw, res, do.float()) if do is not None else None
    return out, grads
