"""Attention dropout (ringattention_jax.py:119-123, :206-208, :311-321) on the GPU against the oracle.

The mask bits come from the Philox stream both sides document (not from jax.random, which is not restated), so
the comparison is exact in the mask and to the parity bar in the values: max-abs 1e-4 (fp32) / 2e-2 (bf16),
relative L2 1e-2."""
import pytest
import torch

import ringattention_amd as ra
from ringattention_amd import _lib as L
from oracle import ringattention_oracle as O
from tests.util import assert_close, errors, kwargs, make_qkv, oracle_fwd_bwd, packed_segment_ids

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("shape,seed,p", [
    ((1, 1, 4, 8), 0, 0.5),
    ((2, 3, 64, 128), 1234, 0.1),
    ((1, 2, 100, 40), (1 << 40) + 17, 0.25),       # an odd number of blocks: the tail of the last thread
    ((1, 1, 256, 4104), 0xFFFFFFFFFFFFFFFF, 0.9),
])
def test_dropout_mask_bits_are_the_documented_philox_stream(shape, seed, p):
    keep = torch.empty(shape, dtype=torch.uint8, device=DEV)
    L.check(L.load().ra_dropout_keep(seed, p, *shape, keep.data_ptr(), None), "ra_dropout_keep")
    torch.cuda.synchronize()
    dropped = O.dropout_mask(seed, p, shape)
    assert torch.equal(keep.cpu() == 0, dropped)
    if dropped.numel() >= 10000:
        assert abs(float(dropped.float().mean()) - p) < 0.02


@pytest.mark.parametrize("shape,seed,p", [((2, 3, 128, 192), 77, 0.3), ((1, 1, 64, 64), 1, 0.999), ((1, 2, 64, 128), 2, 1e-5)])
def test_packed_dropout_mask_equals_packing_the_byte_mask(shape, seed, p):
    B, H, Q, K = shape
    lib = L.load()
    keep = torch.empty(shape, dtype=torch.uint8, device=DEV)
    L.check(lib.ra_dropout_keep(seed, p, B, H, Q, K, keep.data_ptr(), None), "ra_dropout_keep")
    words = Q * K // 64
    mk = lambda: (torch.zeros((B, H, words), dtype=torch.int64, device=DEV),
                  torch.zeros((B, H, words), dtype=torch.int64, device=DEV),
                  torch.full((B, H, words // 64), 9, dtype=torch.uint8, device=DEV))
    a, b = mk(), mk()
    L.check(lib.ra_keep_pack(keep.data_ptr(), keep.stride(0), keep.stride(1), keep.stride(2), keep.stride(3), B, H, Q,
                             K, a[0].data_ptr(), a[1].data_ptr(), a[2].data_ptr(), None), "ra_keep_pack")
    L.check(lib.ra_dropout_keep_packed(seed, p, B, H, Q, K, b[0].data_ptr(), b[1].data_ptr(), b[2].data_ptr(),
                                       0, 0, 0, 0, 0, None), "ra_dropout_keep_packed")
    torch.cuda.synchronize()
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    # under a causal block size only the tiles of chunk pairs that run are written, with the same bits
    c = mk()
    L.check(lib.ra_dropout_keep_packed(seed, p, B, H, Q, K, c[0].data_ptr(), c[1].data_ptr(), c[2].data_ptr(),
                                       1, 64, 64, 0, 0, None), "ra_dropout_keep_packed")
    torch.cuda.synchronize()
    qt, kt = Q // 64, K // 64
    run = torch.tensor([[ra.below_or_on_diag(i, 64, j, 64, 1) for j in range(kt)] for i in range(qt)], device=DEV)
    summ_full, summ_run = b[2].view(B, H, qt, kt), c[2].view(B, H, qt, kt)
    assert torch.equal(summ_run[:, :, run], summ_full[:, :, run]) and bool((summ_run[:, :, ~run] == 9).all())
    wk_full, wk_run = b[0].view(B, H, kt, qt, 64), c[0].view(B, H, kt, qt, 64)       # [kt][q] words
    assert torch.equal(wk_run[:, :, run.t()], wk_full[:, :, run.t()]) and bool((wk_run[:, :, ~run.t()] == 0).all())
    wq_full, wq_run = b[1].view(B, H, qt, kt, 64), c[1].view(B, H, qt, kt, 64)       # [qt][k] words
    assert torch.equal(wq_run[:, :, run], wq_full[:, :, run]) and bool((wq_run[:, :, ~run] == 0).all())


def test_dropout_mask_rejects():
    lib = L.load()
    keep = torch.empty(64, dtype=torch.uint8, device=DEV)
    assert lib.ra_dropout_keep(0, 0.5, 1, 1, 8, 12, keep.data_ptr(), None) == L.RA_ERR_UNSUPPORTED    # K % 8
    assert lib.ra_dropout_keep(0, 0.0, 1, 1, 8, 8, keep.data_ptr(), None) == L.RA_ERR_INVALID
    assert lib.ra_dropout_keep(0, 1.0, 1, 1, 8, 8, keep.data_ptr(), None) == L.RA_ERR_INVALID
    assert lib.ra_dropout_keep(0, 0.5, 1, 1, 8, 8, None, None) == L.RA_ERR_INVALID
    w = torch.empty(4096, dtype=torch.int64, device=DEV)
    args = (w.data_ptr(), w.data_ptr(), keep.data_ptr())
    assert lib.ra_dropout_keep_packed(0, 0.5, 1, 1, 96, 64, *args, 0, 0, 0, 0, 0, None) == L.RA_ERR_UNSUPPORTED  # Q % 64
    assert lib.ra_dropout_keep_packed(0, 0.5, 1, 1, 64, 64, None, None, None, 0, 0, 0, 0, 0, None) == L.RA_ERR_INVALID
    assert lib.ra_dropout_keep_packed(0, 1.5, 1, 1, 64, 64, *args, 0, 0, 0, 0, 0, None) == L.RA_ERR_INVALID
    # chunk sizes that do not divide the mask, under a causal block size
    assert lib.ra_dropout_keep_packed(0, 0.5, 1, 1, 128, 128, *args, 1, 48, 64, 0, 0, None) == L.RA_ERR_INVALID


def _run(q, k, v, do, bias, seg, n, kw):
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    with ra.ring_axis("sp", n):
        out = ra.ringattention(qd, kd, vd, None if bias is None else bias.to(DEV),
                               None if seg is None else seg.to(DEV), None, axis_name="sp", float32_logits=True,
                               blockwise_kwargs=kw)
        out.backward(do.to(DEV))
    torch.cuda.synchronize()
    return out, (qd.grad, kd.grad, vd.grad)


def _compare(q, k, v, do, bias, seg, n, kw, dtype, what):
    print("dropout", what, flush=True)
    ref_out, ref_g = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    out, grads = _run(q, k, v, do, bias, seg, n, kw)
    assert_close(out, ref_out, dtype, what + " out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_g):
        assert_close(a, b, dtype, what + " " + name)
    return out


@pytest.mark.parametrize("n", [1, 2, 4])
@pytest.mark.parametrize("qc,kc,cbs", [(16, 16, 1), (16, 8, 1), (8, 16, 4), (16, 16, None)])
def test_dropout_generic_fp32_matches_oracle(n, qc, kc, cbs):
    """fp32, small chunks: the generic kernels; rings of 2 and 4 read the mask through the clamped slices."""
    B, S, H, D = 2, 64, 2, 32
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.float32, seed=11)
    kw = kwargs(qc, kc, cbs, deterministic=False, dropout_rng=1234, attn_pdrop=0.3)
    _compare(q, k, v, do, None, None, n, kw, torch.float32, "generic n%d %d/%d cbs %s" % (n, qc, kc, cbs))


def test_dropout_with_segments_and_bias_matches_oracle():
    B, S, H, D = 2, 128, 2, 32
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.float32, seed=12)
    seg = packed_segment_ids(B, S, 40, seed=3)
    bias = torch.randn(B, 1, 1, S, generator=torch.Generator().manual_seed(4))
    kw = kwargs(32, 16, 1, deterministic=False, dropout_rng=99, attn_pdrop=0.2)
    _compare(q, k, v, do, bias, seg, 2, kw, torch.float32, "segments + bias")


@pytest.mark.parametrize("n,S,qc,kc,cbs,p", [
    (1, 512, 256, 256, 1, 0.1),
    (1, 1024, 512, 256, 1, 0.5),
    (2, 1024, 256, 256, 1, 0.1),
    (4, 2048, 256, 512, 1, 0.3),
    (1, 512, 256, 256, None, 0.1),
    (2, 1024, 512, 512, 256, 0.2),
])
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_dropout_mfma_bf16_matches_oracle(n, S, qc, kc, cbs, p, D, dtype):
    """D 128 or 64, chunk sizes the MFMA kernels take (bf16 and fp32 family alike): the packed mask, next to the
    causal block size."""
    B, H = 1, 2
    q, k, v, do = make_qkv(B, S, H, D, dtype=dtype, seed=13, scale=D ** -0.25)
    kw = kwargs(qc, kc, cbs, deterministic=False, dropout_rng=7, attn_pdrop=p, impl="mfma")
    _compare(q, k, v, do, None, None, n, kw, dtype, "mfma n%d S%d %d/%d cbs %s p %.1f" % (n, S, qc, kc, cbs, p))


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("use_seg,use_bias,n", [(True, False, 1), (False, True, 2), (True, True, 2), (True, True, 4)])
def test_dropout_mfma_with_documents_and_bias_matches_oracle(use_seg, use_bias, n, D, dtype):
    """The dropout mask next to segment ids and a bias on the MFMA kernels: a pair of two documents counts as masked
    once (finfo.min), masked and dropped as twice (-inf), and the bias is clamped at 0 under a mask as always."""
    B, S, H = 2, 1024, 2
    q, k, v, do = make_qkv(B, S, H, D, dtype=dtype, seed=17, scale=D ** -0.25)
    seg = packed_segment_ids(B, S, 200, seed=6) if use_seg else None
    bias = torch.randn(B, H, 1, S, generator=torch.Generator().manual_seed(8)) if use_bias else None
    kw = kwargs(256, 256, 1, deterministic=False, dropout_rng=11, attn_pdrop=0.3, impl="mfma")
    _compare(q, k, v, do, bias, seg, n, kw, dtype, "mfma seg %s bias %s n%d" % (use_seg, use_bias, n))


def test_dropout_mfma_equals_generic():
    """The same mask through both kernel families, including the rows that lose every allowed key."""
    B, S, H, D = 1, 1024, 4, 128
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=14, scale=D ** -0.25)
    res = {}
    for impl in ("mfma", "generic"):
        kw = kwargs(256, 256, 1, deterministic=False, dropout_rng=5, attn_pdrop=0.5, impl=impl)
        res[impl] = _run(q, k, v, do, None, None, 2, kw)
    # with p = 0.5 row 0 of every head loses its one allowed key with probability 1/2: such rows exist here
    dropped = O.dropout_mask(5, 0.5, (B, H, S // 2, S // 2))
    assert bool(dropped[0, :, 0, 0].any())
    assert_close(res["mfma"][0], res["generic"][0].float(), torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), res["mfma"][1], res["generic"][1]):
        # both sides are rounded to bf16 (2^-8 relative each) and the rows with uniform weights make |dv| reach 4:
        # the absolute bar scales with the magnitude, the relative one is the usual 1e-2
        ma, rl = errors(a, b.float())
        assert ma <= 2e-2 * max(1.0, float(b.abs().max())) and rl <= 1e-2, (name, ma, rl)


def test_dropout_row_without_allowed_key_takes_uniform_weights():
    """Causal row 0 whose key 0 is dropped: logits are finfo.min at key 0 (dropped once) and at the causally masked
    keys that were not dropped, -inf at those masked AND dropped (:321 adds finfo.min twice): the output is the mean
    of V over the first set, in the one key chunk that runs for the row."""
    B, S, H, D, kc = 1, 256, 8, 128, 256
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=15, scale=D ** -0.25)
    seed, p = 21, 0.5
    dropped = O.dropout_mask(seed, p, (B, H, S, S))
    heads = [h for h in range(H) if bool(dropped[0, h, 0, 0])]
    assert heads, "no head drops key 0 of row 0 with this seed"
    for impl in ("mfma", "generic"):
        kw = kwargs(256, kc, 1, deterministic=False, dropout_rng=seed, attn_pdrop=p, impl=impl)
        out, _ = _run(q, k, v, do, None, None, 1, kw)
        for h in heads:
            level1 = ~dropped[0, h, 0, :kc]
            level1[0] = True
            want = v[0, :kc, h].float()[level1].mean(dim=0)
            got = out.detach()[0, 0, h].float().cpu()
            assert float((got - want).abs().max()) <= 2e-2, (impl, h)


def test_dropout_first_chunk_all_minus_inf_turns_the_row_nan_like_the_reference():
    """Small key chunks, a high rate and foreign documents: a row can meet a first key chunk whose pairs are all
    masked AND dropped (-inf) while its running max is still -inf; the reference then computes exp(-inf - -inf) = NaN
    (:138-144) and the row stays NaN, with the gradients that follow from it.  NaN positions must coincide."""
    B, S, H, D = 1, 128, 3, 32
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.float32, seed=16)
    seg = packed_segment_ids(B, S, 10, seed=5)
    for seed in range(50):
        kw = kwargs(32, 8, 1, deterministic=False, dropout_rng=seed, attn_pdrop=0.6)
        ref_out, _ = oracle_fwd_bwd(q, k, v, None, None, seg, None, 1, kw)
        if bool(torch.isnan(ref_out).any()):
            break
    else:
        pytest.fail("no seed below 50 produces the case")
    assert not bool(torch.isnan(ref_out).all())
    _compare(q, k, v, do, None, seg, 1, kw, torch.float32, "first chunk -inf, seed %d" % seed)


def test_dropout_probabilities_still_sum_to_one_at_8k():
    """V = 1: every row is a convex combination, whatever was dropped (rows without any allowed key included)."""
    B, S, H, D = 1, 8192, 4, 128
    g = torch.Generator(device=DEV).manual_seed(0)
    q = (torch.randn(B, S, H, D, device=DEV, generator=g) * D ** -0.25).bfloat16()
    k = (torch.randn(B, S, H, D, device=DEV, generator=g) * D ** -0.25).bfloat16()
    v = torch.ones(B, S, H, D, device=DEV, dtype=torch.bfloat16)
    kw = kwargs(512, 512, 1, deterministic=False, dropout_rng=3, attn_pdrop=0.1)
    out = ra.ringattention(q, k, v, None, None, None, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    assert float((out.float() - 1.0).abs().max()) <= 1e-2
    # and the mask is a function of the seed: same seed same bits, another seed another result
    v2 = torch.randn(B, S, H, D, device=DEV, generator=g).bfloat16()
    a = ra.ringattention(q, k, v2, None, None, None, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    b = ra.ringattention(q, k, v2, None, None, None, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    c = ra.ringattention(q, k, v2, None, None, None, axis_name=None, float32_logits=True,
                         blockwise_kwargs=dict(kw, dropout_rng=4))
    assert torch.equal(a, b) and not torch.equal(a, c)


def test_dropout_rejects():
    q, k, v, _ = make_qkv(1, 64, 2, 32, dtype=torch.float32, seed=1)
    q, k, v = (t.to(DEV) for t in (q, k, v))
    kw = kwargs(16, 16, 1, deterministic=False, attn_pdrop=0.1)          # no dropout_rng
    with pytest.raises(ValueError):
        ra.ringattention(q, k, v, None, None, None, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    kw = kwargs(1, 16, 1, deterministic=False, attn_pdrop=0.1, dropout_rng=1)
    with pytest.raises(NotImplementedError):                                # decode
        ra.ringattention(q[:, :1], k, v, None, None, 5, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    kw = kwargs(16, 16, 1, deterministic=False, attn_pdrop=1.0, dropout_rng=1)
    with pytest.raises(ValueError):
        ra.ringattention(q, k, v, None, None, None, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    # deterministic=True ignores attn_pdrop, as the reference does (:119)
    kw = kwargs(16, 16, 1, deterministic=True, attn_pdrop=0.5)
    a = ra.ringattention(q, k, v, None, None, None, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    b = ra.ringattention(q, k, v, None, None, None, axis_name=None, float32_logits=True,
                         blockwise_kwargs=kwargs(16, 16, 1))
    assert torch.equal(a, b)
