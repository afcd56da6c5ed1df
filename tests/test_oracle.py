"""Pins the CPU oracle against what the mathematics fixes: an independent dense softmax in
float64, torch.autograd / finite differences for the backward, exhaustive integer tables for the
skip predicate, and case enumeration for the bias builder."""
import itertools
import math

import pytest
import torch

from oracle import ringattention_oracle as O

F64 = torch.float64


def kwargs(qc, kc, cbs=1, dtype=torch.float32):
    return dict(causal_block_size=cbs, deterministic=True, dropout_rng=None, attn_pdrop=0.0,
                query_chunk_size=qc, key_chunk_size=kc, dtype=dtype, policy=None, precision=None,
                prevent_cse=True)


def make(B, S, H, D, seed=0, dtype=F64, Skv=None):
    g = torch.Generator().manual_seed(seed)
    Skv = S if Skv is None else Skv
    q = torch.randn(B, S, H, D, generator=g, dtype=dtype)
    k = torch.randn(B, Skv, H, D, generator=g, dtype=dtype)
    v = torch.randn(B, Skv, H, D, generator=g, dtype=dtype)
    return q, k, v


def seg_ids(B, S, seed=1, mean=7):
    g = torch.Generator().manual_seed(seed)
    out = torch.zeros(B, S, dtype=torch.int32)
    for b in range(B):
        pos, doc = 0, 0
        while pos < S:
            ln = int(torch.randint(1, 2 * mean, (1,), generator=g))
            out[b, pos:pos + ln] = doc
            pos += ln
            doc += 1
    return out


# ----------------------------------------------------------------------------- predicate

def brute_tile_has_unmasked(r, qc, c, kc, cbs):
    for i in range(r * qc, (r + 1) * qc):
        for j in range(c * kc, (c + 1) * kc):
            if not (i // cbs < j // cbs):
                return True
    return False


@pytest.mark.parametrize("blk", [2, 3, 4, 8])
@pytest.mark.parametrize("cbs", [1, 2, 4, 8, 16])
def test_predicate_equal_chunks_matches_bruteforce(blk, cbs):
    if cbs > blk and cbs % blk:
        pytest.skip("causal block must be a multiple of the chunk")
    if cbs < blk and blk % cbs:
        pytest.skip("chunk must be a multiple of the causal block")
    for r in range(12):
        for c in range(12):
            assert bool(O.below_or_on_diag(r, blk, c, blk, cbs)) == brute_tile_has_unmasked(r, blk, c, blk, cbs), (r, c)


def test_predicate_off_by_one_cases():
    # chunk sizes (1,1): the strict '>' drops every diagonal tile
    for r in range(8):
        assert not O.below_or_on_diag(r, 1, r, 1, 1)
        if r:
            assert O.below_or_on_diag(r, 1, r - 1, 1, 1)
    # decode shape (1,512): the query's own key chunk runs unless q_pos % 512 == 0
    for pos in [0, 1, 511, 512, 513, 1024, 1500]:
        own = pos // 512
        assert bool(O.below_or_on_diag(pos, 1, own, 512, 1)) == (pos % 512 != 0)
        if own:
            assert O.below_or_on_diag(pos, 1, own - 1, 512, 1)
        assert not O.below_or_on_diag(pos, 1, own + 1, 512, 1)


def test_predicate_closed_form_unequal_chunks():
    # with cbs=1 the predicate is "last row of the q chunk is strictly past the first key of the k chunk"
    for qc, kc in [(2, 4), (4, 2), (8, 2), (2, 8), (3, 5)]:
        for r in range(10):
            for c in range(10):
                assert bool(O.below_or_on_diag(r, qc, c, kc, 1)) == ((r + 1) * qc - 1 > c * kc)


# ----------------------------------------------------------------------------- bias builder

def test_chunk_bias_cases():
    qc, kc = 4, 4
    bias = torch.tensor([0.5, -1.0, 2.0, -3.0, 1.0, -0.25, 0.0, 4.0]).reshape(1, 1, 1, 8)
    seg = torch.tensor([[0, 0, 0, 1, 1, 1, 2, 2]], dtype=torch.int32)
    fmin32 = torch.finfo(torch.float32).min
    # bias only: passed through unclamped, sliced at the global key offset
    t = O.chunk_attention_bias(qc, kc, bias, None, None, torch.float32, 0, 1)
    assert torch.equal(t, bias[..., 4:8])
    # nothing at all: a single zero
    t = O.chunk_attention_bias(qc, kc, None, None, None, torch.float32, 1, 0)
    assert t.shape == (1, 1, 1, 1) and float(t) == 0.0
    # causal only, diagonal tile
    t = O.chunk_attention_bias(qc, kc, None, None, 1, torch.float32, 1, 1)
    exp = torch.triu(torch.ones(4, 4), diagonal=1) * fmin32
    assert torch.equal(t[0, 0], exp)
    # segment + bias: allowed -> min(bias, 0), masked -> finfo.min
    t = O.chunk_attention_bias(qc, kc, bias, seg, None, torch.float32, 0, 1)
    for i in range(4):
        for j in range(4):
            if seg[0, i] == seg[0, 4 + j]:
                assert float(t[0, 0, i, j]) == min(float(bias[0, 0, 0, 4 + j]), 0.0)
            else:
                assert float(t[0, 0, i, j]) == fmin32
    # everything, bf16 kwargs dtype: mask value is the bf16 minimum and the bias is rounded to bf16
    b2 = torch.tensor([-1.001, -2.003, 0.3, -0.7]).reshape(1, 1, 1, 4)
    t = O.chunk_attention_bias(qc, kc, b2, seg[:, :4], 1, torch.bfloat16, 0, 0)
    assert float(t[0, 0, 0, 1]) == torch.finfo(torch.bfloat16).min
    assert float(t[0, 0, 1, 0]) == float(torch.tensor(-1.001).bfloat16())
    assert float(t[0, 0, 2, 2]) == 0.0   # positive bias clamped
    assert abs(torch.finfo(torch.bfloat16).min - (-3.3895314e38)) < 1e32
    assert abs(torch.finfo(torch.float32).min - (-3.4028235e38)) < 1e31


def test_chunk_bias_causal_block_size():
    t = O.chunk_attention_bias(4, 4, None, None, 2, torch.float32, 1, 1)
    # positions 4..7, blocks of 2: (4,5) see (4,5); (6,7) see (4..7)
    exp_masked = torch.tensor([[0, 0, 1, 1], [0, 0, 1, 1], [0, 0, 0, 0], [0, 0, 0, 0]], dtype=torch.bool)
    assert torch.equal(t[0, 0] != 0, exp_masked)


# ----------------------------------------------------------------------------- forward vs dense

FWD_CASES = [
    # B,S,H,D,qc,kc,cbs,N,use_bias,use_seg
    (1, 32, 2, 8, 8, 8, 1, 1, False, False),
    (2, 32, 2, 8, 8, 8, 1, 1, True, True),
    (1, 32, 1, 4, 4, 8, 1, 1, True, False),
    (1, 32, 1, 4, 8, 4, 1, 2, False, True),
    (2, 48, 2, 8, 4, 4, 1, 3, True, True),
    (1, 64, 2, 8, 8, 8, 1, 4, True, True),
    (1, 64, 1, 8, 8, 8, 4, 2, True, True),
    (1, 64, 1, 8, 4, 4, 8, 2, False, False),
    (1, 64, 1, 8, 16, 8, 2, 1, True, False),
    (1, 32, 2, 8, 8, 8, None, 1, True, True),
    (1, 32, 2, 8, 8, 8, None, 2, True, False),
    (1, 32, 2, 8, 8, 8, None, 1, False, False),
    (1, 16, 1, 4, 2, 2, 1, 1, False, False),
]


@pytest.mark.parametrize("case", FWD_CASES)
def test_forward_matches_dense(case):
    B, S, H, D, qc, kc, cbs, N, use_bias, use_seg = case
    q, k, v = make(B, S, H, D, seed=S + H)
    g = torch.Generator().manual_seed(5)
    bias = torch.randn(B, 1, 1, S, generator=g, dtype=F64) if use_bias else None
    seg = seg_ids(B, S) if use_seg else None
    kw = kwargs(qc, kc, cbs)
    out, res = O.ring_attention_fwd(q, k, v, bias, seg, None, N, True, kw, compute_dtype=F64)
    ref = O.dense_attention(q, k, v, bias, seg, None, N, kw)
    assert torch.allclose(out, ref, atol=1e-12, rtol=1e-10)
    # softmax statistics: den * exp(max) is the dense partition function
    assert torch.isfinite(res[-1]).all() and (res[-2] > 0).all()


def test_forward_ring_and_chunk_invariance():
    q, k, v = make(1, 64, 2, 8, seed=3)
    seg = seg_ids(1, 64)
    base = O.ring_attention(q, k, v, None, seg, None, 1, True, kwargs(8, 8), compute_dtype=F64)
    for N, qc, kc in [(2, 8, 8), (4, 8, 8), (8, 8, 8), (1, 16, 4), (2, 4, 16), (1, 2, 32)]:
        o = O.ring_attention(q, k, v, None, seg, None, N, True, kwargs(qc, kc), compute_dtype=F64)
        assert torch.allclose(o, base, atol=1e-12), (N, qc, kc)


def test_rows_sum_to_one_and_head_batch_equivariance():
    q, k, v = make(2, 32, 3, 8, seed=9)
    ones = torch.ones_like(v)
    o = O.ring_attention(q, k, ones, None, None, None, 2, True, kwargs(8, 8), compute_dtype=F64)
    assert torch.allclose(o, ones, atol=1e-13)
    perm_b, perm_h = [1, 0], [2, 0, 1]
    o1 = O.ring_attention(q, k, v, None, None, None, 2, True, kwargs(8, 8), compute_dtype=F64)
    o2 = O.ring_attention(q[perm_b][:, :, perm_h], k[perm_b][:, :, perm_h], v[perm_b][:, :, perm_h],
                          None, None, None, 2, True, kwargs(8, 8), compute_dtype=F64)
    assert torch.equal(o1[perm_b][:, :, perm_h], o2)


def test_positive_bias_is_clamped_only_with_masks():
    q, k, v = make(1, 16, 1, 4, seed=2)
    bias = torch.full((1, 1, 1, 16), 3.0, dtype=F64)
    bias[..., ::2] = -1.0
    kw_nomask = kwargs(4, 4, None)
    a = O.ring_attention(q, k, v, bias, None, None, 1, True, kw_nomask, compute_dtype=F64)
    b = O.ring_attention(q, k, v, torch.clamp(bias, max=0.0), None, None, 1, True, kw_nomask, compute_dtype=F64)
    assert not torch.allclose(a, b)
    kw = kwargs(4, 4, 1)
    a = O.ring_attention(q, k, v, bias, None, None, 1, True, kw, compute_dtype=F64)
    b = O.ring_attention(q, k, v, torch.clamp(bias, max=0.0), None, None, 1, True, kw, compute_dtype=F64)
    assert torch.equal(a, b)


def test_masked_keys_are_bitwise_isolated():
    q, k, v = make(1, 32, 2, 8, seed=4, dtype=torch.float32)
    kw = kwargs(8, 8, 1)
    a = O.ring_attention(q, k, v, None, None, None, 2, True, kw)
    k2, v2 = k.clone(), v.clone()
    k2[:, 20:] += 100.0
    v2[:, 20:] -= 50.0
    b = O.ring_attention(q, k2, v2, None, None, None, 2, True, kw)
    assert torch.equal(a[:, :20], b[:, :20])


def test_fully_masked_then_real_is_annihilated_exactly():
    # key chunk 0 belongs to another segment: the row first sees uniform weights, then exactly none of it
    q, k, v = make(1, 8, 1, 4, seed=6, dtype=torch.float32)
    seg = torch.tensor([[0, 0, 0, 0, 1, 1, 1, 1]], dtype=torch.int32)
    kw = kwargs(4, 4, 1)
    a = O.ring_attention(q, k, v, None, seg, None, 1, True, kw)
    b = O.ring_attention(q[:, 4:], k[:, 4:], v[:, 4:], None, None, None, 1, True, kw)
    assert torch.equal(a[:, 4:], b)


# ----------------------------------------------------------------------------- decode (cache_idx)

@pytest.mark.parametrize("cache_idx", [1, 5, 8, 13, 16, 23])
def test_decode_matches_dense_and_prefill_row(cache_idx):
    L, kc = 32, 8
    q, k, v = make(2, L, 2, 8, seed=11)
    kw = kwargs(1, kc, 1)
    q1 = q[:, cache_idx:cache_idx + 1]
    out = O.ring_attention(q1, k, v, None, None, cache_idx, 1, True, kw, compute_dtype=F64)
    ref = O.dense_attention(q1, k, v, None, None, cache_idx, 1, kw)
    assert torch.allclose(out, ref, atol=1e-12)
    # keys attended: 0..cache_idx, minus the own chunk when cache_idx % kc == 0 (the strict '>')
    last = cache_idx if cache_idx % kc else cache_idx - 1
    w = torch.einsum('bqhd,bkhd->bhqk', q1, k[:, :last + 1]) / math.sqrt(8)
    exp = torch.einsum('bhqk,bkhd->bqhd', torch.softmax(w, -1), v[:, :last + 1])
    assert torch.allclose(out, exp, atol=1e-12)
    if cache_idx % kc:
        pre = O.ring_attention(q, k, v, None, None, None, 1, True, kwargs(8, kc, 1), compute_dtype=F64)
        assert torch.allclose(out[:, 0], pre[:, cache_idx], atol=1e-12)


def test_decode_at_zero_is_nan():
    q, k, v = make(1, 8, 1, 4, seed=1)
    out = O.ring_attention(q[:, :1], k, v, None, None, 0, 1, True, kwargs(1, 4, 1), compute_dtype=F64)
    assert torch.isnan(out).all()


# ----------------------------------------------------------------------------- backward

BWD_CASES = [
    (1, 32, 2, 8, 8, 8, 1, 1, False, False),
    (2, 32, 2, 8, 8, 8, 1, 2, True, True),
    (1, 48, 1, 4, 4, 8, 1, 3, True, False),
    (1, 64, 2, 8, 8, 4, 4, 2, True, True),
    (1, 32, 2, 8, 8, 8, None, 2, True, True),
    (1, 32, 1, 8, 16, 8, 1, 1, False, True),
]


@pytest.mark.parametrize("case", BWD_CASES)
def test_backward_matches_autograd_of_dense(case):
    B, S, H, D, qc, kc, cbs, N, use_bias, use_seg = case
    q, k, v = make(B, S, H, D, seed=S)
    gen = torch.Generator().manual_seed(8)
    g = torch.randn(B, S, H, D, generator=gen, dtype=F64)
    bias = torch.randn(B, 1, 1, S, generator=gen, dtype=F64) if use_bias else None
    seg = seg_ids(B, S) if use_seg else None
    kw = kwargs(qc, kc, cbs)
    _, res = O.ring_attention_fwd(q, k, v, bias, seg, None, N, True, kw, compute_dtype=F64)
    dq, dk, dv = O.ring_attention_bwd(N, True, kw, res, g)
    qa, ka, va = (x.clone().requires_grad_(True) for x in (q, k, v))
    ref = O.dense_attention(qa, ka, va, bias, seg, None, N, kw)
    ref.backward(g)
    for a, b in ((dq, qa.grad), (dk, ka.grad), (dv, va.grad)):
        assert torch.allclose(a, b, atol=1e-11, rtol=1e-9)


def test_backward_finite_differences():
    q, k, v = make(1, 8, 1, 4, seed=21)
    gen = torch.Generator().manual_seed(3)
    g = torch.randn(1, 8, 1, 4, generator=gen, dtype=F64)
    kw = kwargs(4, 4, 1)
    _, res = O.ring_attention_fwd(q, k, v, None, None, None, 2, True, kw, compute_dtype=F64)
    dq, dk, dv = O.ring_attention_bwd(2, True, kw, res, g)

    def f(q_, k_, v_):
        return float((O.ring_attention(q_, k_, v_, None, None, None, 2, True, kw, compute_dtype=F64) * g).sum())
    eps = 1e-6
    for which, grad in ((0, dq), (1, dk), (2, dv)):
        for idx in [(0, 1, 0, 2), (0, 5, 0, 0), (0, 7, 0, 3)]:
            args = [q.clone(), k.clone(), v.clone()]
            args[which][idx] += eps
            up = f(*args)
            args[which][idx] -= 2 * eps
            dn = f(*args)
            assert abs((up - dn) / (2 * eps) - float(grad[idx])) < 1e-6


def test_backward_adds_into_incoming_gradients():
    q, k, v = make(1, 16, 1, 4, seed=5)
    kw = kwargs(4, 4, 1)
    _, res = O.ring_attention_fwd(q, k, v, None, None, None, 1, True, kw, compute_dtype=F64)
    out, qw, kw_, vv, _, _, _, den, mx = res
    g = torch.ones_like(q)
    z = torch.zeros_like(q)
    a = O.blockwise_attention_bwd(qw, kw_, vv, g, (z, z, z, out, den, mx), 0, 0, None, None, **kw)
    one = torch.ones_like(q)
    b = O.blockwise_attention_bwd(qw, kw_, vv, g, (one, 2 * one, 3 * one, out, den, mx), 0, 0, None, None, **kw)
    for i, (x, y) in enumerate(zip(a, b)):
        assert torch.allclose(x + (i + 1), y, atol=1e-13)


# ----------------------------------------------------------------------------- feed-forward

def test_blockwise_feedforward_equals_unchunked_and_uses_strided_groups():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 24, 8, generator=g, dtype=F64)
    w1, w3 = torch.randn(8, 20, generator=g, dtype=F64), torch.randn(8, 20, generator=g, dtype=F64)
    w2 = torch.randn(20, 8, generator=g, dtype=F64)
    seen = []

    def ff(h):
        seen.append(h.clone())
        return O.swiglu(h, w1, w2, w3)
    y = O.blockwise_feedforward(ff, x, 6)
    assert torch.allclose(y, O.swiglu(x, w1, w2, w3), atol=1e-12)
    assert len(seen) == 4 and seen[0].shape == (2, 6, 8)
    # step j gets tokens {ci * n + j}: a strided set, n = S / chunk_size
    assert torch.equal(seen[1], x[:, 1::4])


# --------------------------------------------------------------------------- attention dropout
def test_philox_known_answers():
    """Philox4x32-10 known-answer vectors of the Random123 distribution (kat_vectors): zero, all ones, digits of pi."""
    import numpy as np
    cases = [
        ([0, 0, 0, 0], [0, 0], "6627e8d5 e169c58d bc57ac4c 9b00dbd8"),
        ([0xffffffff] * 4, [0xffffffff] * 2, "408f276d 41c83b0e a20bc7c6 6d5451fd"),
        ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
         "d16cfe09 94fdcceb 5001e420 24126ea1"),
    ]
    for counter, key, want in cases:
        got = O.philox4x32_10(np.array([counter], dtype=np.uint32), np.array([key], dtype=np.uint32))[0]
        assert " ".join("%08x" % int(x) for x in got) == want


def test_dropout_mask_is_a_function_of_seed_and_rate():
    a = O.dropout_mask(5, 0.25, (2, 3, 32, 64))
    assert a.dtype == torch.bool and a.shape == (2, 3, 32, 64)
    assert torch.equal(a, O.dropout_mask(5, 0.25, (2, 3, 32, 64)))
    assert not torch.equal(a, O.dropout_mask(6, 0.25, (2, 3, 32, 64)))
    assert abs(float(a.float().mean()) - 0.25) < 0.02
    # position e takes word e % 4 of block e // 4: a longer mask with the same seed starts with the same bits
    b = O.dropout_mask(5, 0.25, (1, 1, 1, 128))
    assert torch.equal(b.reshape(-1), O.dropout_mask(5, 0.25, (1, 1, 2, 128)).reshape(-1)[:128])
    # a lower rate drops a subset (same words, lower threshold)
    assert bool((O.dropout_mask(5, 0.1, (2, 3, 32, 64)) <= a).all())


def _dropout_kwargs(qc, kc, cbs, p=0.3, seed=1234):
    kw = kwargs(qc, kc, cbs)
    kw.update(deterministic=False, attn_pdrop=p, dropout_rng=seed)
    return kw


@pytest.mark.parametrize("n", [1, 2, 4])
@pytest.mark.parametrize("qc,kc,cbs", [(16, 16, 1), (16, 8, 1), (8, 16, 4), (16, 16, None)])
def test_dropout_blockwise_matches_dense(n, qc, kc, cbs):
    """The chunk loops with the sliced mask (:311-321) against the un-chunked softmax whose mask is built from
    global positions, float64, on the rows that keep an allowed key (the others are covered in fp32 below); rings
    of 2 and 4 read the mask of local shape through the clamped global offsets."""
    q, k, v = make(2, 64, 2, 16, seed=1)
    kw = _dropout_kwargs(qc, kc, cbs)
    out, res = O.ring_attention_fwd(q, k, v, None, None, None, n, True, kw, compute_dtype=F64)
    ref = O.dense_attention(q, k, v, None, None, None, n, kw)
    real = (res[-1] > -1e30).permute(0, 2, 1)
    assert int(real.sum()) >= real.numel() - 8
    assert float((out - ref)[real].abs().max()) < 1e-12
    # backward against autograd of the dense form, on cotangents that vanish on the other rows
    g = torch.randn(out.shape, dtype=F64, generator=torch.Generator().manual_seed(2)) * real[..., None]
    dq, dk, dv = O.ring_attention_bwd(n, True, kw, res, g)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    dense = O.dense_attention(qa, ka, va, None, None, None, n, kw)
    torch.where(real[..., None], dense, torch.zeros_like(dense)).mul(g).sum().backward()
    for a, b in ((dq, qa.grad), (dk, ka.grad), (dv, va.grad)):
        assert float((a - b).abs().max()) < 1e-10


def test_dropped_keys_get_exactly_zero_weight():
    q, k, v = make(1, 64, 2, 16, seed=3)
    kw = _dropout_kwargs(16, 16, None, p=0.4, seed=9)
    dropped = O.dropout_mask(9, 0.4, (1, 2, 64, 64))
    out = O.ring_attention(q, k, v, None, None, None, 1, True, kw, compute_dtype=F64)
    # equals a softmax over the kept keys only
    logits = torch.einsum("bqhd,bkhd->bhqk", q, k) / math.sqrt(16)
    p = torch.softmax(logits.masked_fill(dropped, -math.inf), dim=-1)
    ref = torch.einsum("bhqk,bkhd->bqhd", p, v)
    assert float((out - ref).abs().max()) < 1e-12
    # no rescale by 1 / (1 - p) (:321 only masks): rows still sum to one
    ones = O.ring_attention(q, k, torch.ones_like(v), None, None, None, 1, True, kw, compute_dtype=F64)
    assert float((ones - 1.0).abs().max()) < 1e-12


def test_dropout_row_without_allowed_key_fp32():
    """Causal row 0 with key 0 dropped, fp32 as the reference computes: key 0 holds finfo.min (dropped once), the
    causally masked keys hold finfo.min if kept and -inf if dropped (finfo.min added twice, :321), so the row is the
    mean of V over {key 0} and the kept masked keys of the chunks that run."""
    seed = next(s for s in range(100) if bool(O.dropout_mask(s, 0.5, (1, 1, 16, 16))[0, 0, 0, 0]))
    dropped = O.dropout_mask(seed, 0.5, (1, 1, 16, 16))
    q, k, v = make(1, 16, 1, 8, seed=4, dtype=torch.float32)
    for qc, kc in ((16, 16), (8, 8), (16, 4)):
        kw = _dropout_kwargs(qc, kc, 1, p=0.5, seed=seed)
        out = O.ring_attention(q, k, v, None, None, None, 1, True, kw)
        ncols = kc if qc <= kc else 16     # key chunks that run for row 0: below_or_on_diag keeps c * kc < qc
        level1 = ~dropped[0, 0, 0, :ncols]
        level1[0] = True
        want = v[0, :ncols, 0][level1].mean(dim=0)
        assert float((out[0, 0, 0] - want).abs().max()) < 1e-6, (qc, kc)


# --------------------------------------------------------------------------- ring_attention_inference
INFER_MASK_SHAPES = [("full", lambda B, H, S: (B, H, S, S)), ("bcast_bh", lambda B, H, S: (1, 1, S, S)),
                     ("key_only", lambda B, H, S: (B, 1, 1, S)), ("per_head", lambda B, H, S: (1, H, S, S))]


@pytest.mark.parametrize("name,shape_fn", INFER_MASK_SHAPES)
@pytest.mark.parametrize("n", [1, 2, 4])
def test_inference_ring_matches_dense_masked_softmax(name, shape_fn, n):
    """ringattention_inference.py restated vs an un-chunked masked softmax and its autograd, float64."""
    B, S, H, D = 2, 48, 3, 16
    g0 = torch.Generator().manual_seed(7)
    q, k, v, g = (torch.randn(B, S, H, D, dtype=torch.float64, generator=g0) for _ in range(4))
    mask = torch.rand(shape_fn(B, H, S), generator=g0) > 0.4
    mask[..., 0] = True                      # every row attends to something: the closed form has a gradient
    out, res = O.ring_attention_inference_fwd(q, k, v, mask, n, True, compute_dtype=torch.float64)
    qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
    ref = O.dense_attention_inference(qq, kk, vv, mask)
    assert (out - ref.detach()).abs().max() < 1e-12
    ref.backward(g)
    dq, dk, dv = O.ring_attention_inference_bwd(n, res, g)
    for a, b in ((dq, qq.grad), (dk, kk.grad), (dv, vv.grad)):
        assert (a - b).abs().max() < 1e-11


def test_inference_row_without_attended_key_is_uniform():
    """where(mask, w, finfo.min) leaves equal logits on a fully masked row: its output is the mean of V
    over every key of the ring, whatever the ring size, and dv matches the uniform weights."""
    B, S, H, D = 1, 32, 2, 8
    g0 = torch.Generator().manual_seed(8)
    q, k, v, g = (torch.randn(B, S, H, D, generator=g0) for _ in range(4))
    mask = torch.rand(1, 1, S, S, generator=g0) > 0.5
    mask[..., 0] = True
    mask[:, :, 5, :] = False
    for n in (1, 4):
        out, res = O.ring_attention_inference_fwd(q, k, v, mask, n, True)
        assert torch.allclose(out[:, 5], v.mean(dim=1), atol=1e-6)
        ref = O.dense_attention_inference(q, k, v, mask).float()
        assert (out - ref).abs().max() < 1e-5
        _dq, _dk, dv = O.ring_attention_inference_bwd(n, res, g)
        vv = v.clone().double().requires_grad_(True)
        O.dense_attention_inference(q, k, vv, mask).backward(g.double())
        assert (dv - vv.grad.float()).abs().max() < 1e-5


def test_inference_equals_ring_attention_with_causal_mask():
    """A causal boolean mask reproduces the blockwise path (chunk sizes >= 2, so no diagonal tile is
    dropped): two independently restated reference functions agree."""
    B, S, H, D = 1, 64, 2, 16
    g0 = torch.Generator().manual_seed(9)
    q, k, v = (torch.randn(B, S, H, D, generator=g0) for _ in range(3))
    mask = torch.tril(torch.ones(S, S, dtype=torch.bool)).reshape(1, 1, S, S)
    a, _ = O.ring_attention_inference_fwd(q, k, v, mask, 2, True)
    b = O.ring_attention(q, k, v, None, None, None, 2, True, kwargs(16, 16, 1))
    assert (a - b).abs().max() < 1e-5


# ----------------------------------------------------------------------------- frozen vectors

def test_oracle_reproduces_its_frozen_vectors():
    """tests/golden/oracle_vectors.npz holds outputs of this oracle frozen after it passed the checks above (the
    reference has no vectors): a change that moves them is caught here before it reaches the GPU comparisons."""
    from tests.golden_vectors import load
    cases = load()
    for name in ("ring2_causal_bias_segments", "one_device_causal_block4", "decode_cache_idx_70",
                 "ring2_causal_dropout"):
        c = cases[name]
        i, cfg = c["in"], c["cfg"]
        kw = kwargs(cfg["qc"], cfg["kc"], cfg["cbs"])
        if "drop_permille" in cfg:
            kw.update(deterministic=False, attn_pdrop=cfg["drop_permille"] / 1000.0, dropout_rng=cfg["seed"])
        out, res = O.ring_attention_fwd(i["q"], i["k"], i["v"], i.get("bias"), i.get("seg"), cfg.get("cache_idx"),
                                        cfg["n"], True, kw)
        assert torch.allclose(out, c["out"]["out"], rtol=1e-5, atol=1e-6), name
        if "do" in i:
            grads = O.ring_attention_bwd(cfg["n"], True, kw, res, i["do"])
            for nm, gr in zip(("dq", "dk", "dv"), grads):
                assert torch.allclose(gr, c["out"][nm], rtol=1e-5, atol=1e-6), (name, nm)
    c = cases["inference_ring2"]
    out, res = O.ring_attention_inference_fwd(c["in"]["q"], c["in"]["k"], c["in"]["v"], c["in"]["mask"], 2)
    assert torch.allclose(out, c["out"]["out"], rtol=1e-5, atol=1e-6)
    for nm, gr in zip(("dq", "dk", "dv"), O.ring_attention_inference_bwd(2, res, c["in"]["do"])):
        assert torch.allclose(gr.float(), c["out"][nm], rtol=1e-5, atol=1e-6), nm
    c = cases["ffn_chunk8"]
    x, w1, w2, w3 = (c["in"][n_].clone().requires_grad_(True) for n_ in ("x", "w1", "w2", "w3"))
    y = O.blockwise_feedforward(lambda h: O.swiglu(h, w1, w2, w3), x, 8)
    y.backward(c["in"]["dy"])
    for nm, t in dict(y=y, dx=x.grad, dw1=w1.grad, dw2=w2.grad, dw3=w3.grad).items():
        assert torch.allclose(t, c["out"][nm], rtol=1e-5, atol=1e-6), nm


# ----------------------------------------------------------------------------- steps either side of the path

@pytest.mark.parametrize("style", ["adjacent", "half"])
def test_rope_is_a_rotation_with_the_relative_position_property(style):
    g = torch.Generator().manual_seed(5)
    D = 32
    x, y = torch.randn(3, 1, 2, D, generator=g, dtype=F64), torch.randn(3, 1, 2, D, generator=g, dtype=F64)
    assert torch.equal(O.rope_rotate(x, 0, 10000.0, style), x)                                   # position 0: identity
    r = O.rope_rotate(x, 1234, 10000.0, style)
    assert torch.allclose(r.norm(dim=-1), x.norm(dim=-1), rtol=1e-12)                            # norms are kept
    twice = O.rope_rotate(O.rope_rotate(x, 100, 10000.0, style), 23, 10000.0, style)
    assert torch.allclose(twice, O.rope_rotate(x, 123, 10000.0, style), atol=1e-12)              # angles add
    d1 = (O.rope_rotate(x, 700, 10000.0, style) * O.rope_rotate(y, 650, 10000.0, style)).sum(-1)
    d2 = (O.rope_rotate(x, 50, 10000.0, style) * y).sum(-1)
    assert torch.allclose(d1, d2, atol=1e-10)                                                    # only p - p' matters
    # against complex multiplication by exp(i pos theta^(-2j/D)), an independent formulation
    j = torch.arange(D // 2, dtype=F64)
    w = torch.polar(torch.ones(D // 2, dtype=F64), 77.0 * 10000.0 ** (-2.0 * j / D))
    if style == "adjacent":
        z = torch.view_as_complex(x.reshape(*x.shape[:-1], D // 2, 2).contiguous()) * w
        ref = torch.view_as_real(z).reshape(x.shape)
    else:
        z = torch.complex(x[..., : D // 2], x[..., D // 2:]) * w
        ref = torch.cat((z.real, z.imag), dim=-1)
    assert torch.allclose(O.rope_rotate(x, 77, 10000.0, style), ref, atol=1e-12)


def test_rope_kv_append_writes_one_position():
    g = torch.Generator().manual_seed(6)
    B, L, H, D = 2, 9, 2, 8
    q, kn, vn = (torch.randn(B, 1, H, D, generator=g, dtype=F64) for _ in range(3))
    kc, vc = torch.randn(B, L, H, D, generator=g, dtype=F64), torch.randn(B, L, H, D, generator=g, dtype=F64)
    qr, kc2, vc2 = O.rope_kv_append(q, kn, vn, kc, vc, 4)
    keep = [i for i in range(L) if i != 4]
    assert torch.equal(kc2[:, keep], kc[:, keep]) and torch.equal(vc2[:, keep], vc[:, keep])
    assert torch.equal(vc2[:, 4], vn[:, 0]) and torch.equal(kc2[:, 4], O.rope_rotate(kn, 4)[:, 0])
    assert torch.equal(qr, O.rope_rotate(q, 4))
    q0, kc3, _ = O.rope_kv_append(q, kn, vn, kc, vc, 4, theta=None)
    assert torch.equal(q0, q) and torch.equal(kc3[:, 4], kn[:, 0])


def test_rmsnorm_residual_definition_invariances_and_gradient():
    g = torch.Generator().manual_seed(7)
    T, d = 5, 16
    x, r = torch.randn(T, d, generator=g, dtype=F64), torch.randn(T, d, generator=g, dtype=F64)
    w = torch.randn(d, generator=g, dtype=F64)
    y, n = O.rmsnorm_residual(x, r, w, eps=0.0)
    assert torch.equal(y, x + r)
    ones = torch.ones(d, dtype=F64)
    _, n1 = O.rmsnorm_residual(x, r, ones, eps=0.0)
    assert torch.allclose((n1 * n1).mean(-1), torch.ones(T, dtype=F64), rtol=1e-12)              # unit RMS
    assert torch.allclose(O.rmsnorm_residual(3.0 * x, 3.0 * r, w, eps=0.0)[1], n, rtol=1e-12)    # scale invariant
    for t in range(T):                                                                          # the definition, row by row
        row = (x + r)[t]
        assert torch.allclose(n[t], row / math.sqrt(float((row * row).sum()) / d) * w, rtol=1e-12)
    # the backward formula the kernels use, against autograd
    xx, ww = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    yy, nn_ = O.rmsnorm_residual(xx, r, ww, eps=1e-6)
    dn, dres = torch.randn(T, d, generator=g, dtype=F64), torch.randn(T, d, generator=g, dtype=F64)
    (nn_ * dn).sum().add((yy * dres).sum()).backward()
    rstd = torch.rsqrt((yy * yy).mean(-1, keepdim=True) + 1e-6).detach()
    yd = yy.detach()
    gw = dn * w
    dy = rstd * gw - yd * rstd ** 3 / d * (gw * yd).sum(-1, keepdim=True) + dres
    assert torch.allclose(xx.grad, dy, rtol=1e-10, atol=1e-12)
    assert torch.allclose(ww.grad, (dn * yd * rstd).sum(0), rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("n,qc,kc", [(1, 8, 8), (2, 8, 16), (4, 4, 4)])
def test_padding_mask_as_bias_equals_attention_over_the_real_keys(n, qc, kc):
    """A bias of finfo.min on padded keys (how a model passes its padding mask) must act as if those keys were not
    there at all, for every row that sees a real key: checked against a causal softmax in float64 over the real keys
    only, written here from the definition (keys sliced away, not masked), forward and - through autograd - backward.
    Rows that see padded keys only (left padding) take equal weights over the keys of the chunks that run."""
    B, S, H, D = 2, 64, 2, 8
    q, k, v = make(B, S, H, D, seed=11, dtype=torch.float32)
    keep = torch.ones(B, S, dtype=torch.bool)
    keep[0, 50:] = False                                     # right padding
    keep[1, :5] = False                                      # left padding
    bias = torch.where(keep, 0.0, torch.finfo(torch.float32).min).reshape(B, 1, 1, S)
    kw = kwargs(qc, kc, 1)
    g = torch.randn(B, S, H, D, generator=torch.Generator().manual_seed(12))
    g[1, :5] = 0                                             # no cotangent where no real key is seen
    out, res = O.ring_attention_fwd(q, k, v, bias, None, None, n, True, kw)
    dq, dk, dv = O.ring_attention_bwd(n, True, kw, res, g)
    qa, ka, va = (t.double().requires_grad_(True) for t in (q, k, v))
    ref = torch.zeros(B, S, H, D, dtype=F64)
    rows = []
    for b in range(B):
        real = torch.nonzero(keep[b]).flatten()
        for i in range(S):
            vis = real[real <= i]
            if vis.numel() == 0:
                continue
            w = torch.softmax(torch.einsum("hd,khd->hk", qa[b, i], ka[b, vis]) / D ** 0.5, dim=-1)
            rows.append((b, i, torch.einsum("hk,khd->hd", w, va[b, vis])))
    loss = 0.0
    for b, i, o in rows:
        ref[b, i] = o.detach()
        loss = loss + (o * g[b, i].double()).sum()
    loss.backward()
    seen = torch.zeros(B, S, dtype=torch.bool)
    for b, i, _ in rows:
        seen[b, i] = True
    assert int((~seen).sum()) == 5
    assert float((out.double() - ref)[seen].abs().max()) < 2e-6
    for a, r in ((dq, qa.grad), (dk, ka.grad), (dv, va.grad)):
        assert float((a.double() - r).abs().max()) < 2e-5
    assert float(dk[0, 50:].abs().max()) == 0.0 and float(dv[0, 50:].abs().max()) == 0.0
    # rows 0..4 of batch row 1: equal weights over the keys of the chunks that run for them (:138-144)
    assert torch.isfinite(out[1, :5]).all()
