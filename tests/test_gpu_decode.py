"""Parity of the decode kernel (cache_idx path) with the CPU oracle, including the skip predicate's
edge at cache_idx % key_chunk_size == 0 and the all-NaN row at cache_idx == 0."""
import pytest
import torch

import ringattention_amd as ra
from oracle import ringattention_oracle as O
from tests.util import assert_close, errors, kwargs, make_qkv, oracle_kwargs, packed_segment_ids

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cache_idx", [0, 1, 63, 64, 65, 200, 511, 512, 700])
def test_decode_matches_oracle(cache_idx, dtype):
    B, L, H, D, kc = 2, 768, 4, 128, 64
    print("decode case", cache_idx, dtype, flush=True)
    q, k, v, _ = make_qkv(B, 1, H, D, dtype=dtype, seed=cache_idx, Skv=L)
    kw = kwargs(1, kc, 1)
    ref = O.ring_attention(q, k, v, None, None, cache_idx, 1, True, oracle_kwargs(kw))
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    out = ra.ringattention(qd, kd, vd, None, None, cache_idx, axis_name=None, float32_logits=True,
                           blockwise_kwargs=kw)
    assert_close(out, ref, dtype, "decode host cache_idx")
    ci = torch.tensor(cache_idx, dtype=torch.int32, device=DEV)
    out2 = ra.ringattention(qd, kd, vd, None, None, ci, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    assert torch.equal(torch.nan_to_num(out), torch.nan_to_num(out2))


def test_decode_with_bias_segments_and_heads_not_filling_a_group():
    B, L, H, D, kc = 3, 512, 5, 64, 32
    cache_idx = 300
    q, k, v, _ = make_qkv(B, 1, H, D, dtype=torch.float32, seed=2, Skv=L)
    g = torch.Generator().manual_seed(3)
    bias = torch.randn(B, 1, 1, L, generator=g)
    seg = packed_segment_ids(B, L, 120, seed=5)
    kw = kwargs(1, kc, 1)
    ref = O.ring_attention(q, k, v, bias, seg, cache_idx, 1, True, oracle_kwargs(kw))
    out = ra.decode_attention(q.to(DEV), k.to(DEV), v.to(DEV), bias.to(DEV), seg.to(DEV), cache_idx, kw)
    assert_close(out, ref, torch.float32, "decode bias+seg")


def test_decode_equals_generic_blockwise_path():
    """The same call through the blockwise kernels (autograd on) and through the decode kernel."""
    B, L, H, D, kc = 2, 512, 2, 128, 64
    q, k, v, _ = make_qkv(B, 1, H, D, dtype=torch.float32, seed=4, Skv=L)
    kw = kwargs(1, kc, 1, impl="generic")
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    fast = ra.ringattention(qd, kd, vd, None, None, 333, None, True, kw)
    slow = ra.ringattention(qd.clone().requires_grad_(True), kd, vd, None, None, 333, None, True, kw)
    assert errors(fast, slow)[0] < 1e-5


def test_decode_split_counts_agree():
    B, L, H, D, kc = 1, 2048, 2, 128, 128
    q, k, v, _ = make_qkv(B, 1, H, D, dtype=torch.bfloat16, seed=6, Skv=L)
    kw = kwargs(1, kc, 1)
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    outs = [ra.decode_attention(qd, kd, vd, None, None, 1999, kw, num_splits=ns).float() for ns in (1, 3, 8, 64)]
    for o in outs[1:]:
        assert errors(o, outs[0])[0] < 1e-2


@pytest.mark.parametrize("n", [2, 4, 8])
@pytest.mark.parametrize("cache_idx", [65535, 40000, 8192])
def test_ring_sharded_decode_matches_oracle(n, cache_idx):
    """cache_idx with an axis size above one (ringattention_jax.py:31-37): one query token per virtual device, the
    cache of 65536 positions sharded over the ring; every shard goes through the streaming kernel with a carry.
    8192 is the edge at which the query's own key chunk does not run (:324-331) and, on rings of 8, a shard start."""
    B, L, H, D, kc = 1, 65536, 4, 128, 512
    print("ring decode", n, cache_idx, flush=True)
    q, k, v, _ = make_qkv(B, n, H, D, dtype=torch.bfloat16, seed=n, Skv=L, scale=D ** -0.25)
    g = torch.Generator().manual_seed(11)
    bias = torch.randn(B, 1, 1, L, generator=g)
    seg = packed_segment_ids(B, L, 20000, seed=12)
    kw = kwargs(1, kc, 1)
    ref = O.ring_attention(q, k, v, bias, seg, cache_idx, n, True, oracle_kwargs(kw))
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    with ra.ring_axis("sp", n):
        out = ra.ringattention(qd, kd, vd, bias.to(DEV), seg.to(DEV), cache_idx, axis_name="sp", float32_logits=True,
                               blockwise_kwargs=kw)
        # the same call through the blockwise kernels (wanting gradients keeps it off the streaming kernel)
        slow = ra.ringattention(qd.clone().requires_grad_(True), kd, vd, bias.to(DEV), seg.to(DEV), cache_idx,
                                axis_name="sp", float32_logits=True, blockwise_kwargs=kw)
    assert_close(out, ref, torch.bfloat16, "ring decode")
    assert errors(out, slow)[0] <= 2e-2


def test_ring_sharded_decode_position_zero_is_nan_everywhere():
    n, B, L, H, D, kc = 4, 1, 2048, 2, 64, 128
    q, k, v, _ = make_qkv(B, n, H, D, dtype=torch.float32, seed=1, Skv=L)
    kw = kwargs(1, kc, 1)
    ref = O.ring_attention(q, k, v, None, None, 0, n, True, oracle_kwargs(kw))
    with ra.ring_axis("sp", n):
        out = ra.ringattention(q.to(DEV), k.to(DEV), v.to(DEV), None, None, 0, axis_name="sp", float32_logits=True,
                               blockwise_kwargs=kw)
    assert torch.isnan(ref).all() and torch.isnan(out).all()


def test_decode_carry_of_one_step_equals_the_plain_call_bitwise():
    """A ring of one through the carry form: numerator / denominator of the single step is the plain result."""
    B, L, H, D, kc = 2, 4096, 4, 128, 256
    q, k, v, _ = make_qkv(B, 1, H, D, dtype=torch.bfloat16, seed=9, Skv=L)
    kw = kwargs(1, kc, 1)
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    plain = ra.decode_attention(qd, kd, vd, None, None, 3000, kw)
    num = torch.empty((B, 1, H, D), dtype=torch.float32, device=DEV)
    den = torch.empty((B, H, 1), dtype=torch.float32, device=DEV)
    mx = torch.empty((B, H, 1), dtype=torch.float32, device=DEV)
    out = ra.decode_attention(qd, kd, vd, None, None, 3000, kw, carry=(num, den, mx), carry_is_initial=True)
    assert torch.equal(plain, out)
    assert torch.equal((num / den.reshape(B, 1, H, 1)).to(torch.bfloat16), plain)


def test_default_workspace_is_sized_for_the_automatic_split_count():
    from ringattention_amd import _lib
    from ringattention_amd.decode import decode_workspace
    B, L, H, D = 4, 8192, 32, 128
    q = torch.empty((B, 1, H, D), dtype=torch.bfloat16, device=DEV)
    k = torch.empty((B, L, H, D), dtype=torch.bfloat16, device=DEV)
    ns = _lib.load().ra_decode_auto_splits(B, L, H, D, _lib.RA_BF16)
    assert 1 <= ns <= 256
    assert decode_workspace(q, k).numel() == B * H * ns * (D + 2) * 4
    assert decode_workspace(q, k).numel() < _lib.load().ra_decode_workspace_bytes(B, L, H, D, 0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("cache_idx", [5, 63, 64, 700])
def test_decode_does_not_read_cache_slots_behind_the_query(cache_idx, dtype):
    """A cache allocated with torch.empty holds anything behind the last token written, NaN included.  Those keys are
    masked and weigh 0, but 0 * NaN is NaN: the streaming kernel neither looks at a masked key's logit nor multiplies a
    value by a weight of 0 there, so the result is that of the zero-filled cache, bit for bit."""
    B, L, H, D, kc = 2, 1024, 4, 128, 64
    q, k, v, _ = make_qkv(B, 1, H, D, dtype=dtype, seed=cache_idx, Skv=L)
    kw = kwargs(1, kc, 1)
    kz, vz = k.clone(), v.clone()
    kz[:, cache_idx + 1:] = 0
    vz[:, cache_idx + 1:] = 0
    kn, vn = kz.clone(), vz.clone()
    kn[:, cache_idx + 1:] = float("nan")
    vn[:, cache_idx + 1:] = float("inf")
    clean = ra.ringattention(q.to(DEV), kz.to(DEV), vz.to(DEV), None, None, cache_idx, None, True, kw)
    dirty = ra.ringattention(q.to(DEV), kn.to(DEV), vn.to(DEV), None, None, cache_idx, None, True, kw)
    assert torch.isfinite(dirty).all() and torch.equal(clean, dirty)
    ref = O.ring_attention(q, kz, vz, None, None, cache_idx, 1, True, oracle_kwargs(kw))
    assert_close(dirty, ref, dtype, "decode over a dirty cache")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [32, 40, 80, 96, 112, 160, 192, 256])
@pytest.mark.parametrize("n", [1, 2])
def test_decode_head_sizes(D, dtype, n):
    """The streaming kernel at the other head sizes it is built for - among them those whose elements take a number of
    lanes that is no power of two (96: 12 of a group of 16) -, alone and as a ring of 2."""
    B, L, H, kc, cache_idx = 2, 2048, 3, 128, 1500
    q, k, v, _ = make_qkv(B, n, H, D, dtype=dtype, seed=D + n, Skv=L)
    g = torch.Generator().manual_seed(D)
    bias = torch.randn(B, 1, 1, L, generator=g)
    seg = packed_segment_ids(B, L, 900, seed=D)
    kw = kwargs(1, kc, 1)
    ref = O.ring_attention(q, k, v, bias, seg, cache_idx, n, True, oracle_kwargs(kw))
    with ra.ring_axis("sp", n):
        out = ra.ringattention(q.to(DEV), k.to(DEV), v.to(DEV), bias.to(DEV), seg.to(DEV), cache_idx, axis_name="sp",
                               float32_logits=True, blockwise_kwargs=kw)
        slow = ra.ringattention(q.to(DEV).requires_grad_(True), k.to(DEV), v.to(DEV), bias.to(DEV), seg.to(DEV),
                                cache_idx, axis_name="sp", float32_logits=True, blockwise_kwargs=kw)
    assert_close(out, ref, dtype, "decode D %d" % D)
    assert errors(out, slow)[0] <= (2e-2 if dtype == torch.bfloat16 else 1e-5)
