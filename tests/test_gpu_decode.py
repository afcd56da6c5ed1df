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
