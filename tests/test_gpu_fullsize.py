"""The hot path at the sizes its throughput is quoted on, checked through properties that do not need a CPU run
of that size (the oracle takes hours there): softmax rows sum to one, a virtual ring agrees with one device,
keys that are masked have bitwise no effect, the backward pass is linear in the cotangent, the chunked FFN agrees
with the unchunked one.  The oracle-against-HIP comparisons at sizes the oracle finishes in seconds are in the
other test_gpu_* files."""
import pytest
import torch

import ringattention_amd as ra
from tests.util import kwargs, packed_segment_ids

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _attn(q, k, v, bias, seg, n, kw, do=None):
    q, k, v = (t.detach().requires_grad_(do is not None) for t in (q, k, v))
    with ra.ring_axis("sp", n):
        out = ra.ringattention(q, k, v, bias, seg, None, axis_name="sp", float32_logits=True, blockwise_kwargs=kw)
        if do is None:
            return out, None
        out.backward(do)
    return out.detach(), (q.grad, k.grad, v.grad)


def _rel(a, b):
    a, b = a.detach().float(), b.detach().float()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def test_causal_32k_properties():
    """B1 H32 S32768 D128 bf16, causal, chunks 512/512 (the configuration of the headline figure)."""
    B, S, H, D = 1, 32768, 32, 128
    print("full size causal 32k", flush=True)
    g = torch.Generator(device=DEV).manual_seed(0)
    mk = lambda: (torch.randn(B, S, H, D, device=DEV, generator=g) * D ** -0.25).bfloat16()
    q, k, v = mk(), mk(), torch.randn(B, S, H, D, device=DEV, generator=g).bfloat16()
    do = torch.randn(B, S, H, D, device=DEV, generator=g).bfloat16()
    kw = kwargs(512, 512, 1)
    # rows of the softmax sum to one: with V = 1 every output element is 1 (bf16 rounding of P: 2^-8 relative)
    ones = torch.ones_like(v)
    out1, _ = _attn(q, k, ones, None, None, 1, kw)
    assert float((out1.float() - 1.0).abs().max()) <= 1e-2
    # one device, and a virtual ring of 8: the same result up to the order of the fp32 accumulation
    out, grads = _attn(q, k, v, None, None, 1, kw, do)
    out8, grads8 = _attn(q, k, v, None, None, 8, kw, do)
    assert not torch.isnan(out).any()
    assert float((out.float() - out8.float()).abs().max()) <= 2e-2 and _rel(out8, out) <= 1e-2
    for name, a, b in zip(("dq", "dk", "dv"), grads8, grads):
        assert _rel(a, b) <= 1e-2, name
    # causality, bitwise: keys and values after position p have no effect on the rows up to p
    p = 20000
    k2, v2 = k.clone(), v.clone()
    k2[:, p + 1:] = 3.0
    v2[:, p + 1:] = -7.0
    out_p, _ = _attn(q, k2, v2, None, None, 1, kw)
    assert torch.equal(out_p[:, :p + 1], out[:, :p + 1])
    # the backward pass is linear in the cotangent
    _, g2 = _attn(q, k, v, None, None, 1, kw, (2.0 * do.float()).bfloat16())
    for name, a, b in zip(("dq", "dk", "dv"), g2, grads):
        assert _rel(a, 2.0 * b.float()) <= 1e-2, name


def test_packed_documents_131k_ring8_properties():
    """B1 H32 S131072 D128 bf16 as 8 virtual shards of 16384 with document ids and an additive bias."""
    B, S, H, D, n = 1, 131072, 32, 128, 8
    print("full size ring 131k", flush=True)
    g = torch.Generator(device=DEV).manual_seed(1)
    mk = lambda: (torch.randn(B, S, H, D, device=DEV, generator=g) * D ** -0.25).bfloat16()
    q, k, v = mk(), mk(), torch.randn(B, S, H, D, device=DEV, generator=g).bfloat16()
    seg = packed_segment_ids(1, S, 4096, seed=2).to(DEV)
    bias = torch.randn(1, 1, 1, S, device=DEV, generator=g)
    kw = kwargs(512, 512, 1)
    out, _ = _attn(q, k, v, bias, seg, n, kw)
    assert not torch.isnan(out).any()
    # rows sum to one under the document mask too
    out1, _ = _attn(q, k, torch.ones_like(v), bias, seg, n, kw)
    assert float((out1.float() - 1.0).abs().max()) <= 1e-2
    # documents are isolated bitwise: changing the keys and values of one document changes no other document's rows
    ids = seg[0]
    doc = int(ids[S // 2])
    inside = ids == doc
    k2, v2 = k.clone(), v.clone()
    k2[:, inside] = 2.0
    v2[:, inside] = 5.0
    out2, _ = _attn(q, k2, v2, bias, seg, n, kw)
    assert torch.equal(out2[:, ~inside], out[:, ~inside])
    assert not torch.equal(out2[:, inside], out[:, inside])


def test_decode_long_cache_properties():
    """One query token against a cache of 262144 positions (B2 H32 D128 bf16, key chunks of 512)."""
    B, L, H, D, kc = 2, 262144 + 512, 32, 128, 512
    print("full size decode", flush=True)
    g = torch.Generator(device=DEV).manual_seed(3)
    q = torch.randn(B, 1, H, D, device=DEV, generator=g).bfloat16()
    k = torch.randn(B, L, H, D, device=DEV, generator=g).bfloat16()
    v = torch.randn(B, L, H, D, device=DEV, generator=g).bfloat16()
    kw = kwargs(1, kc, 1)
    cache_idx = 262144 + 100
    ci = torch.tensor(cache_idx, dtype=torch.int32, device=DEV)
    out = ra.ringattention(q, k, v, None, None, ci, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    assert not torch.isnan(out).any()
    out1 = ra.ringattention(q, k, torch.ones_like(v), None, None, ci, axis_name=None, float32_logits=True,
                            blockwise_kwargs=kw)
    assert float((out1.float() - 1.0).abs().max()) <= 1e-2
    # positions after cache_idx are not attended to: bitwise
    k2, v2 = k.clone(), v.clone()
    k2[:, cache_idx + 1:] = 4.0
    v2[:, cache_idx + 1:] = -9.0
    out2 = ra.ringattention(q, k2, v2, None, None, ci, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    assert torch.equal(out2, out)
    # against a dense fp32 softmax over the attended positions, computed here in slabs
    scores = torch.einsum("bqhd,bkhd->bhqk", q.float(), k[:, :cache_idx + 1].float()) / D ** 0.5
    ref = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(scores, dim=-1), v[:, :cache_idx + 1].float())
    assert float((out.float() - ref).abs().max()) <= 2e-2 and _rel(out, ref) <= 1e-2


def test_ffn_65k_tokens_chunked_equals_unchunked():
    """SwiGLU 4096 -> 11008 over 65536 tokens: blockwise in chunks of 2048 against one call over all tokens."""
    T, d, f, chunk = 65536, 4096, 11008, 2048
    print("full size ffn", flush=True)
    g = torch.Generator(device=DEV).manual_seed(4)
    ff = ra.SwiGLU(d, f, device=DEV)
    x = torch.randn(1, T, d, device=DEV, generator=g).bfloat16()
    dy = torch.randn(1, T, d, device=DEV, generator=g).bfloat16()

    def run(fn):
        xx = x.detach().requires_grad_(True)
        for p in ff.parameters():
            p.grad = None
        y = fn(xx)
        y.backward(dy)
        return y.detach(), xx.grad, [p.grad.clone() for p in ff.parameters()]

    y_b, dx_b, dw_b = run(lambda t: ra.blockwise_feedforward(ff, t, chunk))
    y_2, dx_2, dw_2 = run(lambda t: ra.blockwise_feedforward(ff, t, chunk))
    assert torch.equal(y_b, y_2) and torch.equal(dx_b, dx_2)          # same inputs, same bits
    for a, b in zip(dw_b, dw_2):
        assert torch.equal(a, b)
    y_u, dx_u, dw_u = run(lambda t: ff(t))
    assert not torch.isnan(y_b).any()
    assert _rel(y_b, y_u) <= 1e-3 and _rel(dx_b, dx_u) <= 1e-3
    for a, b in zip(dw_b, dw_u):
        assert _rel(a, b) <= 1e-2
    # tokens are independent: the first chunk alone gives the same rows
    y_c = ff(x[:, :chunk])
    assert _rel(y_c, y_b[:, :chunk]) <= 1e-3


def test_forward_and_backward_are_bitwise_reproducible():
    """Same inputs, same bits: no kernel adds in an order that depends on timing (no atomics), so a difference
    between two runs can only come from a wavefront reading a tile another one is still writing."""
    B, S, H, D = 1, 32768, 8, 128
    g = torch.Generator(device=DEV).manual_seed(5)
    mk = lambda: (torch.randn(B, S, H, D, device=DEV, generator=g) * D ** -0.25).bfloat16()
    q, k, v = mk(), mk(), torch.randn(B, S, H, D, device=DEV, generator=g).bfloat16()
    do = torch.randn(B, S, H, D, device=DEV, generator=g).bfloat16()
    seg = packed_segment_ids(1, S, 3000, seed=6).to(DEV)
    bias = torch.randn(1, 1, 1, S, device=DEV, generator=g)
    for name, b_, s_, n in (("causal", None, None, 1), ("causal ring 4", None, None, 4), ("documents + bias", bias, seg, 2)):
        print("reproducible", name, flush=True)
        kw = kwargs(512, 512, 1)
        first = _attn(q, k, v, b_, s_, n, kw, do)
        for _ in range(2):
            again = _attn(q, k, v, b_, s_, n, kw, do)
            assert torch.equal(torch.nan_to_num(first[0]), torch.nan_to_num(again[0])), name + " out"
            for nm, a, b2 in zip(("dq", "dk", "dv"), again[1], first[1]):
                assert torch.equal(a, b2), name + " " + nm
