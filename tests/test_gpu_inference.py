"""Parity of ring_attention_inference (boolean-mask ring, ringattention_inference.py) on the HIP path
with the CPU oracle.  Tolerances: fp32 max-abs 1e-4, bf16 2e-2, rel-L2 1e-2 (tests/util.assert_close)."""
import pytest
import torch

import ringattention_amd as ra
from oracle import ringattention_oracle as O
from tests.util import assert_close, make_qkv

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _mask(shape, seed, p_keep=0.6, causal=False):
    g = torch.Generator().manual_seed(seed)
    m = torch.rand(shape, generator=g) < p_keep
    if causal:
        S = shape[-1]
        m = m & torch.tril(torch.ones(S, S, dtype=torch.bool))
    m[..., 0] = True
    return m


def _run(q, k, v, do, mask, n, f32_logits=True):
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    with ra.ring_axis("sp", n):
        out = ra.ringattention_inference(qd, kd, vd, mask.to(DEV), "sp", f32_logits)
    out.backward(do.to(DEV))
    return out.detach().cpu(), tuple(t.grad.cpu() for t in (qd, kd, vd))


CASES = [
    # B, S, H, D, n, mask shape kind, dtype
    (2, 128, 2, 64, 1, "full", torch.float32),
    (2, 128, 2, 64, 4, "full", torch.float32),
    (1, 192, 3, 32, 2, "bcast_bh", torch.float32),
    (2, 256, 2, 128, 2, "key_only", torch.float32),
    (1, 256, 2, 128, 4, "per_head", torch.bfloat16),
    (2, 512, 2, 128, 2, "full", torch.bfloat16),
]


@pytest.mark.parametrize("case", CASES)
def test_inference_matches_oracle(case):
    B, S, H, D, n, kind, dtype = case
    shape = {"full": (B, H, S, S), "bcast_bh": (1, 1, S, S), "key_only": (B, 1, 1, S), "per_head": (1, H, S, S)}[kind]
    q, k, v, do = make_qkv(B, S, H, D, dtype=dtype, seed=3, scale=D ** -0.25)
    mask = _mask(shape, 11, causal=(kind == "bcast_bh"))
    out, grads = _run(q, k, v, do, mask, n)
    ref_out, res = O.ring_attention_inference_fwd(q, k, v, mask, n, True)
    ref_grads = O.ring_attention_inference_bwd(n, res, do)
    assert_close(out, ref_out, dtype, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close(a, b, dtype, name)


def test_inference_fully_masked_row_and_ring_invariance():
    """A query row that attends to nothing gets the mean of V (equal finfo.min logits) and, as in the
    reference's backward formula, uniform weights in the gradients; the ring size changes nothing."""
    B, S, H, D = 1, 128, 2, 64
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.float32, seed=5)
    mask = _mask((1, 1, S, S), 13)
    mask[:, :, 7, :] = False
    ref_out, res = O.ring_attention_inference_fwd(q, k, v, mask, 4, True)
    ref_grads = O.ring_attention_inference_bwd(4, res, do)
    outs = {}
    for n in (1, 4):
        out, grads = _run(q, k, v, do, mask, n)
        assert torch.allclose(out[:, 7], v.mean(dim=1), atol=1e-5)
        assert_close(out, ref_out, torch.float32, "out")
        for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
            assert_close(a, b, torch.float32, name)
        outs[n] = out
    assert (outs[1] - outs[4]).abs().max() < 1e-5


def test_inference_causal_mask_equals_blockwise_ring_attention():
    """The same causal problem through both entry points of the library."""
    from tests.util import kwargs
    B, S, H, D = 1, 512, 2, 128
    q, k, v, _ = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=6, scale=D ** -0.25)
    mask = torch.tril(torch.ones(S, S, dtype=torch.bool)).reshape(1, 1, S, S)
    with ra.ring_axis("sp", 2):
        a = ra.ringattention_inference(q.to(DEV), k.to(DEV), v.to(DEV), mask.to(DEV), "sp", True)
        b = ra.ringattention(q.to(DEV), k.to(DEV), v.to(DEV), None, None, None, axis_name="sp",
                             float32_logits=True, blockwise_kwargs=kwargs(128, 128, 1))
    assert_close(a.cpu(), b.cpu(), torch.bfloat16, "out")


def test_inference_rejects_bad_mask_shapes():
    q = torch.zeros(1, 128, 2, 64, device=DEV)
    with ra.ring_axis("sp", 1):
        with pytest.raises(ValueError):
            ra.ringattention_inference(q, q, q, torch.ones(1, 1, 64, 128, dtype=torch.bool, device=DEV), "sp", True)
        with pytest.raises(ValueError):
            ra.ringattention_inference(q, q, q, torch.ones(128, 128, dtype=torch.bool, device=DEV), "sp", True)


def _structured_mask(B, H, S, kind, seed):
    """Masks with whole tiles kept / dropped (what the packed summary shortcuts) plus ragged edges."""
    g = torch.Generator().manual_seed(seed)
    causal = torch.tril(torch.ones(S, S, dtype=torch.bool))
    if kind == "causal":
        return causal.reshape(1, 1, S, S).clone()
    if kind == "causal_padding":
        m = causal.reshape(1, 1, S, S).repeat(B, 1, 1, 1)
        for b in range(B):
            m[b, :, :, S - 37 * (b + 1):] = False
        m[..., 0] = True
        return m
    if kind == "band_per_head":
        idx = torch.arange(S)
        m = torch.stack([(idx[:, None] - idx[None, :]).abs() <= 100 * (h + 1) for h in range(H)]).reshape(1, H, S, S)
        return m & (torch.rand(1, H, S, S, generator=g) < 0.97) | torch.eye(S, dtype=torch.bool)
    if kind == "key_only":
        m = torch.rand(B, 1, 1, S, generator=g) < 0.7
        m[..., 0] = True
        return m
    raise ValueError(kind)


MFMA_CASES = [
    # B, S, H, n, mask kind   (bf16, D = 128 or 64, shards of a multiple of 256 rows: the MFMA kernels run)
    (1, 512, 2, 1, "causal"),
    (1, 1024, 2, 2, "causal"),
    (2, 1024, 2, 2, "causal_padding"),
    (1, 1024, 3, 4, "band_per_head"),
    (2, 512, 2, 2, "key_only"),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("case", MFMA_CASES)
def test_inference_mfma_path_matches_oracle(case, D, dtype):
    """bf16 on the bf16 MFMA kernels, fp32 on the fp32 ones (both read the packed mask)."""
    B, S, H, n, kind = case
    q, k, v, do = make_qkv(B, S, H, D, dtype=dtype, seed=21, scale=D ** -0.25)
    mask = _structured_mask(B, H, S, kind, 22)
    out, grads = _run(q, k, v, do, mask, n)
    ref_out, res = O.ring_attention_inference_fwd(q, k, v, mask, n, True)
    ref_grads = O.ring_attention_inference_bwd(n, res, do)
    assert_close(out, ref_out, dtype, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close(a, b, dtype, name)


def test_inference_fp32_matrix_core_and_vector_kernels_agree():
    """fp32 inputs: the same call with the packed mask (fp32 matrix-core kernels) and without it (vector kernels),
    including a row that attends to nothing."""
    from ringattention_amd import ringattention_hip as rh
    B, S, H, D, n = 2, 1024, 2, 128, 2
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.float32, seed=27, scale=D ** -0.25)
    mask = _structured_mask(B, H, S, "causal_padding", 28)
    mask[:, :, 700, :] = False
    out, grads = _run(q, k, v, do, mask, n)
    orig = rh._MaskInputs.set_keep

    def no_pack(self, *a, **kw):
        orig(self, *a, **kw)
        self.keep_packed = None

    rh._MaskInputs.set_keep = no_pack
    try:
        out_g, grads_g = _run(q, k, v, do, mask, n)
    finally:
        rh._MaskInputs.set_keep = orig
    assert torch.allclose(out[:, 700], v.mean(dim=1), atol=1e-5)
    for name, a, b in zip(("out", "dq", "dk", "dv"), (out,) + grads, (out_g,) + grads_g):
        assert_close(a, b, torch.float32, name)
        assert float((a - b).abs().max()) <= 2e-5, name


def test_inference_mfma_path_with_a_row_that_attends_to_nothing():
    """Tile skipping is switched off by the host when a row has no attended key: that row must come out
    as the mean of V on the MFMA kernels too."""
    B, S, H, D, n = 1, 512, 2, 128, 2
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=23, scale=D ** -0.25)
    mask = _structured_mask(B, H, S, "causal", 24)
    mask[:, :, 300, :] = False
    out, grads = _run(q, k, v, do, mask, n)
    ref_out, res = O.ring_attention_inference_fwd(q, k, v, mask, n, True)
    ref_grads = O.ring_attention_inference_bwd(n, res, do)
    assert torch.allclose(out[:, 300].float(), v.float().mean(dim=1), atol=2e-2)
    assert_close(out, ref_out, torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close(a, b, torch.bfloat16, name)


def test_inference_mfma_and_generic_kernels_agree():
    """Same call with and without the packed mask (the latter forces the generic kernels)."""
    from ringattention_amd import inference as inf, ringattention_hip as rh
    B, S, H, D, n = 1, 1024, 2, 128, 2
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=25, scale=D ** -0.25)
    mask = _structured_mask(B, H, S, "causal_padding", 26)
    out, grads = _run(q, k, v, do, mask, n)
    orig = rh._MaskInputs.set_keep

    def unpacked(self, attn_mask, device, q_total, k_total):
        orig(self, attn_mask, device, q_total, k_total)
        self.keep_packed = None
    rh._MaskInputs.set_keep = unpacked
    try:
        out_g, grads_g = _run(q, k, v, do, mask, n)
    finally:
        rh._MaskInputs.set_keep = orig
    assert_close(out, out_g, torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, grads_g):
        assert_close(a, b, torch.bfloat16, name)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_inference_frozen_vectors(dtype):
    """The HIP path against tests/golden/oracle_vectors.npz (outputs of the CPU oracle, frozen)."""
    from tests.golden_vectors import load
    c = load()["inference_ring2"]
    i = c["in"]
    out, grads = _run(i["q"].to(dtype), i["k"].to(dtype), i["v"].to(dtype), i["do"].to(dtype), i["mask"], 2)
    assert_close(out, c["out"]["out"], dtype, "out")
    for name, a in zip(("dq", "dk", "dv"), grads):
        assert_close(a, c["out"][name], dtype, name)


def test_inference_mfma_path_is_bitwise_reproducible():
    B, S, H, D, n = 1, 8192, 8, 128, 2
    g = torch.Generator().manual_seed(21)
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=21, scale=D ** -0.25)
    mask = (torch.rand(1, 1, S, S, generator=g) < 0.7) & torch.tril(torch.ones(S, S, dtype=torch.bool))
    mask[..., 0] = True
    first = _run(q, k, v, do, mask, n)
    again = _run(q, k, v, do, mask, n)
    assert torch.equal(first[0], again[0])
    for a, b in zip(first[1], again[1]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("S,Sk,n,kind", [(1000, 1000, 1, "full"), (1000, 1000, 2, "per_head"), (900, 1024, 1, "full"),
                                         (1024, 1000, 2, "key_only"), (200, 1000, 1, "bcast_bh")])
def test_inference_lengths_off_the_128_grid_run_on_the_matrix_cores(S, Sk, n, kind, dtype):
    """A prompt of 1000 tokens: q, k, v and the mask are padded to the next multiple of 128 per device (positions mean
    nothing but what the mask says) and the result is cut back; against the oracle at the original lengths."""
    B, H, D = 2, 2, 128
    g = torch.Generator().manual_seed(S + Sk)
    q = (torch.randn(B, S, H, D, generator=g) * D ** -0.25).to(dtype)
    k = (torch.randn(B, Sk, H, D, generator=g) * D ** -0.25).to(dtype)
    v = torch.randn(B, Sk, H, D, generator=g).to(dtype)
    do = torch.randn(B, S, H, D, generator=g).to(dtype)
    shape = {"full": (B, H, S, Sk), "bcast_bh": (1, 1, S, Sk), "key_only": (B, 1, 1, Sk), "per_head": (1, H, S, Sk)}[kind]
    mask = torch.rand(shape, generator=g) < 0.5
    mask[..., 0] = True
    out, grads = _run(q, k, v, do, mask, n)
    fam = ra.kernel_family_of_last_call()
    assert "mfma" in fam["forward"] and "mfma" in fam["backward"], fam
    ref_out, res = O.ring_attention_inference_fwd(q, k, v, mask, n, True)
    ref_grads = O.ring_attention_inference_bwd(n, res, do)
    assert_close(out, ref_out, dtype, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close(a, b, dtype, name)
