"""Parity of the HIP attention path (through the C-ABI) with the CPU oracle.

Bar: forward output and dq/dk/dv within max-abs 1e-4 (fp32 inputs) or 2e-2 (bf16 inputs) and
relative L2 <= 1e-2; NaN rows (no tile runs) must coincide; masked keys must have bitwise no effect.
"""
import pytest
import torch

import ringattention_amd as ra
from tests.util import (assert_close, errors, kwargs, make_qkv, oracle_fwd_bwd, packed_segment_ids)

pytestmark = pytest.mark.gpu
DEV = "cuda"


def run_hip(q, k, v, do, bias, seg, cache_idx, n, kw, name="sp"):
    qd, kd, vd = (t.to(DEV).requires_grad_(do is not None) for t in (q, k, v))
    bd = bias.to(DEV) if bias is not None else None
    sd = seg.to(DEV) if seg is not None else None
    with ra.ring_axis(name, n):
        out = ra.ringattention(qd, kd, vd, bd, sd, cache_idx, axis_name=name, float32_logits=True,
                               blockwise_kwargs=kw)
        grads = None
        if do is not None:
            out.backward(do.to(DEV))
            grads = (qd.grad, kd.grad, vd.grad)
    torch.cuda.synchronize()
    return out, grads


def check_case(B, S, H, D, qc, kc, cbs, n, use_bias, use_seg, dtype, impl="auto", seed=0, bwd=True,
               seg_mean=None, bias_heads=False):
    print("case", dict(B=B, S=S, H=H, D=D, qc=qc, kc=kc, cbs=cbs, n=n, bias=use_bias, seg=use_seg,
                       dtype=str(dtype), impl=impl), flush=True)
    q, k, v, do = make_qkv(B, S, H, D, dtype=dtype, seed=seed, scale=1.0)
    g = torch.Generator().manual_seed(seed + 100)
    bias = torch.randn(B, H if bias_heads else 1, 1, S, generator=g) if use_bias else None
    seg = packed_segment_ids(B, S, seg_mean or max(4, S // 6), seed=seed + 7) if use_seg else None
    kw = kwargs(qc, kc, cbs, dtype=torch.float32, impl=impl)
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do if bwd else None, bias, seg, None, n, kw)
    out, grads = run_hip(q, k, v, do if bwd else None, bias, seg, None, n, kw)
    assert out.dtype == dtype and out.shape == q.shape
    assert_close(out, ref_out, dtype, "out")
    if bwd:
        for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
            assert a.dtype == dtype
            assert_close(a, b, dtype, name)


# --- B1 H8 S2048 D64 fp32, chunks 512 / 512: the case the reference itself can run on a CPU
def test_config1_fp32_fwd_bwd():
    B, S, H, D = 1, 2048, 8, 64
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.float32, seed=0)
    bias = torch.zeros(1, 1, 1, S)
    seg = torch.zeros(1, S, dtype=torch.int32)
    kw = kwargs(512, 512, 1, dtype=torch.float32)
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, 1, kw)
    out, grads = run_hip(q, k, v, do, bias, seg, None, 1, kw)
    assert_close(out, ref_out, torch.float32, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close(a, b, torch.float32, name)


GENERIC_CASES = [
    # B, S, H, D, qc, kc, cbs, n, bias, seg, dtype
    (2, 128, 2, 32, 32, 32, 1, 1, False, False, torch.float32),
    (2, 128, 2, 32, 32, 32, 1, 2, True, True, torch.float32),
    (1, 192, 3, 64, 16, 32, 1, 3, True, True, torch.float32),
    (1, 256, 2, 64, 64, 16, 1, 4, True, False, torch.float32),
    (1, 256, 2, 64, 32, 32, 8, 2, False, True, torch.float32),
    (1, 256, 2, 64, 8, 8, 32, 2, True, True, torch.float32),
    (1, 128, 2, 64, 32, 32, None, 2, True, True, torch.float32),
    (1, 128, 2, 64, 32, 32, None, 1, False, False, torch.float32),
    (1, 200, 1, 32, 20, 10, 1, 2, False, False, torch.float32),
    (1, 256, 2, 128, 64, 64, 1, 2, True, True, torch.float32),
    (2, 256, 4, 128, 64, 64, 1, 2, True, True, torch.bfloat16),
    (1, 256, 2, 64, 32, 64, 1, 1, False, True, torch.bfloat16),
    (1, 128, 2, 32, 2, 2, 1, 1, False, False, torch.float32),
]


@pytest.mark.parametrize("case", GENERIC_CASES)
def test_generic_kernels_match_oracle(case):
    B, S, H, D, qc, kc, cbs, n, use_bias, use_seg, dtype = case
    check_case(B, S, H, D, qc, kc, cbs, n, use_bias, use_seg, dtype, impl="generic")


def test_bias_per_head_and_batch():
    check_case(2, 128, 3, 32, 32, 32, 1, 2, True, True, torch.float32, impl="generic", bias_heads=True)


def test_ring_sizes_agree_with_single_device():
    B, S, H, D = 1, 512, 2, 64
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.float32, seed=3)
    seg = packed_segment_ids(B, S, 100, seed=4)
    kw = kwargs(32, 32, 1, impl="generic")
    base, gb = run_hip(q, k, v, do, None, seg, None, 1, kw)
    for n in (2, 4, 8):
        o, gg = run_hip(q, k, v, do, None, seg, None, n, kw)
        assert errors(o, base)[0] < 2e-6
        for a, b in zip(gg, gb):
            assert errors(a, b)[0] < 2e-5


def test_masked_keys_are_bitwise_isolated():
    B, S, H, D = 1, 256, 2, 64
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.float32, seed=5)
    kw = kwargs(32, 32, 1, impl="generic")
    a, ga = run_hip(q, k, v, do, None, None, None, 2, kw)
    k2, v2 = k.clone(), v.clone()
    k2[:, 150:] += 50.0
    v2[:, 150:] -= 20.0
    do2 = do.clone()
    do2[:, 150:] = 0.0
    b, gb = run_hip(q, k2, v2, do, None, None, None, 2, kw)
    assert torch.equal(a[:, :150], b[:, :150])
    # with no cotangent on rows >= 150, keys >= 150 get exactly zero gradient and dq rows < 150 do not move
    c, gc = run_hip(q, k, v, do2, None, None, None, 2, kw)
    d, gd = run_hip(q, k2, v2, do2, None, None, None, 2, kw)
    assert torch.equal(gc[0][:, :150], gd[0][:, :150])
    assert float(gd[1][:, 150:].abs().max()) == 0.0 and float(gd[2][:, 150:].abs().max()) == 0.0


def test_blockwise_fwd_carry_roundtrip_matches_oracle():
    """_blockwise_attention_fwd called step by step with an explicit carry, like the ring does."""
    from oracle import ringattention_oracle as O
    B, S, H, D = 1, 128, 2, 32
    q, k, v, _ = make_qkv(B, S, H, D, seed=9)
    kw = kwargs(16, 16, 1)
    okw = {kk: vv for kk, vv in kw.items()}
    num = torch.zeros(B, 64, H, D)
    den = torch.zeros(B, H, 64)
    mx = torch.full((B, H, 64), float("-inf"))
    # device 1 of a ring of 2: its own shard (step 0), then shard 0 (step 1)
    ref = (num, den, mx)
    ref = O.blockwise_attention_fwd(q[:, 64:], k[:, 64:], v[:, 64:], ref, 4, 4, None, None, **okw)
    ref = O.blockwise_attention_fwd(q[:, 64:], k[:, :64], v[:, :64], ref, 4, 0, None, None, **okw)
    carry = tuple(t.to(DEV) for t in (num, den, mx))
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    ra._blockwise_attention_fwd(qd[:, 64:], kd[:, 64:], vd[:, 64:], carry, 4, 4, None, None, impl="generic", **kw)
    ra._blockwise_attention_fwd(qd[:, 64:], kd[:, :64], vd[:, :64], carry, 4, 0, None, None, impl="generic", **kw)
    torch.cuda.synchronize()
    for a, b, name in zip(carry, ref, ("numerator", "denominator", "max_score")):
        assert errors(a, b)[0] < 1e-4, name


def test_invalid_shapes_raise():
    q = torch.zeros(1, 100, 1, 64, device=DEV)
    with pytest.raises(ValueError):
        ra.ringattention(q, q, q, None, None, None, "sp", True, kwargs(32, 32, 1))
    q = torch.zeros(1, 64, 1, 272, device=DEV)       # head sizes above 256: no kernel family
    with pytest.raises(NotImplementedError):
        ra.ringattention(q, q, q, None, None, None, "sp", True, kwargs(32, 32, 1))
    q = torch.zeros(1, 64, 1, 48, device=DEV)        # any head size up to 256 runs (zero-padded to one a kernel tiles)
    assert ra.ringattention(q, q, q, None, None, None, "sp", True, kwargs(32, 32, 1)).shape == q.shape


# --------------------------------------------------------------------------- MFMA kernels (bf16, D = 128 or 64)
MFMA_FWD_CASES = [
    # B, S, H, qc, kc, cbs, n, bias, seg
    (1, 256, 1, 128, 64, 1, 1, False, False),
    (1, 512, 2, 128, 128, 1, 1, False, False),
    (2, 512, 2, 256, 128, 1, 2, True, True),
    (1, 1024, 2, 128, 64, 1, 4, False, True),
    (1, 1024, 1, 256, 256, 1, 1, True, False),
    (1, 512, 2, 128, 128, None, 2, True, True),
    (1, 512, 2, 128, 128, None, 1, False, False),
    (1, 1024, 1, 128, 128, 256, 2, False, False),
    (1, 1024, 1, 128, 64, 32, 1, False, True),
    (1, 2048, 2, 512, 512, 1, 2, False, True),
]


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("case", MFMA_FWD_CASES)
def test_mfma_forward_matches_oracle(case, D):
    B, S, H, qc, kc, cbs, n, use_bias, use_seg = case
    check_case(B, S, H, D, qc, kc, cbs, n, use_bias, use_seg, torch.bfloat16, impl="mfma", bwd=False,
               seg_mean=S // 5)


def test_mfma_forward_matches_generic_kernels_at_4k():
    """Beyond what the CPU oracle does quickly: the two kernel families against each other."""
    B, S, H, D = 1, 4096, 4, 128
    q, k, v, _ = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=11, scale=D ** -0.25)
    seg = packed_segment_ids(B, S, 700, seed=12)
    g = torch.Generator().manual_seed(13)
    bias = torch.randn(B, 1, 1, S, generator=g)
    outs = {}
    for impl in ("generic", "mfma"):
        outs[impl], _ = run_hip(q, k, v, None, bias, seg, None, 4, kwargs(512, 512, 1, impl=impl))
    assert_close(outs["mfma"], outs["generic"], torch.bfloat16, "mfma vs generic")


def test_mfma_skip_masked_tiles_flag_is_exact_here():
    B, S, H, D = 1, 1024, 2, 128
    q, k, v, _ = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=14)
    a, _ = run_hip(q, k, v, None, None, None, None, 2, kwargs(256, 256, 1, impl="mfma", skip_masked_tiles=True))
    b, _ = run_hip(q, k, v, None, None, None, None, 2, kwargs(256, 256, 1, impl="mfma", skip_masked_tiles=False))
    assert torch.equal(a, b)


MFMA_BWD_CASES = [
    # B, S, H, qc, kc, cbs, n, bias, seg
    (1, 256, 1, 128, 128, 1, 1, False, False),
    (1, 512, 2, 128, 128, 1, 1, False, False),
    (2, 512, 2, 256, 128, 1, 2, True, True),
    (1, 1024, 2, 128, 128, 1, 4, False, True),
    (1, 1024, 1, 256, 256, 1, 1, True, False),
    (1, 512, 2, 128, 128, None, 2, True, True),
    (1, 512, 2, 128, 128, None, 1, False, False),
    (1, 1024, 1, 128, 128, 256, 2, False, False),
    (1, 1024, 1, 128, 128, 32, 1, False, True),
    (1, 2048, 2, 512, 512, 1, 2, False, True),
]


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("case", MFMA_BWD_CASES)
def test_mfma_backward_matches_oracle(case, D):
    B, S, H, qc, kc, cbs, n, use_bias, use_seg = case
    check_case(B, S, H, D, qc, kc, cbs, n, use_bias, use_seg, torch.bfloat16, impl="mfma", bwd=True,
               seg_mean=S // 5)


@pytest.mark.parametrize("D", [128, 64])
def test_mfma_backward_matches_generic_kernels_at_4k(D):
    B, S, H = 1, 4096, 2
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=21, scale=D ** -0.25)
    seg = packed_segment_ids(B, S, 700, seed=22)
    res = {}
    for impl in ("generic", "mfma"):
        res[impl] = run_hip(q, k, v, do, None, seg, None, 2, kwargs(512, 512, 1, impl=impl))
    assert_close(res["mfma"][0], res["generic"][0], torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), res["mfma"][1], res["generic"][1]):
        assert_close(a, b, torch.bfloat16, name)


def test_mfma_segment_tile_skipping_matches_generic_for_unsorted_ids():
    """Segment ids that are not sorted (the same id reappears): the tile hull is conservative there."""
    B, S, H, D = 1, 2048, 2, 128
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=31, scale=D ** -0.25)
    seg = (torch.arange(S) // 192 % 3).to(torch.int32).reshape(1, S)
    res = {}
    for impl in ("generic", "mfma"):
        res[impl] = run_hip(q, k, v, do, None, seg, None, 2, kwargs(256, 128, 1, impl=impl))
    assert_close(res["mfma"][0], res["generic"][0], torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), res["mfma"][1], res["generic"][1]):
        assert_close(a, b, torch.bfloat16, name)


def test_mfma_packed_documents_with_bias_ring8():
    """A small version of the packed-document ring workload: 8 virtual shards, geometric document
    lengths, additive bias; the MFMA path (tile skipping on) against the oracle."""
    B, S, H, D = 1, 4096, 2, 128
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=41, scale=D ** -0.25)
    seg = packed_segment_ids(B, S, 300, seed=42)
    g = torch.Generator().manual_seed(43)
    bias = torch.randn(1, 1, 1, S, generator=g)
    kw = kwargs(256, 256, 1, impl="mfma")
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, 8, kw)
    out, grads = run_hip(q, k, v, do, bias, seg, None, 8, kw)
    assert_close(out, ref_out, torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close(a, b, torch.bfloat16, name)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_frozen_vectors(dtype):
    """The HIP path against tests/golden/oracle_vectors.npz (outputs of the CPU oracle, frozen; inputs are
    bf16-representable, so both dtypes see the same numbers)."""
    from tests.golden_vectors import load
    cases = load()
    for name in ("ring2_causal_bias_segments", "one_device_causal_block4", "decode_cache_idx_70",
                 "ring2_causal_dropout"):
        c = cases[name]
        i, cfg = c["in"], c["cfg"]
        print("frozen", name, dtype, flush=True)
        kw = kwargs(cfg["qc"], cfg["kc"], cfg["cbs"])
        if "drop_permille" in cfg:
            kw.update(deterministic=False, attn_pdrop=cfg["drop_permille"] / 1000.0, dropout_rng=cfg["seed"])
        do = i["do"].to(dtype) if "do" in i else None
        out, grads = run_hip(i["q"].to(dtype), i["k"].to(dtype), i["v"].to(dtype), do, i.get("bias"), i.get("seg"),
                             cfg.get("cache_idx"), cfg["n"], kw)
        assert_close(out, c["out"]["out"], dtype, name + " out")
        if grads is not None:
            for nm, gr in zip(("dq", "dk", "dv"), grads):
                assert_close(gr, c["out"][nm], dtype, name + " " + nm)


@pytest.mark.parametrize("impl,dtype,S,D,qc", [("generic", torch.float32, 128, 32, 16), ("generic", torch.bfloat16, 128, 64, 32),
                                                ("mfma", torch.bfloat16, 1024, 128, 256),
                                                ("mfma", torch.float32, 512, 64, 128), ("mfma", torch.float32, 512, 128, 256)])
def test_first_and_last_step_modes_give_the_bits_of_the_separate_passes(impl, dtype, S, D, qc):
    """Two ring steps of one device (own shard, then the shard before it), once with explicit fp32 carries, a
    finalize pass and a cast, once with the first step starting the carries (uninitialised memory behind them) and
    the last step writing out / dq / dk / dv in the primal dtype.  Same fp32 sums, one rounding: equal bits."""
    from ringattention_amd import _lib as L
    from ringattention_amd import ringattention_hip as rh
    B, H = 1, 2
    q, k, v, do = make_qkv(B, 2 * S, H, D, dtype=dtype, seed=31, scale=D ** -0.25)
    q, k, v, do = (t.to(DEV) for t in (q, k, v, do))
    kw = dict(causal_block_size=1, query_chunk_size=qc, key_chunk_size=qc, impl=impl)
    nq = S // qc
    qs = slice(S, 2 * S)                                   # the second device of a ring of two
    steps = [(nq, slice(S, 2 * S), nq), (nq, slice(0, S), 0)]
    f32 = lambda *shape: torch.full(shape, float("nan"), dtype=torch.float32, device=DEV)

    # reference way: carry initialised, every step reads and writes it, finalize, delta, zeroed accumulators, cast
    num, den, mx = f32(B, S, H, D), f32(B, H, S), f32(B, H, S)
    rh._carry_init(num, den, mx)
    for q_start, ks, k_start in steps:
        ra._blockwise_attention_fwd(q[:, qs], k[:, ks], v[:, ks], (num, den, mx), q_start, k_start, None, None, **kw)
    out_a = torch.empty(B, S, H, D, dtype=dtype, device=DEV)
    rh._finalize(num, den, out_a)
    delta = rh._bwd_delta(do[:, qs].contiguous(), out_a)
    dq = torch.zeros(B, S, H, D, dtype=torch.float32, device=DEV)
    dk, dv = (torch.zeros(B, 2 * S, H, D, dtype=torch.float32, device=DEV) for _ in range(2))
    for q_start, ks, k_start in steps:
        ra._blockwise_attention_bwd(q[:, qs], k[:, ks], v[:, ks], do[:, qs], (dq, dk[:, ks], dv[:, ks], out_a, den, mx),
                                    q_start, k_start, None, None, _delta=delta, **kw)
    ref = (out_a, dq.to(dtype), dk.to(dtype), dv.to(dtype))

    # first / last modes: NaN-filled carries prove that the first step reads nothing
    num2, den2, mx2 = f32(B, S, H, D), f32(B, H, S), f32(B, H, S)
    out_b = torch.empty(B, S, H, D, dtype=dtype, device=DEV)
    for j, (q_start, ks, k_start) in enumerate(steps):
        ra._blockwise_attention_fwd(q[:, qs], k[:, ks], v[:, ks], (num2, den2, mx2), q_start, k_start, None, None,
                                    _carry_is_initial=j == 0, _out=out_b if j == 1 else None, **kw)
    assert torch.equal(den2, den) and torch.equal(mx2, mx)
    dq2 = f32(B, S, H, D)
    dq_o = torch.empty(B, S, H, D, dtype=dtype, device=DEV)
    dk_o, dv_o = (torch.empty(B, 2 * S, H, D, dtype=dtype, device=DEV) for _ in range(2))
    for j, (q_start, ks, k_start) in enumerate(steps):
        # every K/V shard gets one call here: it is the first and the last one for its dk, dv (no fp32 array at all)
        ra._blockwise_attention_bwd(q[:, qs], k[:, ks], v[:, ks], do[:, qs], (dq2, None, None, out_b, den2, mx2),
                                    q_start, k_start, None, None, _delta=delta,
                                    _grads_initial=(L.RA_GRAD_INIT_DQ if j == 0 else 0) | L.RA_GRAD_INIT_DKV,
                                    _dq_out=dq_o if j == 1 else None, _dkv_out=(dk_o[:, ks], dv_o[:, ks]), **kw)
    torch.cuda.synchronize()
    for name, a, b in zip(("out", "dq", "dk", "dv"), ref, (out_b, dq_o, dk_o, dv_o)):
        assert torch.equal(torch.nan_to_num(a.float()), torch.nan_to_num(b.float())), name


def test_first_and_last_step_modes_reject_missing_buffers():
    from ringattention_amd import ringattention_hip as rh
    q, k, v, do = (t.to(DEV) for t in make_qkv(1, 64, 2, 32, dtype=torch.float32, seed=32))
    den, mx = (torch.empty(1, 2, 64, dtype=torch.float32, device=DEV) for _ in range(2))
    kw = dict(causal_block_size=1, query_chunk_size=16, key_chunk_size=16)
    with pytest.raises(ValueError):       # no numerator, but the carry is not initial
        ra._blockwise_attention_fwd(q, k, v, (None, den, mx), 0, 0, None, None, _out=torch.empty_like(q), **kw)
    with pytest.raises(ValueError):       # no numerator and no out
        ra._blockwise_attention_fwd(q, k, v, (None, den, mx), 0, 0, None, None, _carry_is_initial=True, **kw)
    out = torch.empty_like(q)
    delta = torch.zeros_like(den)
    with pytest.raises(ValueError):       # dq missing although it is not the first call
        ra._blockwise_attention_bwd(q, k, v, do, (None, torch.zeros_like(q), torch.zeros_like(q), out, den, mx), 0, 0,
                                    None, None, _delta=delta, _dq_out=torch.empty_like(q), **kw)


# --- a scan step of all virtual devices as one launch per kernel (ra_attn_*_ring_step) against one launch per device
@pytest.mark.parametrize("n,cbs,use_seg,use_bias,D", [(2, 1, False, False, 128), (4, 1, True, True, 128),
                                                      (8, 1, True, False, 128), (4, None, False, True, 128),
                                                      (8, 256, True, True, 128), (4, 1, True, True, 64)])
def test_ring_step_launch_equals_device_launches_bitwise(n, cbs, use_seg, use_bias, D):
    B, S, H = 2, 4096, 2
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=n, scale=1.0)
    g = torch.Generator().manual_seed(n + 50)
    bias = torch.randn(B, H, 1, S, generator=g) if use_bias else None
    seg = packed_segment_ids(B, S, 700, seed=n + 3) if use_seg else None
    res = {}
    for mode in ("step", "device"):
        kw = kwargs(128, 128, cbs, dtype=torch.float32, impl="mfma", ring_launch=mode)
        out, grads = run_hip(q, k, v, do, bias, seg, None, n, kw)
        res[mode] = (out,) + grads
    for name, a, b in zip(("out", "dq", "dk", "dv"), res["step"], res["device"]):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)), name
    # and the oracle, so that both are right and not only equal
    kw = kwargs(128, 128, cbs, dtype=torch.float32)
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    for name, a, b in zip(("out", "dq", "dk", "dv"), res["step"], (ref_out,) + tuple(ref_grads)):
        assert_close(a, b, torch.bfloat16, name)


def test_ring_step_entry_points_refuse_what_they_do_not_take():
    import ctypes
    from ringattention_amd import _lib as L
    lib = L.load()
    p, r = L.RaAttnFwdParams(), L.RaRingStep()
    r.n_dev, r.idx = 4, 4
    x = torch.zeros(1, 512, 1, 128, dtype=torch.bfloat16, device=DEV)
    st = torch.zeros(1, 1, 512, device=DEV)
    p.q = p.k = p.v = x.data_ptr()
    p.denominator = p.max_score = st.data_ptr()
    p.B, p.Sq, p.Skv, p.H, p.D, p.dtype = 1, 512, 512, 1, 128, L.RA_BF16
    p.mask.query_chunk_size = p.mask.key_chunk_size = 128
    assert lib.ra_attn_fwd_ring_step(ctypes.byref(p), ctypes.byref(r), None) == L.RA_ERR_INVALID    # idx == n_dev
    r.idx, r.run = 0, 1 << 5
    assert lib.ra_attn_fwd_ring_step(ctypes.byref(p), ctypes.byref(r), None) == L.RA_ERR_INVALID    # bit beyond the ring
    r.run = 1
    assert lib.ra_attn_fwd_ring_step(ctypes.byref(p), ctypes.byref(r), None) == L.RA_ERR_INVALID    # numerator needed
    p.impl = L.RA_IMPL_GENERIC
    assert lib.ra_attn_fwd_ring_step(ctypes.byref(p), ctypes.byref(r), None) == L.RA_ERR_UNSUPPORTED


def test_residuals_are_saved_tensors():
    """A second backward pass with retain_graph gives the same gradients; editing q in place between the forward
    and the backward pass is refused by autograd instead of giving gradients of the wrong input."""
    q, k, v, do = (t.to(DEV) for t in make_qkv(1, 256, 2, 128, dtype=torch.bfloat16, seed=5))
    q, k, v = (t.requires_grad_(True) for t in (q, k, v))
    out = ra.ringattention(q, k, v, None, None, None, "sp", True, kwargs(128, 128, 1))
    g1 = torch.autograd.grad(out, (q, k, v), do, retain_graph=True)
    g2 = torch.autograd.grad(out, (q, k, v), do)
    for a, b in zip(g1, g2):
        assert torch.equal(a, b)
    q2 = q.detach().clone().requires_grad_(True)
    qq = q2 * 1.0
    out = ra.ringattention(qq, k, v, None, None, None, "sp", True, kwargs(128, 128, 1))
    qq.add_(1.0)
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        out.backward(do)


def test_ring_forward_with_segment_ids_replays_from_a_hip_graph():
    """The ring forward with segment ids and a bias, captured once after a first eager call (which fills the
    per-tensor cache of the segment tile ranges, so that nothing is copied to the host under capture) and replayed
    with new q / k / v contents: every replay equals the eager result on the same inputs."""
    B, S, H, D, n = 1, 2048, 2, 128, 4
    kw = kwargs(256, 256, 1, impl="mfma")
    seg = packed_segment_ids(B, S, 500, seed=2).to(DEV)
    bias = torch.randn(1, 1, 1, S, generator=torch.Generator().manual_seed(3)).to(DEV)
    qs, ks, vs = (torch.zeros(B, S, H, D, dtype=torch.bfloat16, device=DEV) for _ in range(3))

    def call():
        with ra.ring_axis("sp", n):
            return ra.ringattention(qs, ks, vs, bias, seg, None, axis_name="sp", float32_logits=True,
                                    blockwise_kwargs=kw)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        call()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.no_grad(), torch.cuda.graph(graph):
        out_graph = call()
    for seed in (1, 2, 3):
        q, k, v, _ = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=seed)
        qs.copy_(q), ks.copy_(k), vs.copy_(v)
        graph.replay()
        torch.cuda.synchronize()
        with torch.no_grad():
            eager = call()
        torch.cuda.synchronize()
        assert torch.equal(out_graph.view(torch.int16), eager.view(torch.int16)), seed
        assert float(eager.float().abs().max()) > 0


# --- chunk sizes off the 128-grid of the MFMA kernels: served by them with 128 x 128 chunks where that sums over the
# same pairs (even sizes under causal_block_size 1, a block size dividing both, or no causal mask at all)
@pytest.mark.parametrize("qc,kc,cbs,n,use_seg", [(64, 64, 1, 1, False), (192, 64, 1, 2, True), (32, 96, 1, 1, True),
                                                  (384, 192, None, 2, False), (64, 192, 32, 1, False),
                                                  (96, 96, 1, 4, True)])
def test_mfma_serves_chunk_sizes_off_its_grid(qc, kc, cbs, n, use_seg):
    B, S, H, D = 1, 1536, 2, 128
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=qc + kc, scale=1.0)
    seg = packed_segment_ids(B, S, 400, seed=5) if use_seg else None
    kw = kwargs(qc, kc, cbs, dtype=torch.float32, impl="mfma")       # "mfma": raises if the generic kernels were needed
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, None, seg, None, n, kw)
    out, grads = run_hip(q, k, v, do, None, seg, None, n, kw)
    assert_close(out, ref_out, torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close(a, b, torch.bfloat16, name)


def test_mfma_refuses_chunk_sizes_whose_chunking_matters():
    """Odd chunk sizes under a causal mask (the reference then drops the diagonal pair of some chunk corners,
    :324-331) stay with the generic kernels: impl="mfma" refuses, "auto" matches the oracle."""
    B, S, H, D = 1, 384, 1, 128
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=3, scale=1.0)
    with pytest.raises(NotImplementedError):
        run_hip(q, k, v, None, None, None, None, 1, kwargs(3, 3, 1, impl="mfma"))
    kw = kwargs(3, 3, 1)
    ref_out, _ = oracle_fwd_bwd(q, k, v, None, None, None, None, 1, kw)
    out, _ = run_hip(q, k, v, None, None, None, None, 1, kw)
    assert_close(out, ref_out, torch.bfloat16, "out")


# --- the residual `output` of the reference (ringattention_jax.py:53) is the quotient before it is rounded
@pytest.mark.parametrize("impl,D,n,use_seg,mode", [("mfma", 128, 1, False, "step"), ("mfma", 64, 4, True, "step"),
                                                   ("mfma", 128, 4, True, "device"), ("generic", 64, 2, False, "step")])
def test_output_residual_is_the_unrounded_quotient(impl, D, n, use_seg, mode):
    """bf16 inputs: the forward pass keeps numerator / denominator in fp32 next to the rounded output; rounding it
    gives the returned output bit for bit, and it matches the oracle's fp32 output and residual product
    delta = sum_d g * output (:218) to what the bf16 rounding of the probabilities inside the MFMA kernels leaves
    (the generic kernels keep them in fp32)."""
    from ringattention_amd import ringattention_hip as rh
    from oracle import ringattention_oracle as O
    from tests.util import oracle_kwargs
    B, S, H = 1, 1024 if impl == "mfma" else 256, 2
    qc = 128 if impl == "mfma" else 32
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=11, scale=1.0)
    seg = packed_segment_ids(B, S, 300, seed=5) if use_seg else None      # documents shorter than a shard: rows
    kw = kwargs(qc, qc, 1, dtype=torch.float32, impl=impl, ring_launch=mode)   # of later shards are passed through
    with ra.ring_axis("sp", n):
        out, res = rh._ring_attention_fwd(q.to(DEV), k.to(DEV), v.to(DEV), None, None if seg is None else seg.to(DEV),
                                          None, "sp", True, kw)
    out32 = res[0]
    assert out32.dtype == torch.float32 and out.dtype == torch.bfloat16
    assert torch.equal(out32.to(torch.bfloat16).view(torch.int16), out.view(torch.int16))
    ref_out, ref_res = O.ring_attention_fwd(q, k, v, None, seg, None, n, True, oracle_kwargs(kw))
    tol = 3e-3 if impl == "mfma" else 1e-5
    ma, rl = errors(out32, ref_res[0])
    print("un-rounded output against the oracle's: max-abs %.2e, rel-L2 %.2e" % (ma, rl), flush=True)
    assert rl <= tol, (ma, rl)
    delta = rh._bwd_delta(do.to(DEV), out32)
    ref_delta = (do.float() * ref_res[0].float()).sum(-1).permute(0, 2, 1)
    ma, rl = errors(delta, ref_delta)
    print("delta against the oracle's: max-abs %.2e, rel-L2 %.2e" % (ma, rl), flush=True)
    assert rl <= tol, (ma, rl)
    # the kernel's sum is the plain fp32 one of these very numbers
    mine = (do.to(DEV).float() * out32).sum(-1).permute(0, 2, 1)
    assert errors(delta, mine)[1] <= 1e-6
    # the rounded output as residual stays available and is what it says
    with ra.ring_axis("sp", n):
        out_r, res_r = rh._ring_attention_fwd(q.to(DEV), k.to(DEV), v.to(DEV), None,
                                              None if seg is None else seg.to(DEV), None, "sp", True,
                                              dict(kw, output_residual="rounded"))
    assert res_r[0].dtype == torch.bfloat16 and torch.equal(res_r[0].view(torch.int16), out.view(torch.int16))


def test_gradients_with_the_fp32_residual_match_the_oracle_more_closely():
    """What the residual is for: with output values of order one and a cotangent correlated with them, delta carries
    the output's rounding error (2^-9 relative) into dS when it is taken from the rounded output."""
    B, S, H, D = 1, 1024, 2, 128
    q, k, v, _ = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=21, scale=1.0)
    v = (v.float() + 4.0).to(torch.bfloat16)            # outputs near 4: large delta, visible rounding
    do = torch.ones(B, S, H, D, dtype=torch.bfloat16)
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, None, None, None, 1, kwargs(128, 128, 1))
    errs = {}
    for mode in ("fp32", "rounded"):
        kw = kwargs(128, 128, 1, dtype=torch.float32, impl="mfma", output_residual=mode)
        _, grads = run_hip(q, k, v, do, None, None, None, 1, kw)
        errs[mode] = [errors(a, b)[1] for a, b in zip(grads, ref_grads)]
        assert_close(grads[2], ref_grads[2], torch.bfloat16, "dv")
    print("relative L2 error of dq, dk, dv:", errs, flush=True)
    # a stress case (dP - delta cancels to a fortieth of either term): no fixed bar, the comparison is the point
    assert errs["fp32"][0] < errs["rounded"][0] and errs["fp32"][1] < errs["rounded"][1]


# --- fp32 inputs on the matrix cores (v_mfma_f32_32x32x2_f32): head size 64 or 128, chunk sizes on the 128-grid
F32_MFMA_CASES = [
    # B, S, H, D, qc, kc, cbs, n, bias, seg
    (1, 2048, 8, 64, 512, 512, 1, 1, True, True),          # the reference's CPU-runnable configuration
    (2, 512, 2, 128, 128, 128, 1, 1, False, False),
    (1, 1024, 3, 128, 256, 128, 1, 2, True, True),
    (2, 1024, 2, 64, 128, 256, 1, 4, True, False),
    (1, 1024, 2, 128, 128, 128, None, 2, False, True),
    (1, 1024, 2, 64, 128, 128, None, 1, True, False),
    (1, 2048, 2, 128, 256, 256, 64, 2, False, True),
    (1, 2048, 1, 64, 128, 128, 512, 4, True, True),
    (1, 1024, 2, 128, 64, 64, 1, 2, False, True),           # off the grid: served as 128 x 128 chunks
]


@pytest.mark.parametrize("case", F32_MFMA_CASES)
def test_fp32_mfma_kernels_match_oracle(case):
    B, S, H, D, qc, kc, cbs, n, use_bias, use_seg = case
    impl = "mfma" if qc % 128 == 0 and kc % 128 == 0 else "auto"
    check_case(B, S, H, D, qc, kc, cbs, n, use_bias, use_seg, torch.float32, impl=impl, seg_mean=200)


@pytest.mark.parametrize("D,n,cbs,use_seg,use_bias", [(128, 1, 1, False, False), (64, 2, 1, True, True),
                                                      (128, 4, 256, True, False), (64, 1, None, False, True)])
def test_fp32_mfma_kernels_agree_with_the_vector_kernels(D, n, cbs, use_seg, use_bias):
    """Same inputs through the fp32 matrix-core kernels and the one-row-per-lane kernels: both sum in fp32, so they
    agree to a few ulp of the largest term."""
    B, S, H = 2, 1024, 2
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.float32, seed=3, scale=1.0)
    g = torch.Generator().manual_seed(9)
    bias = torch.randn(B, H, 1, S, generator=g) if use_bias else None
    seg = packed_segment_ids(B, S, 150, seed=4) if use_seg else None
    res = {}
    for impl in ("mfma", "generic"):
        out, grads = run_hip(q, k, v, do, bias, seg, None, n, kwargs(128, 128, cbs, dtype=torch.float32, impl=impl))
        res[impl] = (out,) + grads
    for name, a, b in zip(("out", "dq", "dk", "dv"), res["mfma"], res["generic"]):
        ma, rl = errors(a, b)
        assert ma <= 2e-5 and rl <= 1e-5, (name, ma, rl)


def test_fp32_mfma_kernels_refuse_what_they_do_not_take():
    """A per-row bias and head sizes above 128 stay with the vector kernels (which stop at 256 themselves); asking for
    the matrix-core kernels by name then is an error, not a silent fallback.  Head sizes below 128 are zero-padded."""
    q, k, v, _ = make_qkv(1, 256, 1, 256, dtype=torch.float32, seed=1)
    with pytest.raises(NotImplementedError):
        run_hip(q, k, v, None, None, None, None, 1, kwargs(128, 128, 1, dtype=torch.float32, impl="mfma"))
    q, k, v, _ = make_qkv(1, 256, 1, 32, dtype=torch.float32, seed=1)
    out, _ = run_hip(q, k, v, None, None, None, None, 1, kwargs(128, 128, 1, dtype=torch.float32, impl="mfma"))
    assert out.shape == q.shape and ra.kernel_family_of_last_call()["forward"] == "mfma_f32"
    q, k, v, _ = make_qkv(1, 256, 1, 64, dtype=torch.float32, seed=1)
    bias = torch.zeros(1, 1, 128, 256)
    with pytest.raises(NotImplementedError):
        run_hip(q, k, v, None, bias, None, None, 1, kwargs(128, 128, 1, dtype=torch.float32, impl="mfma"))
    out, _ = run_hip(q, k, v, None, bias, None, None, 1, kwargs(128, 128, 1, dtype=torch.float32))   # auto: served
    assert torch.isfinite(out).all()


# --- head sizes the matrix-core kernels do not tile: q, k, v zero-padded to 64 / 128, logits scaled by the original
# head size (ra_attn_*_params.logit_dim); the generic kernels remain the cross-check
@pytest.mark.parametrize("D,dtype,n,use_seg", [(32, torch.bfloat16, 1, False), (32, torch.bfloat16, 2, True),
                                               (96, torch.bfloat16, 2, True), (40, torch.bfloat16, 1, False),
                                               (32, torch.float32, 2, True), (80, torch.float32, 1, False)])
def test_other_head_sizes_run_on_the_mfma_kernels(D, dtype, n, use_seg):
    B, S, H = 1, 512 * n, 2
    print("head size case", D, dtype, n, use_seg, flush=True)
    q, k, v, do = make_qkv(B, S, H, D, dtype=dtype, seed=D, scale=D ** -0.25)
    bias = torch.randn(B, 1, 1, S, generator=torch.Generator().manual_seed(1)) if use_seg else None
    seg = packed_segment_ids(B, S, S // 3, seed=2) if use_seg else None
    kw = kwargs(128, 128, 1, dtype=torch.float32)
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    out, grads = run_hip(q, k, v, do, bias, seg, None, n, kw)
    fam = ra.kernel_family_of_last_call()
    want = "mfma_bf16" if dtype == torch.bfloat16 else "mfma_f32"
    assert fam == {"forward": want, "backward": want}, fam
    assert out.shape == q.shape and out.is_contiguous()
    assert_close(out, ref_out, dtype, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert a.shape == q.shape
        assert_close(a, b, dtype, name)
    if D == 32:         # the vector kernels take this head size as it is: same result within the parity bar
        g_out, g_grads = run_hip(q, k, v, do, bias, seg, None, n, dict(kw, impl="generic"))
        assert ra.kernel_family_of_last_call() == {"forward": "generic", "backward": "generic"}
        assert_close(out, g_out, dtype, "mfma vs generic out")
        for name, a, b in zip(("dq", "dk", "dv"), grads, g_grads):
            assert_close(a, b, dtype, "mfma vs generic " + name)


def test_a_large_call_on_the_generic_kernels_warns_once():
    """RA_IMPL_AUTO falls back to the vector-ALU kernels silently for small problems; from 2^28 (query, key) pairs
    on it says so, once per cause, and kernel_family_of_last_call tells which family ran.  (fp32 inputs with a bias
    row per query: bf16 ones take the matrix-core kernels that evaluate the mask element by element, silently.)"""
    import warnings
    B, S, H, D, qc = 1, 8192, 4, 64, 128
    q, k, v, _ = make_qkv(B, S, H, D, dtype=torch.float32, seed=1, scale=D ** -0.25)
    bias = torch.randn(1, 1, qc, S, generator=torch.Generator().manual_seed(2))       # one bias row per query of a chunk
    kw = kwargs(qc, qc, 1)
    qd, kd, vd, bd = (t.to(DEV) for t in (q, k, v, bias))
    with torch.no_grad(), warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        ra.ringattention(qd, kd, vd, bd, None, None, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
        ra.ringattention(qd, kd, vd, bd, None, None, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
        torch.cuda.synchronize()
    assert ra.kernel_family_of_last_call()["forward"] == "generic"
    mine = [w for w in seen if issubclass(w.category, RuntimeWarning) and "generic vector-ALU kernels" in str(w.message)]
    assert len(mine) <= 1
    from ringattention_amd import ringattention_hip as R
    assert any(key[0] == "forward" and any("bias with one row per query" in t for t in key[1]) for key in R._WARNED)
    # a small call of the same kind stays silent
    with torch.no_grad(), warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        ra.ringattention(qd[:, :256], kd[:, :256], vd[:, :256], bd[..., :256], None, None, axis_name=None,
                         float32_logits=True, blockwise_kwargs=kw)
    assert not [w for w in seen if "generic vector-ALU kernels" in str(w.message)]
    # the same large call in bf16
    with torch.no_grad(), warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        ra.ringattention(qd.bfloat16(), kd.bfloat16(), vd.bfloat16(), bd, None, None, axis_name=None, float32_logits=True,
                         blockwise_kwargs=kw)
    assert ra.kernel_family_of_last_call()["forward"] == "mfma_bf16_any"
    assert not [w for w in seen if "generic vector-ALU kernels" in str(w.message)]


def test_float16_inputs_are_computed_in_fp32_and_rounded():
    """float16 q, k, v (the reference is dtype-generic, ringattention_jax.py:18-23): computed on exact fp32 copies,
    output and gradients rounded to float16.  Bar: the oracle on the same float16 inputs, fp32 tolerance on values of
    order one widened by the float16 rounding of the results (2^-11 relative)."""
    B, S, H, D, n = 1, 512, 2, 64, 2
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.float16, seed=4, scale=D ** -0.25)
    seg = packed_segment_ids(B, S, 200, seed=3)
    kw = kwargs(128, 128, 1, dtype=torch.float32)
    ref_out, ref_grads = oracle_fwd_bwd(q.float(), k.float(), v.float(), do.float(), None, seg, None, n, kw)
    out, grads = run_hip(q, k, v, do, None, seg, None, n, kw)
    assert out.dtype == torch.float16 and all(g.dtype == torch.float16 for g in grads)
    assert ra.kernel_family_of_last_call() == {"forward": "mfma_f32", "backward": "mfma_f32"}
    for name, a, b in zip(("out", "dq", "dk", "dv"), (out,) + tuple(grads), (ref_out,) + tuple(ref_grads)):
        ma, rl = errors(a, b)
        assert ma <= 1e-4 + 2.0 ** -11 * float(b.abs().max()) and rl <= 1e-3, (name, ma, rl)


def test_segment_run_hulls_equal_brute_force():
    """ra_segment_run_hulls: for every run of 128 positions the hull of the 64-position tiles whose id range meets
    the run's, against a double loop in numpy; packed documents (monotone ids) and ids in arbitrary order."""
    import ctypes
    import numpy as np
    from ringattention_amd import _lib as L
    S = 4096 + 64                     # an odd number of tiles: the last run has one tile
    rng = np.random.default_rng(0)
    packed = packed_segment_ids(2, S, 300, seed=1).numpy()
    shuffled = rng.integers(0, 6, size=(2, S // 32)).repeat(32, axis=1).astype(np.int32)
    for ids in (packed, shuffled):
        seg = torch.from_numpy(ids).to(DEV)
        tiles = (S + 63) // 64
        mm = torch.empty((2, tiles, 2), dtype=torch.int32, device=DEV)
        hull = torch.empty((2, (tiles + 1) // 2, 2), dtype=torch.int32, device=DEV)
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        L.check(L.load().ra_segment_tile_ranges(seg.data_ptr(), seg.stride(0), 2, S, mm.data_ptr(), st), "ranges")
        L.check(L.load().ra_segment_run_hulls(mm.data_ptr(), 2, tiles, hull.data_ptr(), st), "hulls")
        mmh, got = mm.cpu().numpy(), hull.cpu().numpy()
        for b in range(2):
            for r in range((tiles + 1) // 2):
                ts = [t for t in (2 * r, 2 * r + 1) if t < tiles]
                lo, hi = min(mmh[b, t, 0] for t in ts), max(mmh[b, t, 1] for t in ts)
                meet = [t for t in range(tiles) if mmh[b, t, 1] >= lo and mmh[b, t, 0] <= hi]
                assert (got[b, r, 0], got[b, r, 1]) == (meet[0], meet[-1] + 1), (b, r)


@pytest.mark.parametrize("dtype,ids", [(torch.bfloat16, "packed"), (torch.bfloat16, "interleaved"), (torch.float32, "packed")])
def test_hull_table_gives_the_results_of_the_scan(dtype, ids):
    """The per-run hull table (the default when segment_ids covers every position) against the in-kernel scan of the
    tile ranges: the same bits for packed documents, where the two hulls coincide; with documents interleaved in
    blocks the table's hull is wider by fully masked tiles, which add exact zeros."""
    B, S, H, D, n = 1, 2048, 2, 128, 4
    q, k, v, do = make_qkv(B, S, H, D, dtype=dtype, seed=8, scale=D ** -0.25)
    if ids == "packed":
        seg = packed_segment_ids(B, S, 300, seed=5)
    else:
        seg = (torch.arange(S) // 192 % 3).to(torch.int32).reshape(1, S)       # three documents in alternating blocks
    bias = torch.randn(B, 1, 1, S, generator=torch.Generator().manual_seed(6))
    kw = kwargs(128, 128, 1, dtype=torch.float32, impl="mfma")
    a_out, a_g = run_hip(q, k, v, do, bias, seg, None, n, kw)
    b_out, b_g = run_hip(q, k, v, do, bias, seg, None, n, dict(kw, segment_hull_table=False))
    assert not torch.isnan(a_out).any()
    assert torch.equal(a_out, b_out)
    for x, y in zip(a_g, b_g):
        assert torch.equal(x, y)
    ref_out, ref_g = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    assert_close(a_out, ref_out, dtype, "out")
    for name, x, y in zip(("dq", "dk", "dv"), a_g, ref_g):
        assert_close(x, y, dtype, name)


@pytest.mark.parametrize("dtype,D,chunk", [(torch.bfloat16, 128, 128), (torch.float32, 64, 32)])
def test_strided_views_of_q_k_v_give_the_bits_of_contiguous_arrays(dtype, D, chunk):
    """q, k, v as slices of one fused (B, S, 3, H, D) projection, as transposed (B, H, S, D) arrays, and k, v as
    slices of a longer cache buffer: the results - output and, through autograd, the gradients in the layout of the
    views - are those of contiguous copies, bit for bit (the reference's arrays have no strides to speak of)."""
    B, S, H, n = 2, 512, 2, 2
    g = torch.Generator().manual_seed(21)
    qkv = torch.randn(B, S, 3, H, D, generator=g).to(dtype).to(DEV)
    do = torch.randn(B, S, H, D, generator=g).to(dtype).to(DEV)
    seg = packed_segment_ids(B, S, 150, seed=22).to(DEV)
    kw = kwargs(chunk, chunk, 1)

    def run(q, k, v):
        q, k, v = (t.detach().requires_grad_(True) for t in (q, k, v))
        with ra.ring_axis("sp", n):
            out = ra.ringattention(q, k, v, None, seg, None, axis_name="sp", float32_logits=True, blockwise_kwargs=kw)
            out.backward(do)
        return out.detach(), q.grad, k.grad, v.grad

    base = run(*(qkv[:, :, i].contiguous() for i in range(3)))
    fused = run(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2])
    bhsd = qkv.permute(2, 0, 3, 1, 4).contiguous()                      # (3, B, H, S, D)
    transposed = run(*(bhsd[i].transpose(1, 2) for i in range(3)))
    cache = torch.zeros(2, B, S + 256, H, D, dtype=dtype, device=DEV)
    cache[0, :, :S], cache[1, :, :S] = qkv[:, :, 1], qkv[:, :, 2]
    cached = run(qkv[:, :, 0].contiguous(), cache[0, :, :S], cache[1, :, :S])
    mixed = run(qkv[:, :, 0], cache[0, :, :S], qkv[:, :, 2].contiguous())   # k and v with different batch strides
    longer = torch.zeros(B, S + 128, H, D, dtype=dtype, device=DEV)
    longer[:, :S] = qkv[:, :, 0]
    prefix = run(longer[:, :S], qkv[:, :, 1], qkv[:, :, 2])                # q as the first positions of a longer array
    for name, res in (("fused", fused), ("transposed", transposed), ("cache", cached), ("mixed", mixed),
                      ("prefix", prefix)):
        for what, a, b in zip(("out", "dq", "dk", "dv"), res, base):
            assert a.shape == b.shape and torch.equal(a, b), (name, what)
    # the same through the boolean-mask ring
    mask = torch.ones(1, 1, S, S, dtype=torch.bool, device=DEV).tril()

    def run_inf(q, k, v):
        q, k, v = (t.detach().requires_grad_(True) for t in (q, k, v))
        with ra.ring_axis("sp", n):
            out = ra.ringattention_inference(q, k, v, mask, "sp", True)
            out.backward(do)
        return out.detach(), q.grad, k.grad, v.grad

    base = run_inf(*(qkv[:, :, i].contiguous() for i in range(3)))
    for what, a, b in zip(("out", "dq", "dk", "dv"), run_inf(longer[:, :S], cache[0, :, :S], qkv[:, :, 2]), base):
        assert a.shape == b.shape and torch.equal(a, b), ("inference prefix", what)
    for what, a, b in zip(("out", "dq", "dk", "dv"), run_inf(qkv[:, :, 0], cache[0, :, :S], qkv[:, :, 2]), base):
        assert torch.equal(a, b), ("inference", what)


def test_empty_inputs_give_empty_results():
    """No batch rows, no positions, no tokens: nothing is launched and the (empty) result stays attached to its inputs
    for autograd; queries without a single key end as the 0 / 0 of ringattention_jax.py:52."""
    kw = kwargs(128, 128, 1)
    for shape in ((0, 256, 2, 128), (1, 0, 2, 128)):
        q = torch.zeros(shape, device=DEV, dtype=torch.bfloat16, requires_grad=True)
        out = ra.ringattention(q, q, q, None, None, None, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
        assert out.shape == q.shape and out.dtype == q.dtype
        out.sum().backward()
        assert q.grad.shape == q.shape
        with ra.ring_axis("sp", 1):
            mask = torch.ones(1, 1, shape[1], shape[1], dtype=torch.bool, device=DEV)
            assert ra.ringattention_inference(q, q, q, mask, "sp", True).shape == q.shape
    q = torch.zeros(1, 128, 2, 128, device=DEV, dtype=torch.bfloat16)
    k = torch.zeros(1, 0, 2, 128, device=DEV, dtype=torch.bfloat16)
    assert torch.isnan(ra.ringattention(q, k, k, None, None, None, axis_name=None, float32_logits=True,
                                        blockwise_kwargs=kw)).all()
    ff = ra.SwiGLU(128, 256, device=DEV)
    x = torch.zeros(0, 256, 128, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    y = ra.blockwise_feedforward(ff, x, 128)
    assert y.shape == (0, 256, 128)
    y.sum().backward()
    assert x.grad.shape == x.shape and ff.w1.grad is not None and not ff.w1.grad.any()
    assert ff(torch.zeros(0, 128, device=DEV, dtype=torch.bfloat16)).shape == (0, 128)


@pytest.mark.parametrize("skip", [False, None])
@pytest.mark.parametrize("dtype,D,chunk,n", [(torch.bfloat16, 128, 128, 2), (torch.float32, 64, 32, 1), (torch.bfloat16, 64, 256, 4),
                                             (torch.float32, 128, 128, 2)])
def test_padding_mask_as_bias_matches_oracle(dtype, D, chunk, n, skip):
    """How a model built on the reference passes its padding mask: attn_bias = where(mask, 0, finfo.min) per key,
    (B, 1, 1, K), next to the causal mask.  A padded key's logit is absorbed by finfo.min exactly as a masked one's
    (ringattention_jax.py:135-136), so it weighs exp(finfo.min - max) = 0 in every row that sees a real key.  Batch
    row 1 starts with padding: its first 70 rows see padded and masked keys only and take the uniform weights of equal
    finfo.min logits over the keys of the chunks that run (:138-144).  With skip_masked_tiles=False every tile of those
    chunks runs here too and the whole output is the oracle's; with the default (tiles that hold masked pairs only
    are skipped, which asks for an unmasked key in every row) the rows that see a real key are the oracle's and the
    others stay finite.  With no cotangent on those rows - a model's loss mask - all gradients are the oracle's."""
    B, S, H = 2, 1024, 2
    q, k, v, do = make_qkv(B, S, H, D, dtype=dtype, seed=31, scale=D ** -0.25)
    keep = torch.ones(B, S, dtype=torch.bool)
    keep[0, 900:] = False                 # right padding
    keep[1, :70] = False                  # left padding
    bias = torch.where(keep, 0.0, torch.finfo(torch.float32).min).reshape(B, 1, 1, S)
    kw = kwargs(chunk, chunk, 1, dtype=torch.float32, skip_masked_tiles=skip)
    do = do.clone()
    do[1, :70] = 0                        # no cotangent on the rows that see no real key (a model's loss mask)
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, None, None, n, kw)
    out, grads = run_hip(q, k, v, do, bias, None, None, n, kw)
    print("padding mask", dtype, D, chunk, n, skip, ra.kernel_family_of_last_call(), flush=True)
    assert torch.isfinite(out).all() and all(torch.isfinite(t).all() for t in grads)
    if skip is None:                      # rows without a real key: defined, but not the reference's average
        out, ref_out = out.clone(), ref_out.clone()
        out[1, :70] = 0
        ref_out[1, :70] = 0
    assert_close(out, ref_out, dtype, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close(a, b, dtype, name)
    # padded keys get no gradient from rows that see a real key as well
    assert float(grads[1][0, 900:].abs().max()) == 0.0 and float(grads[2][0, 900:].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("S,chunk,cbs,use_bias,use_seg", [
    (1000, 100, 1, False, False), (1000, 250, 1, True, True), (5000, 500, 1, False, True), (1000, 500, None, False, False),
    (1000, 200, None, False, True), (1000, 200, None, True, True), (1016, 8, 8, True, False), (72, 24, 1, False, False)])
def test_lengths_off_the_128_grid_run_on_the_matrix_cores(S, chunk, cbs, use_bias, use_seg, dtype):
    """One device, a length that is no multiple of 128, chunk sizes that divide it (as the reference asks): the call
    is made on arrays padded to the next multiple of 128 and cut back, where the chunking cannot change the result;
    forward and backward against the oracle run at the original length and chunk sizes."""
    B, H, D = 2, 2, 128 if dtype == torch.bfloat16 else 64
    q, k, v, do = make_qkv(B, S, H, D, dtype=dtype, seed=S + chunk, scale=D ** -0.25)
    g = torch.Generator().manual_seed(S)
    bias = torch.randn(B, 1, 1, S, generator=g) if use_bias else None
    seg = packed_segment_ids(B, S, S // 4, seed=S) if use_seg else None
    kw = kwargs(chunk, chunk, cbs)
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, 1, kw)
    out, grads = run_hip(q, k, v, do, bias, seg, None, 1, kw)
    fam = ra.kernel_family_of_last_call()
    assert out.shape == q.shape and "mfma" in fam["forward"] and "mfma" in fam["backward"], fam
    assert_close(out, ref_out, dtype, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert a.shape == q.shape
        assert_close(a, b, dtype, name)
