"""The matrix-core kernels that evaluate the mask element by element (blockwise_kwargs["impl"] = "mfma_any") against the
CPU oracle: the random configurations of test_gpu_random_configs with bf16 inputs."""
import pytest
import torch

import ringattention_amd as ra
from tests.test_gpu_attention import run_hip
from tests.test_gpu_random_configs import OFFSET, draw
from tests.util import assert_close_scaled, kwargs, make_qkv, oracle_fwd_bwd, packed_segment_ids

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(OFFSET, OFFSET + 160))
def test_random_configuration_on_the_elementwise_matrix_core_kernels(seed):
    c = draw(seed)
    c["dtype"] = torch.bfloat16
    print("any case", seed, c, flush=True)
    n, B, H, D = c["n"], c["B"], c["H"], c["D"]
    S, Skv = n * c["q_len"], n * c["kv_len"]
    q, k, v, do = make_qkv(B, S, H, D, dtype=c["dtype"], seed=seed, Skv=Skv, scale=c["qk_std"])
    g = torch.Generator().manual_seed(seed + 500)
    bias = None
    if c["bias"] == "key":
        bias = torch.randn(1, 1, 1, Skv, generator=g)
    elif c["bias"] == "head":
        bias = torch.randn(B, H, 1, Skv, generator=g)
    elif c["bias"] == "row":
        bias = torch.randn(1, H, c["qc"], Skv, generator=g)
    elif c["bias"] == "pad":
        keep = torch.arange(Skv)[None, :] < torch.randint(1, Skv + 1, (B, 1), generator=g)
        bias = torch.where(keep, 0.0, torch.finfo(c["kw_dtype"]).min).reshape(B, 1, 1, Skv)
    seg = None
    if c["seg"] in ("docs", "relabelled"):
        seg = packed_segment_ids(B, max(S, Skv), max(4, S // 5), seed=seed + 7)
    elif c["seg"] == "one":
        seg = torch.zeros(B, max(S, Skv), dtype=torch.int32)
    if c["seg"] == "relabelled":
        table = torch.randint(-3, 4, (int(seg.max()) + 1,), generator=g, dtype=torch.int32)
        seg = table[seg[:1].long()]
    if c["bias"] == "pad" and c["seg"] in ("docs", "relabelled"):
        seg = None
    kw = kwargs(c["qc"], c["kc"], c["cbs"], dtype=c["kw_dtype"], impl="mfma_any")
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    out, grads = run_hip(q, k, v, do, bias, seg, None, n, kw)
    fam = ra.kernel_family_of_last_call()
    print("  family", fam, flush=True)
    assert fam == {"forward": "mfma_bf16_any", "backward": "mfma_bf16_any"}, fam
    assert_close_scaled(out, ref_out, torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close_scaled(a, b, torch.bfloat16, name)


def _qkv(B, S, H, D, seed, Skv=None):
    return make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=seed, Skv=Skv, scale=D ** -0.25)


@pytest.mark.parametrize("D", [160, 192, 256])
@pytest.mark.parametrize("n", [1, 4])
def test_head_sizes_above_128_take_the_elementwise_matrix_core_kernels(D, n):
    """bf16 calls with a head size above 128 (zero-padded to 256) are dispatched to these kernels by themselves, with
    documents and a bias, on one device and on a ring; fp32 inputs of the same shape stay on the vector kernels."""
    B, S, H = 1, 1024, 2
    q, k, v, do = _qkv(B, S, H, D, 3)
    seg = packed_segment_ids(B, S, 300, seed=5)
    bias = torch.randn(1, 1, 1, S, generator=torch.Generator().manual_seed(6))
    kw = kwargs(128, 128, 1)
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    out, grads = run_hip(q, k, v, do, bias, seg, None, n, kw)
    assert ra.kernel_family_of_last_call() == {"forward": "mfma_bf16_any", "backward": "mfma_bf16_any"}
    assert_close_scaled(out, ref_out, torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close_scaled(a, b, torch.bfloat16, name)
    if n == 1:
        run_hip(q.float(), k.float(), v.float(), do.float(), bias, seg, None, n, kw)
        assert ra.kernel_family_of_last_call() == {"forward": "generic", "backward": "generic"}


def test_attention_dropout_stays_off_the_elementwise_matrix_core_kernels():
    """Attention dropout at a head size above 128: the vector kernels (they hold the -inf bookkeeping of
    ringattention_jax.py:321); asking for the element-wise matrix-core kernels by name is refused."""
    B, S, H, D = 1, 256, 1, 160
    q, k, v, do = _qkv(B, S, H, D, 4)
    kw = kwargs(64, 64, 1, deterministic=False, attn_pdrop=0.1, dropout_rng=3)
    run_hip(q, k, v, do, None, None, None, 1, kw)
    assert ra.kernel_family_of_last_call() == {"forward": "generic", "backward": "generic"}
    with pytest.raises(NotImplementedError):
        run_hip(q, k, v, do, None, None, None, 1, dict(kw, impl="mfma_any"))


@pytest.mark.parametrize("D,S,Sk,n", [(256, 512, 512, 1), (128, 200, 328, 1), (192, 384, 384, 2), (64, 1000, 1000, 1)])
def test_boolean_mask_ring_on_the_elementwise_matrix_core_kernels(D, S, Sk, n):
    """ring_attention_inference with a mask that leaves some rows without a key (so the lengths are not padded) or a
    head size above 128: the mask is read as bytes, element by element, and a row that attends to nothing averages
    over all keys (ringattention_inference.py:22-24)."""
    from oracle import ringattention_oracle as O
    from tests.test_gpu_inference import _run
    B, H = 2, 2
    g = torch.Generator().manual_seed(S + D)
    q = (torch.randn(B, S, H, D, generator=g) * D ** -0.25).to(torch.bfloat16)
    k = (torch.randn(B, Sk, H, D, generator=g) * D ** -0.25).to(torch.bfloat16)
    v = torch.randn(B, Sk, H, D, generator=g).to(torch.bfloat16)
    do = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16)
    mask = torch.rand(B, H, S, Sk, generator=g) < 0.5
    mask[:, :, 5] = False                                   # a row that attends to nothing
    out, grads = _run(q, k, v, do, mask, n)
    fam = ra.kernel_family_of_last_call()
    assert fam == {"forward": "mfma_bf16_any", "backward": "mfma_bf16_any"}, fam
    ref_out, res = O.ring_attention_inference_fwd(q, k, v, mask, n, True)
    ref_grads = O.ring_attention_inference_bwd(n, res, do)
    assert_close_scaled(out, ref_out, torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close_scaled(a, b, torch.bfloat16, name)


def test_carry_of_a_ring_step_moves_between_the_kernel_families():
    """A device's carry (numerator, denominator, max) written by the tiled matrix-core kernels and continued by the
    element-wise ones, and the other way round, ends where one family alone ends (ringattention_jax.py:38-46)."""
    B, S, H, D = 1, 512, 2, 128
    q, k, v, _ = _qkv(B, S, H, D, 8)
    kw = kwargs(128, 128, 1)
    qd, kd, vd = (t.to("cuda") for t in (q, k, v))

    def two_steps(first, second):
        num = torch.zeros(B, 256, H, D, device="cuda")
        den = torch.zeros(B, H, 256, device="cuda")
        mx = torch.full((B, H, 256), float("-inf"), device="cuda")
        carry = (num, den, mx)
        # device 1 of a ring of two: its own shard, then shard 0
        ra._blockwise_attention_fwd(qd[:, 256:], kd[:, 256:], vd[:, 256:], carry, 2, 2, None, None, impl=first, **kw)
        ra._blockwise_attention_fwd(qd[:, 256:], kd[:, :256], vd[:, :256], carry, 2, 0, None, None, impl=second, **kw)
        torch.cuda.synchronize()
        return carry

    base = two_steps("mfma", "mfma")
    for first, second in (("mfma", "mfma_any"), ("mfma_any", "mfma"), ("mfma_any", "mfma_any")):
        got = two_steps(first, second)
        out_b, out_g = base[0] / base[1].transpose(1, 2)[..., None], got[0] / got[1].transpose(1, 2)[..., None]
        assert float((out_b - out_g).abs().max()) < 2e-2, (first, second)
        assert float((base[2] - got[2]).abs().max()) < 1e-3, (first, second)


def test_head_size_256_at_16k_ring4_matches_oracle():
    """B1 H2 S16384 D256 bf16 as a ring of four shards of 4096 with packed documents and a bias, chunks 512 / 512:
    the size class the family's throughput is quoted on, against the CPU oracle's ring loop, forward and backward."""
    import time
    B, S, H, D, n = 1, 16384, 2, 256, 4
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=41, scale=D ** -0.25)
    seg = packed_segment_ids(B, S, 3000, seed=42)
    bias = torch.randn(1, 1, 1, S, generator=torch.Generator().manual_seed(43))
    kw = kwargs(512, 512, 1)
    t0 = time.time()
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    print("oracle %.1f s" % (time.time() - t0), flush=True)
    out, grads = run_hip(q, k, v, do, bias, seg, None, n, kw)
    assert ra.kernel_family_of_last_call() == {"forward": "mfma_bf16_any", "backward": "mfma_bf16_any"}
    assert_close_scaled(out, ref_out, torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close_scaled(a, b, torch.bfloat16, name)


def test_families_agree_at_8k_on_the_tiled_kernels_shape():
    """The same bf16 call (8192 positions, documents, a bias, head size 128) on the tiled matrix-core kernels and on
    the element-wise ones: two independent implementations within the bf16 bar of each other."""
    B, S, H, D = 1, 8192, 2, 128
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=44, scale=D ** -0.25)
    seg = packed_segment_ids(B, S, 1500, seed=45)
    bias = torch.randn(1, 1, 1, S, generator=torch.Generator().manual_seed(46))
    a_out, a_grads = run_hip(q, k, v, do, bias, seg, None, 1, kwargs(512, 512, 1, impl="mfma"))
    assert ra.kernel_family_of_last_call()["forward"] == "mfma_bf16"
    b_out, b_grads = run_hip(q, k, v, do, bias, seg, None, 1, kwargs(512, 512, 1, impl="mfma_any"))
    assert ra.kernel_family_of_last_call()["forward"] == "mfma_bf16_any"
    assert_close_scaled(b_out, a_out.float().cpu(), torch.bfloat16, "out")
    for name, x, y in zip(("dq", "dk", "dv"), b_grads, a_grads):
        assert_close_scaled(x, y.float().cpu(), torch.bfloat16, name)


@pytest.mark.parametrize("D", [128, 256])
def test_elementwise_kernels_repeat_their_bits_and_isolate_masked_keys(D):
    """Two runs of one call give the same bits (every output element has one owner, no atomics); keys behind a row under
    the causal mask, or in another document, have bitwise no effect on it, and get exactly zero gradient from rows whose
    cotangent is zero."""
    B, S, H = 1, 640, 2
    q, k, v, do = _qkv(B, S, H, D, 12)
    seg = torch.cat((torch.zeros(1, 400, dtype=torch.int32), torch.ones(1, 240, dtype=torch.int32)), dim=1)
    kw = kwargs(40, 40, 1, impl="mfma_any")
    a, ga = run_hip(q, k, v, do, None, seg, None, 1, kw)
    b, gb = run_hip(q, k, v, do, None, seg, None, 1, kw)
    assert torch.equal(a, b) and all(torch.equal(x, y) for x, y in zip(ga, gb))
    k2, v2 = k.clone(), v.clone()
    k2[:, 400:] += 50.0                                  # the second document's keys: invisible to rows < 400
    v2[:, 400:] -= 20.0
    c, _ = run_hip(q, k2, v2, do, None, seg, None, 1, kw)
    assert torch.equal(a[:, :400], c[:, :400])
    k3, v3 = k.clone(), v.clone()
    k3[:, 300:400] += 50.0                               # keys behind row 299 under the causal mask
    v3[:, 300:400] -= 20.0
    d, _ = run_hip(q, k3, v3, do, None, seg, None, 1, kw)
    assert torch.equal(a[:, :300], d[:, :300])
    do2 = do.clone()
    do2[:, 400:] = 0.0                                   # no cotangent on the second document's rows
    _, g2 = run_hip(q, k, v, do2, None, seg, None, 1, kw)
    assert float(g2[1][:, 400:].abs().max()) == 0.0 and float(g2[2][:, 400:].abs().max()) == 0.0
    assert float(g2[0][:, 400:].abs().max()) == 0.0
