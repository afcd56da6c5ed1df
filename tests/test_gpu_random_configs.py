"""Seeded random configurations of ring_attention, HIP (through the C-ABI) against the CPU oracle.

The hand-picked cases of the other files follow the kernels' known seams; these draw the whole argument space of
ringattention_jax.py:17-97 at once - input type, head size, ring size, chunk sizes on and off the matrix-core grid,
causal block size or none, bias broadcast or per head / batch / row, packed segment ids, unequal query and key
lengths - so that a combination nobody thought of still meets the oracle.  Same bar as everywhere: max-abs 1e-4
(fp32 inputs) or 2e-2 (bf16 / fp16 inputs) for results of order one, scaled with the largest reference element
beyond that (tests/util.assert_close_scaled), relative L2 1e-2, NaN rows coinciding.
"""
import os
import random

import pytest
import torch

import ringattention_amd as ra
from tests.test_gpu_attention import run_hip
from tests.util import assert_close_scaled, kwargs, make_qkv, oracle_fwd_bwd, packed_segment_ids

pytestmark = pytest.mark.gpu

N_CASES = 160
# RA_TEST_SEED_OFFSET=1000 (say) draws another set of configurations with the same tests
OFFSET = int(os.environ.get("RA_TEST_SEED_OFFSET", "0"))


def draw(seed):
    r = random.Random(1000 + seed)
    dtype = r.choice([torch.float32, torch.bfloat16, torch.bfloat16, torch.float16])
    D = r.choice([16, 32, 40, 64, 64, 80, 96, 128, 128, 128, 160, 256])
    n = r.choice([1, 1, 2, 2, 4, 8])
    on_grid = r.random() < 0.6                      # chunk sizes the matrix-core kernels tile as they are
    if on_grid:
        qc, kc = r.choice([128, 128, 256]), r.choice([128, 128, 256])
    else:
        qc, kc = r.choice([8, 16, 32, 48, 64, 96]), r.choice([8, 16, 32, 48, 64, 96])
    # per-device lengths: multiples of both chunk sizes, the whole ring at most 2048 positions
    unit = qc * kc // __import__("math").gcd(qc, kc)
    per_dev_max = max(unit, (2048 // n) // unit * unit)
    q_len = unit * r.randint(1, max(1, min(4, per_dev_max // unit)))
    kv_len = q_len
    if n == 1 and r.random() < 0.3:                 # cross-length attention (one device only: a ring rotates equal shards)
        kv_len = unit * r.randint(1, max(1, min(4, per_dev_max // unit)))
    cbs = r.choice([1, 1, 1, None, 2, 8, 32, 128])
    if cbs not in (None, 1) and (max(cbs, qc) % min(cbs, qc) or max(cbs, kc) % min(cbs, kc)):
        cbs = 1                                     # :327-330 divide block size and chunk sizes by one another
    B, H = r.choice([1, 1, 2]), r.choice([1, 2, 3])
    bias = r.choice([None, None, "key", "key", "head", "row"])
    seg = r.choice([None, "docs", "docs", "one", "relabelled"])
    if r.random() < 0.15:
        bias = "pad"                                # a padding mask as a bias: where(keep, 0, finfo.min), padding on the right
    # blockwise_kwargs["dtype"]: the type the bias is rounded to and whose finfo.min is the mask value (:322, :298)
    kw_dtype = r.choice([torch.float32, torch.float32, torch.bfloat16])
    # standard deviation of q and k: the logits' is its square (1: the usual; 3: rows dominated by one or two keys)
    qk_std = r.choice([1.0, 1.0, 1.0, 3.0, 0.3])
    return dict(qk_std=qk_std, kw_dtype=kw_dtype, dtype=dtype, D=D, n=n, qc=qc, kc=kc, q_len=q_len, kv_len=kv_len, cbs=cbs, B=B, H=H, bias=bias, seg=seg)


@pytest.mark.parametrize("seed", range(OFFSET, OFFSET + N_CASES))
def test_random_configuration_matches_oracle(seed):
    c = draw(seed)
    print("case", seed, c, flush=True)
    n, B, H, D = c["n"], c["B"], c["H"], c["D"]
    S, Skv = n * c["q_len"], n * c["kv_len"]
    q, k, v, do = make_qkv(B, S, H, D, dtype=c["dtype"], seed=seed, Skv=Skv, scale=c["qk_std"])
    g = torch.Generator().manual_seed(seed + 500)
    bias = None
    if c["bias"] == "key":
        bias = torch.randn(1, 1, 1, Skv, generator=g)
    elif c["bias"] == "head":
        bias = torch.randn(B, H, 1, Skv, generator=g)
    elif c["bias"] == "row":                        # :279-283: rows 0:qc of the bias serve every query chunk
        bias = torch.randn(1, H, c["qc"], Skv, generator=g)
    elif c["bias"] == "pad":                        # every batch row keeps a prefix of real keys, at least one
        keep = torch.arange(Skv)[None, :] < torch.randint(1, Skv + 1, (B, 1), generator=g)
        # the mask value of the dtype the bias is rounded to (finfo(float32).min would round to -inf in bfloat16, and
        # a first chunk of -inf logits turns the row NaN in the reference, exp(-inf - -inf); here it counts as masked)
        bias = torch.where(keep, 0.0, torch.finfo(c["kw_dtype"]).min).reshape(B, 1, 1, Skv)
    seg = None
    if c["seg"] in ("docs", "relabelled"):
        seg = packed_segment_ids(B, max(S, Skv), max(4, S // 5), seed=seed + 7)
    elif c["seg"] == "one":
        seg = torch.zeros(B, max(S, Skv), dtype=torch.int32)
    if c["seg"] == "relabelled":
        # ids in no order and used more than once (the reference compares them for equality only, :294: two documents
        # with one id see each other across what lies between), one row of ids for the whole batch
        table = torch.randint(-3, 4, (int(seg.max()) + 1,), generator=g, dtype=torch.int32)
        seg = table[seg[:1].long()]
    if c["bias"] == "pad" and c["seg"] in ("docs", "relabelled"):
        seg = None                                  # a padded document's rows would see no real key at all
    kw = kwargs(c["qc"], c["kc"], c["cbs"], dtype=c["kw_dtype"])
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    out, grads = run_hip(q, k, v, do, bias, seg, None, n, kw)
    print("  family", ra.kernel_family_of_last_call(), flush=True)
    tol_dtype = torch.float32 if c["dtype"] == torch.float32 else torch.bfloat16
    assert out.dtype == c["dtype"] and out.shape == q.shape
    assert_close_scaled(out, ref_out, tol_dtype, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert a.dtype == c["dtype"]
        assert_close_scaled(a, b, tol_dtype, name)


def draw_cache(seed):
    r = random.Random(5000 + seed)
    dtype = r.choice([torch.float32, torch.bfloat16, torch.bfloat16, torch.float16])
    D = r.choice([32, 64, 64, 80, 128, 128, 128, 256])
    n = r.choice([1, 1, 1, 2, 4])
    qc = r.choice([1, 1, 1, 1, 2, 4, 16])
    kc = r.choice([16, 32, 64, 128, 512])
    q_len = qc * r.choice([1, 1, 2])                 # query tokens per device
    kv_len = kc * r.randint(1, max(1, 2048 // (n * kc)))
    L = n * kv_len
    edge = r.random()
    if edge < 0.15:
        cache_idx = r.choice([0, 1, L - 1])
    elif edge < 0.45:
        cache_idx = min(L - 1, kc * r.randint(0, L // kc))        # the skip predicate's edge (:324-331)
    else:
        cache_idx = r.randint(0, L - 1)
    cbs = r.choice([1, 1, 1, None])
    B, H = r.choice([1, 2, 3]), r.choice([1, 2, 5])
    bias = r.choice([None, None, "key", "head", "pad"])
    seg = r.choice([None, None, "docs"])
    device_idx = r.random() < 0.5                     # cache_idx as a device scalar (a traced value under jit)
    return dict(dtype=dtype, D=D, n=n, qc=qc, kc=kc, q_len=q_len, kv_len=kv_len, cache_idx=cache_idx, cbs=cbs, B=B, H=H,
                bias=bias, seg=seg, device_idx=device_idx)


@pytest.mark.parametrize("seed", range(OFFSET, OFFSET + 96))
def test_random_cache_idx_configuration_matches_oracle(seed):
    """The cache_idx path (ringattention_jax.py:31-35, :72-73): the query tokens sit at global positions
    (cache_idx // query_chunk_size) * query_chunk_size + row, the keys are the whole cache."""
    from oracle import ringattention_oracle as O
    from tests.util import oracle_kwargs
    c = draw_cache(seed)
    print("cache case", seed, c, flush=True)
    n, B, H, D = c["n"], c["B"], c["H"], c["D"]
    S, L = n * c["q_len"], n * c["kv_len"]
    q, k, v, _ = make_qkv(B, S, H, D, dtype=c["dtype"], seed=seed, Skv=L)
    g = torch.Generator().manual_seed(seed + 900)
    bias = None
    if c["bias"] == "key":
        bias = torch.randn(1, 1, 1, L, generator=g)
    elif c["bias"] == "head":
        bias = torch.randn(B, H, 1, L, generator=g)
    elif c["bias"] == "pad":                        # a left-padded prompt: where(keep, 0, finfo.min)
        keep = torch.arange(L)[None, :] >= torch.randint(0, L, (B, 1), generator=g)
        bias = torch.where(keep, 0.0, torch.finfo(torch.float32).min).reshape(B, 1, 1, L)
    seg = packed_segment_ids(B, L, max(4, L // 3), seed=seed + 3) if c["seg"] == "docs" else None
    kw = kwargs(c["qc"], c["kc"], c["cbs"], dtype=torch.float32)
    ref = O.ring_attention(q, k, v, bias, seg, c["cache_idx"], n, True, oracle_kwargs(kw))
    ci = torch.tensor(c["cache_idx"], dtype=torch.int32, device="cuda") if c["device_idx"] else c["cache_idx"]
    with ra.ring_axis("sp", n):
        out = ra.ringattention(q.cuda(), k.cuda(), v.cuda(), bias.cuda() if bias is not None else None,
                               seg.cuda() if seg is not None else None, ci, axis_name="sp", float32_logits=True,
                               blockwise_kwargs=kw)
    torch.cuda.synchronize()
    assert out.dtype == c["dtype"] and out.shape == q.shape
    assert_close_scaled(out, ref, torch.float32 if c["dtype"] == torch.float32 else torch.bfloat16, "out")


def draw_ffn(seed):
    r = random.Random(9000 + seed)
    d = 128 * r.choice([1, 1, 2, 3])
    f = 128 * r.choice([1, 2, 3, 5, 7])
    chunk = r.choice([8, 40, 100, 128, 128, 200, 256, 384, 512])
    n = r.randint(1, 6)                              # scan steps
    b = r.choice([1, 1, 2, 3])
    policy = r.choice([None, "nothing_saveable", "save_preactivations"])
    launch = r.choice([None, None, 512, 1024])
    group = r.choice([1, 2, 4, 4])
    tile = r.choice([None, None, None, 0, 1, 2, 3])
    if d % 256 or f % 256 or chunk % 256:
        tile = None                                   # a forced tile kernel wants its own multiples
    return dict(d=d, f=f, chunk=chunk, n=n, b=b, policy=policy, launch=launch, group=group, tile=tile)


@pytest.mark.parametrize("seed", range(OFFSET, OFFSET + 48))
def test_random_blockwise_feedforward_matches_oracle(seed):
    """blockwise_feedforward (ringattention_jax.py:333-352) over a SwiGLU MLP against the oracle's scan and fp32
    autograd of the oracle's formula, relative L2 1e-2 on y, dx and the three weight gradients: chunk sizes on and
    off the GEMM's token grid, every policy, shared launches, grouped weight gradients, every tile kernel."""
    from oracle import ringattention_oracle as O
    from tests.util import errors
    c = draw_ffn(seed)
    print("ffn case", seed, c, flush=True)
    b, s, d, f = c["b"], c["chunk"] * c["n"], c["d"], c["f"]
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(b, s, d, generator=g).bfloat16()
    dy = torch.randn(b, s, d, generator=g).bfloat16()
    ff = ra.SwiGLU(d, f, device="cuda", init_std=0.05, gemm_tile=c["tile"])
    w1, w2, w3 = (w.detach().float().cpu().requires_grad_(True) for w in (ff.w1, ff.w2, ff.w3))
    xr = x.float().requires_grad_(True)
    yr = O.blockwise_feedforward(lambda h: O.swiglu(h, w1, w2, w3), xr, c["chunk"])
    yr.backward(dy.float())
    xd = x.cuda().requires_grad_(True)
    y = ra.blockwise_feedforward(ff, xd, c["chunk"], policy=c["policy"], launch_tokens=c["launch"],
                                 weight_grad_chunks=c["group"])
    y.backward(dy.cuda())
    torch.cuda.synchronize()
    assert y.shape == yr.shape and y.dtype == torch.bfloat16
    for name, got, ref in (("y", y, yr), ("dx", xd.grad, xr.grad), ("dw1", ff.w1.grad, w1.grad),
                           ("dw2", ff.w2.grad, w2.grad), ("dw3", ff.w3.grad, w3.grad)):
        rel = errors(got, ref)[1]
        assert rel <= 1e-2, "%s: rel-L2 %.3e" % (name, rel)
    # the module alone, on a token count off the grid
    t = 1 + seed * 37 % 300
    y1 = ff(x.cuda().reshape(-1, d)[:t])
    assert errors(y1, O.swiglu(x.float().reshape(-1, d)[:t], w1, w2, w3))[1] <= 1e-2


def draw_inference(seed):
    r = random.Random(13000 + seed)
    dtype = r.choice([torch.float32, torch.bfloat16, torch.bfloat16, torch.float16])
    D = r.choice([32, 40, 64, 96, 128, 128, 128, 160, 256])
    n = r.choice([1, 2, 2, 4])
    per_dev = r.choice([8, 24, 64, 100, 128, 256, 256, 512])
    B, H = r.choice([1, 2]), r.choice([1, 2, 3])
    kind = r.choice(["full", "bcast_bh", "key_only", "per_head", "per_batch"])
    p_keep = r.choice([0.05, 0.5, 0.9])
    empty_row = r.random() < 0.25                    # a row that attends to nothing: uniform weights (:22-24)
    causal = r.random() < 0.4
    return dict(dtype=dtype, D=D, n=n, per_dev=per_dev, B=B, H=H, kind=kind, p_keep=p_keep, empty_row=empty_row,
                causal=causal)


@pytest.mark.parametrize("seed", range(OFFSET, OFFSET + 64))
def test_random_inference_configuration_matches_oracle(seed):
    """ring_attention_inference (ringattention_inference.py:8-73): boolean masks of every broadcast form, sparse
    and dense, with and without rows that attend to nothing, shards on and off the packed-mask grid."""
    from oracle import ringattention_oracle as O
    c = draw_inference(seed)
    print("inference case", seed, c, flush=True)
    n, B, H, D = c["n"], c["B"], c["H"], c["D"]
    S = n * c["per_dev"]
    q, k, v, do = make_qkv(B, S, H, D, dtype=c["dtype"], seed=seed, scale=D ** -0.25)
    shape = {"full": (B, H, S, S), "bcast_bh": (1, 1, S, S), "key_only": (B, 1, 1, S), "per_head": (1, H, S, S),
             "per_batch": (B, 1, S, S)}[c["kind"]]
    g = torch.Generator().manual_seed(seed + 77)
    mask = torch.rand(shape, generator=g) < c["p_keep"]
    if c["causal"] and shape[2] == S:
        mask = mask & torch.tril(torch.ones(S, S, dtype=torch.bool))
    mask[..., 0] = True
    if c["empty_row"] and shape[2] == S:
        mask[:, :, S // 3, :] = False
    ref_out, res = O.ring_attention_inference_fwd(q, k, v, mask, n, True)
    ref_grads = O.ring_attention_inference_bwd(n, res, do)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    # the mask as callers hold it: boolean, or 0 / 1 in another type; dense, or a broadcast view
    md = mask.cuda()
    form = seed % 4
    if form == 1:
        md = md.to(torch.uint8)
    elif form == 2:
        md = md.to(torch.float32)
    elif form == 3 and md.shape[1] == 1:
        md = md.expand(md.shape[0], H, md.shape[2], md.shape[3])
    with ra.ring_axis("sp", n):
        out = ra.ringattention_inference(qd, kd, vd, md, "sp", True)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    tol_dtype = torch.float32 if c["dtype"] == torch.float32 else torch.bfloat16
    assert out.dtype == c["dtype"] and out.shape == q.shape
    assert_close_scaled(out, ref_out, tol_dtype, "out")
    for name, a, b in zip(("dq", "dk", "dv"), (qd.grad, kd.grad, vd.grad), ref_grads):
        assert_close_scaled(a, b, tol_dtype, name)


def draw_long(seed):
    r = random.Random(17000 + seed)
    dtype = r.choice([torch.float32, torch.bfloat16, torch.bfloat16])
    D = r.choice([64, 128, 128, 96])
    n = r.choice([1, 2, 4, 8])
    qc, kc = r.choice([128, 256, 512, 1024]), r.choice([128, 256, 512, 1024])
    unit = max(qc, kc)
    S = unit * n * r.randint(1, max(1, 8192 // (unit * n)))
    cbs = r.choice([1, 1, 1, None, 256, 2048])
    if cbs not in (None, 1) and (max(cbs, qc) % min(cbs, qc) or max(cbs, kc) % min(cbs, kc)):
        cbs = 1
    bias = r.choice([None, "key", "head"])
    seg = r.choice([None, "docs", "docs", "short", "relabelled", "relabelled"])
    return dict(dtype=dtype, D=D, n=n, qc=qc, kc=kc, S=S, cbs=cbs, bias=bias, seg=seg, H=r.choice([1, 2]))


@pytest.mark.parametrize("seed", range(OFFSET, OFFSET + 24))
def test_random_long_configuration_matches_oracle(seed):
    """Up to 8192 positions on the matrix-core kernels: loops of many key tiles, the tile buffers coming round, packed
    documents from a few positions to thousands, whole-ring launches."""
    c = draw_long(seed)
    print("long case", seed, c, flush=True)
    n, H, D, S = c["n"], c["H"], c["D"], c["S"]
    q, k, v, do = make_qkv(1, S, H, D, dtype=c["dtype"], seed=seed, scale=D ** -0.25)
    g = torch.Generator().manual_seed(seed + 300)
    bias = {"key": lambda: torch.randn(1, 1, 1, S, generator=g), "head": lambda: torch.randn(1, H, 1, S, generator=g),
            None: lambda: None}[c["bias"]]()
    seg = None
    if c["seg"] == "docs":
        seg = packed_segment_ids(1, S, S // 6, seed=seed + 7)
    elif c["seg"] == "short":
        seg = packed_segment_ids(1, S, 90, seed=seed + 7)
    elif c["seg"] == "relabelled":
        # documents of a few hundred positions whose ids come in no order and repeat: two documents with one id see
        # each other across what lies between (:294 compares for equality only), so the key tiles a row can meet are
        # not one run around the diagonal
        seg = packed_segment_ids(1, S, 400, seed=seed + 7)
        seg = torch.randint(0, 5, (int(seg.max()) + 1,), generator=g, dtype=torch.int32)[seg.long()]
    kw = kwargs(c["qc"], c["kc"], c["cbs"], dtype=torch.float32)
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    out, grads = run_hip(q, k, v, do, bias, seg, None, n, kw)
    fam = ra.kernel_family_of_last_call()
    print("  family", fam, flush=True)
    assert "generic" not in str(fam)
    tol_dtype = torch.float32 if c["dtype"] == torch.float32 else torch.bfloat16
    assert_close_scaled(out, ref_out, tol_dtype, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close_scaled(a, b, tol_dtype, name)


@pytest.mark.parametrize("seed", range(OFFSET, OFFSET + 64))
def test_random_dropout_configuration_matches_oracle(seed):
    """The draws of the first test with attention dropout on (ringattention_jax.py:119-123, :311-321): the mask of the
    documented Philox stream, seeded by an integer, on both sides; dropped pairs take finfo.min once more, rows may
    lose every allowed key."""
    c = draw(seed + 40000)
    r = random.Random(21000 + seed)
    p = r.choice([0.1, 0.3, 0.5, 0.9])
    if c["dtype"] == torch.float16:
        c["dtype"] = torch.bfloat16
    c["bias"] = c["bias"] if c["bias"] != "row" else "head"
    print("dropout case", seed, c, p, flush=True)
    n, B, H, D = c["n"], c["B"], c["H"], c["D"]
    S, Skv = n * c["q_len"], n * c["kv_len"]
    q, k, v, do = make_qkv(B, S, H, D, dtype=c["dtype"], seed=seed, Skv=Skv)
    g = torch.Generator().manual_seed(seed + 500)
    bias = None
    if c["bias"] == "key":
        bias = torch.randn(1, 1, 1, Skv, generator=g)
    elif c["bias"] == "head":
        bias = torch.randn(B, H, 1, Skv, generator=g)
    elif c["bias"] == "pad":                        # dropped and padded: finfo.min twice, -inf (:321)
        keep = torch.arange(Skv)[None, :] < torch.randint(1, Skv + 1, (B, 1), generator=g)
        bias = torch.where(keep, 0.0, torch.finfo(torch.float32).min).reshape(B, 1, 1, Skv)
    seg = None
    if c["seg"] == "docs":
        seg = packed_segment_ids(B, max(S, Skv), max(4, S // 5), seed=seed + 7)
    elif c["seg"] == "one":
        seg = torch.zeros(B, max(S, Skv), dtype=torch.int32)
    kw = kwargs(c["qc"], c["kc"], c["cbs"], dtype=torch.float32, deterministic=False, dropout_rng=seed + 1, attn_pdrop=p)
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    out, grads = run_hip(q, k, v, do, bias, seg, None, n, kw)
    tol_dtype = torch.float32 if c["dtype"] == torch.float32 else torch.bfloat16
    assert_close_scaled(out, ref_out, tol_dtype, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close_scaled(a, b, tol_dtype, name)


def draw_ring_cross(seed):
    r = random.Random(21000 + seed)
    n = r.choice([2, 4, 8])
    dtype = r.choice([torch.float32, torch.bfloat16])
    D = r.choice([64, 128])
    qc, kc = r.choice([(128, 128), (128, 256), (256, 128), (32, 64), (64, 32), (16, 16)])
    q_len = qc * r.randint(1, 3) * (kc // qc if kc > qc else 1)
    kv_len = kc * r.randint(1, 3) * (qc // kc if qc > kc else 1)
    cbs = r.choice([1, None, max(qc, kc)])
    return dict(n=n, dtype=dtype, D=D, qc=qc, kc=kc, q_len=q_len, kv_len=kv_len, cbs=cbs, B=r.choice([1, 2]),
                H=r.choice([1, 2]), bias=r.random() < 0.5, seg=r.random() < 0.5)


@pytest.mark.parametrize("seed", range(OFFSET, OFFSET + 32))
def test_random_ring_with_unequal_query_and_key_shards_matches_oracle(seed):
    """A ring whose query shards and key shards differ in length (ringattention_jax.py:31-37 places a device's chunks
    by its own shard lengths: query chunk start dev * q_len / qc, key chunk start src * kv_len / kc), with and without a
    causal block size, bias and segment ids."""
    c = draw_ring_cross(seed)
    print("ring cross case", seed, c, flush=True)
    n, B, H, D = c["n"], c["B"], c["H"], c["D"]
    S, Skv = n * c["q_len"], n * c["kv_len"]
    q, k, v, do = make_qkv(B, S, H, D, dtype=c["dtype"], seed=seed, Skv=Skv, scale=1.0)
    g = torch.Generator().manual_seed(seed + 900)
    bias = torch.randn(1, 1, 1, Skv, generator=g) if c["bias"] else None
    seg = packed_segment_ids(B, max(S, Skv), max(4, S // 5), seed=seed + 7) if c["seg"] else None
    kw = kwargs(c["qc"], c["kc"], c["cbs"])
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    out, grads = run_hip(q, k, v, do, bias, seg, None, n, kw)
    print("  family", ra.kernel_family_of_last_call(), flush=True)
    assert_close_scaled(out, ref_out, c["dtype"], "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close_scaled(a, b, c["dtype"], name)
