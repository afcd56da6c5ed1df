"""The HIP path against the CPU oracle at the sizes its throughput is quoted on: the oracle finishes four heads
of the 32K causal case in seconds, one batch row of the 262144-position decode in seconds, and a ring of 8 over
65536 positions with documents and a bias in under two minutes.

Bar (bf16 inputs): forward output and dq / dk / dv within max-abs 2e-2 and relative L2 1e-2 of the oracle, NaN
positions equal.  q and k are N(0,1), unscaled: the logits have unit variance, so the softmax has real dynamic
range (some rows are dominated by a few keys), unlike the near-uniform weights of the benchmark's inputs."""
import time

import pytest
import torch

import ringattention_amd as ra
from oracle import ringattention_oracle as O
from tests.util import assert_close, errors, kwargs, make_qkv, oracle_fwd_bwd, oracle_kwargs, packed_segment_ids

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _hip(q, k, v, do, bias, seg, n, kw):
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    with ra.ring_axis("sp", n):
        out = ra.ringattention(qd, kd, vd, bias.to(DEV) if bias is not None else None,
                               seg.to(DEV) if seg is not None else None, None, axis_name="sp",
                               float32_logits=True, blockwise_kwargs=kw)
        out.backward(do.to(DEV))
    torch.cuda.synchronize()
    return out.detach(), (qd.grad, kd.grad, vd.grad)


def _compare(tag, out, grads, ref_out, ref_grads, secs):
    rows = [("out",) + assert_close(out, ref_out, torch.bfloat16, tag + " out")]
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        rows.append((name,) + assert_close(a, b, torch.bfloat16, tag + " " + name))
    print(tag, "oracle %.1f s;" % secs, "; ".join("%s max-abs %.2e rel-L2 %.2e" % r for r in rows), flush=True)


def test_causal_32k_matches_oracle():
    """B1 H4 S32768 D128 bf16, causal, chunks 512/512: the shape, chunking and kernels of the headline figure on
    4 of its 32 heads (heads are independent; the launch is the same grid with fewer of them)."""
    B, S, H, D = 1, 32768, 4, 128
    print("oracle parity at 32k causal", flush=True)
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=40)
    kw = kwargs(512, 512, 1, impl="mfma")
    t0 = time.time()
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, None, None, None, 1, kw)
    secs = time.time() - t0
    out, grads = _hip(q, k, v, do, None, None, 1, kw)
    _compare("32k causal", out, grads, ref_out, ref_grads, secs)


def test_packed_documents_ring8_matches_oracle():
    """B1 H1 S65536 D128 bf16 as 8 virtual shards of 8192, document ids from geometric lengths (mean 4096) and an
    additive bias: the oracle runs the reference's ring loop (8 devices x 8 steps, 8224 chunk pairs of 512 x 512),
    forward and backward, in about 100 s on 8 cores.  At 131072 positions it needs 32896 chunk pairs, beyond 6
    minutes, so the ring is checked against the oracle at half that length (same chunk sizes, same number of
    devices and ring steps, same kernels) and at full length against one device and through the isolation
    properties below."""
    B, S, H, D, n = 1, 65536, 1, 128, 8
    print("oracle parity at 64k ring 8", flush=True)
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=41)
    seg = packed_segment_ids(B, S, 4096, seed=42)
    bias = torch.randn(1, 1, 1, S, generator=torch.Generator().manual_seed(43))
    kw = kwargs(512, 512, 1, impl="mfma")
    t0 = time.time()
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    secs = time.time() - t0
    out, grads = _hip(q, k, v, do, bias, seg, n, kw)
    _compare("64k ring 8 documents + bias", out, grads, ref_out, ref_grads, secs)


def _document_dense_check(q, k, v, do, bias, ids, out, grads, heads, tag):
    """One document of a packed sequence against the oracle's dense closed form in float64 (with its autograd for the
    gradients): a document attends to itself only, so its rows of out / dq / dk / dv are those of causal attention
    over the document alone with its slice of the bias."""
    S = ids.numel()
    starts = torch.nonzero(torch.cat([torch.ones(1, dtype=torch.bool, device=ids.device), ids[1:] != ids[:-1]]))[:, 0]
    ends = torch.cat([starts[1:], torch.tensor([S], device=ids.device)])
    lens = (ends - starts).tolist()
    # documents of 1500..5000 positions: one that crosses a multiple of 16384 (a shard boundary of the ring of 8) if
    # there is one, the first one that lies inside a shard, and the last one of the sequence of that length
    docs = [(s0, ln, (s0 // 16384) != ((s0 + ln - 1) // 16384)) for s0, ln in zip(starts.tolist(), lens) if 1500 <= ln <= 5000]
    assert docs
    picks = []
    for want in (lambda d: d[2], lambda d: not d[2]):
        hit = [d for d in docs if want(d)]
        if hit:
            picks.append(hit[0])
    if docs[-1] not in picks:
        picks.append(docs[-1])
    hs = list(heads)
    for s0, ln, crosses in picks:
        sl = slice(s0, s0 + ln)
        qd, kd, vd = (t[:, sl][:, :, hs].double().cpu().requires_grad_(True) for t in (q, k, v))
        kw = oracle_kwargs(kwargs(ln, ln, 1))
        ref = O.dense_attention(qd, kd, vd, bias[..., sl].double().cpu(), None, None, 1, kw)
        ref.backward(do[:, sl][:, :, hs].double().cpu())
        rows = [("out",) + assert_close(out[:, sl][:, :, hs], ref.detach(), torch.bfloat16, tag + " out")]
        for name, a, b in zip(("dq", "dk", "dv"), grads, (qd.grad, kd.grad, vd.grad)):
            rows.append((name,) + assert_close(a[:, sl][:, :, hs], b, torch.bfloat16, tag + " " + name))
        print(tag, "document at %d, %d positions, crosses a shard boundary: %s;" % (s0, ln, crosses),
              "; ".join("%s max-abs %.2e rel-L2 %.2e" % r for r in rows), flush=True)


def _sampled_rows_check(q, k, v, do, bias, ids, out, dq, n_rows, seed, tag):
    """n_rows (head, position) pairs drawn at random: out and dq of each row recomputed in float64 straight from
    the definition - softmax over the keys of the row's document up to the row, bias clamped to <= 0
    (ringattention_jax.py:299,:309), dS = P (dP - sum(dO out)) (:226-230)."""
    B, S, H, D = q.shape
    gen = torch.Generator().manual_seed(seed)
    worst = [0.0, 0.0]
    for _ in range(n_rows):
        h = int(torch.randint(H, (1,), generator=gen))
        pos = int(torch.randint(S, (1,), generator=gen))
        first = int(torch.nonzero(ids[:pos + 1] == ids[pos])[0, 0])
        kk, vv = k[0, first:pos + 1, h].double(), v[0, first:pos + 1, h].double()
        qq, gg = q[0, pos, h].double(), do[0, pos, h].double()
        logits = kk @ qq / D ** 0.5 + bias[0, 0, 0, first:pos + 1].double().clamp(max=0.0)
        p = torch.softmax(logits, dim=0)
        o = p @ vv
        ds = p * (vv @ gg - gg @ o)
        dq_row = ds @ kk / D ** 0.5
        for got, want, i in ((out[0, pos, h], o, 0), (dq[0, pos, h], dq_row, 1)):
            err = float((got.double() - want).abs().max())
            worst[i] = max(worst[i], err)
            assert err <= 2e-2, (tag, "out" if i == 0 else "dq", h, pos, err)
    print(tag, "%d sampled rows: worst max-abs out %.2e dq %.2e" % (n_rows, worst[0], worst[1]), flush=True)


def test_packed_documents_131k_ring8_full_size():
    """B1 H32 S131072 D128 bf16, 8 virtual shards of 16384, document ids and a bias: the whole configuration,
    forward and backward.  (1) up to three documents (one across a shard boundary, one inside a shard, the last one; two
    heads) against the oracle's dense closed form and its autograd in float64: out, dq, dk and dv; (2) 64 random rows of out and dq recomputed from the definition in float64; (3) a ring of 8 agrees with
    one device on out / dq / dk / dv; (4) documents are isolated bitwise in the gradients too: changing one
    document's keys, values and cotangents changes no other document's dq, dk or dv."""
    B, S, H, D, n = 1, 131072, 32, 128, 8
    print("131k ring 8 full size", flush=True)
    g = torch.Generator(device=DEV).manual_seed(44)
    mk = lambda: torch.randn(B, S, H, D, device=DEV, generator=g).bfloat16()
    q, k, v, do = mk(), mk(), mk(), mk()
    seg = packed_segment_ids(1, S, 4096, seed=45).to(DEV)
    bias = torch.randn(1, 1, 1, S, device=DEV, generator=g)
    kw = kwargs(512, 512, 1)

    def run(k_, v_, do_, ring):
        qd, kd, vd = (t.detach().requires_grad_(True) for t in (q, k_, v_))
        with ra.ring_axis("sp", ring):
            out = ra.ringattention(qd, kd, vd, bias, seg, None, axis_name="sp", float32_logits=True,
                                   blockwise_kwargs=kw)
            out.backward(do_)
        return out.detach(), (qd.grad, kd.grad, vd.grad)

    out8, g8 = run(k, v, do, n)
    assert not torch.isnan(out8).any()
    _document_dense_check(q, k, v, do, bias, seg[0], out8, g8, (0, 17), "131k ring 8")
    _sampled_rows_check(q, k, v, do, bias, seg[0], out8, g8[0], 64, 46, "131k ring 8")
    out1, g1 = run(k, v, do, 1)
    for name, a, b in zip(("out", "dq", "dk", "dv"), (out8,) + g8, (out1,) + g1):
        assert not torch.isnan(a).any(), name
        ma, rl = errors(a, b)
        assert ma <= 2e-2 and rl <= 1e-2, (name, ma, rl)
    del g1, out1
    ids = seg[0]
    doc = int(ids[S // 2 + 1234])
    inside = ids == doc
    k2, v2, do2 = k.clone(), v.clone(), do.clone()
    k2[:, inside] = 2.0
    v2[:, inside] = 5.0
    do2[:, inside] = -3.0
    _, g8b = run(k2, v2, do2, n)
    for name, a, b in zip(("dq", "dk", "dv"), g8b, g8):
        assert torch.equal(a[:, ~inside], b[:, ~inside]), name
        assert not torch.equal(a[:, inside], b[:, inside]), name


def test_one_million_positions_ring8():
    """B1 H32 S1048576 D128 bf16, causal, a ring of 8 shards of 131072 positions, chunks 512 / 512, forward and
    backward: the context length the reference was written for, on one GPU (8.6 GB per operand; element offsets pass
    2^32 and byte offsets 2^33, so every index of the path has to be 64-bit).  48 random rows of out and dq, and the last
    row, recomputed from the definition in float64; dk and dv of key rows near the end of the sequence (head 31,
    where the offsets are largest) against a float64 dense reference over the query rows that see them."""
    B, S, H, D, n = 1, 1 << 20, 32, 128, 8
    print("1M positions ring 8", flush=True)
    g = torch.Generator(device=DEV).manual_seed(51)
    mk = lambda: torch.randn(B, S, H, D, device=DEV, generator=g).bfloat16()
    q, k, v, do = mk(), mk(), mk(), mk()
    kw = kwargs(512, 512, 1)
    qd, kd, vd = (t.detach().requires_grad_(True) for t in (q, k, v))
    t0 = time.time()
    with ra.ring_axis("sp", n):
        out = ra.ringattention(qd, kd, vd, None, None, None, axis_name="sp", float32_logits=True, blockwise_kwargs=kw)
        out.backward(do)
    torch.cuda.synchronize()
    print("1M positions: forward + backward %.1f s, kernels %s" % (time.time() - t0, ra.kernel_family_of_last_call()),
          flush=True)
    out, dq, dk, dv = out.detach(), qd.grad, kd.grad, vd.grad
    for name, t in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
        assert torch.isfinite(t[:, -4096:]).all() and torch.isfinite(t[:, :4096]).all(), name
    ids = torch.zeros(S, dtype=torch.int32, device=DEV)
    zero_bias = torch.zeros(1, 1, 1, S, device=DEV)
    _sampled_rows_check(q, k, v, do, zero_bias, ids, out, dq, 48, 52, "1M ring 8")
    # the last row of the last head by name
    h, pos = H - 1, S - 1
    kk, vv = k[0, :, h].double(), v[0, :, h].double()
    p = torch.softmax(kk @ q[0, pos, h].double() / D ** 0.5, dim=0)
    o = p @ vv
    gg = do[0, pos, h].double()
    dq_row = (p * (vv @ gg - gg @ o)) @ kk / D ** 0.5
    assert float((out[0, pos, h].double() - o).abs().max()) <= 2e-2
    assert float((dq[0, pos, h].double() - dq_row).abs().max()) <= 2e-2
    # dk, dv of the last 2048 key rows of head 31: only the query rows from there on see them
    j0 = S - 2048
    dk_ref = torch.zeros(S - j0, D, dtype=torch.float64, device=DEV)
    dv_ref = torch.zeros_like(dk_ref)
    posn = torch.arange(S, device=DEV)
    for r0 in range(j0, S, 256):
        r1 = r0 + 256
        qq, gg = q[0, r0:r1, h].double(), do[0, r0:r1, h].double()
        logits = qq @ kk[:r1].T / D ** 0.5
        logits = logits.masked_fill(posn[None, :r1] > posn[r0:r1, None], float("-inf"))
        p = torch.softmax(logits, dim=1)
        o = p @ vv[:r1]
        ds = p * (gg @ vv[:r1].T - (gg * o).sum(dim=1, keepdim=True))
        dk_ref[:r1 - j0] += ds[:, j0:].T @ qq / D ** 0.5
        dv_ref[:r1 - j0] += p[:, j0:].T @ gg
        del logits, p, ds
    for name, a, b in (("dk", dk[0, j0:, h], dk_ref), ("dv", dv[0, j0:, h], dv_ref)):
        ma, rl = assert_close(a, b, torch.bfloat16, "1M ring 8 head 31 " + name)
        print("1M ring 8, last 2048 keys of head 31", name, "max-abs %.2e rel-L2 %.2e" % (ma, rl), flush=True)


def test_causal_32k_all_heads_sampled_rows():
    """B1 H32 S32768 D128 bf16 causal, chunks 512/512 - all 32 heads of the headline configuration: 64 random rows of
    out and dq recomputed from the definition in float64, and head 9 (of 32) of dk / dv against a float64 dense
    reference over the whole sequence."""
    B, S, H, D = 1, 32768, 32, 128
    print("32k causal all heads", flush=True)
    g = torch.Generator(device=DEV).manual_seed(47)
    mk = lambda: torch.randn(B, S, H, D, device=DEV, generator=g).bfloat16()
    q, k, v, do = mk(), mk(), mk(), mk()
    kw = kwargs(512, 512, 1)
    qd, kd, vd = (t.detach().requires_grad_(True) for t in (q, k, v))
    out = ra.ringattention(qd, kd, vd, None, None, None, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    out.backward(do)
    ids = torch.zeros(S, dtype=torch.int32, device=DEV)
    zero_bias = torch.zeros(1, 1, 1, S, device=DEV)
    _sampled_rows_check(q, k, v, do, zero_bias, ids, out.detach(), qd.grad, 64, 48, "32k causal")
    # dk, dv of one head: dense float64 on the GPU, query rows in slabs of 2048 (a slab's logits are 2048 x 32768)
    h = 9
    kk, vv = k[0, :, h].double(), v[0, :, h].double()
    dk_ref, dv_ref = torch.zeros_like(kk), torch.zeros_like(vv)
    pos = torch.arange(S, device=DEV)
    for r0 in range(0, S, 2048):
        r1 = r0 + 2048
        qq, gg = q[0, r0:r1, h].double(), do[0, r0:r1, h].double()
        logits = qq @ kk[:r1].T / D ** 0.5
        logits = logits.masked_fill(pos[None, :r1] > pos[r0:r1, None], float("-inf"))
        p = torch.softmax(logits, dim=1)
        o = p @ vv[:r1]
        ds = p * (gg @ vv[:r1].T - (gg * o).sum(dim=1, keepdim=True))
        dk_ref[:r1] += ds.T @ qq / D ** 0.5
        dv_ref[:r1] += p.T @ gg
    for name, a, b in (("dk", kd.grad[0, :, h], dk_ref), ("dv", vd.grad[0, :, h], dv_ref)):
        ma, rl = assert_close(a, b, torch.bfloat16, "32k causal head 9 " + name)
        print("32k causal head 9", name, "max-abs %.2e rel-L2 %.2e" % (ma, rl), flush=True)


def test_decode_full_cache_every_batch_row():
    """B16 H32 D128 bf16, cache of 262144 positions (+ one spare key chunk): 69 GB of K and V, the configuration the
    decode bandwidth is quoted on.  Every batch row against a dense fp32 softmax computed on the GPU in slabs; batch
    row 5 against the CPU oracle."""
    B, Lf, H, D, kc = 16, 262144, 32, 128, 512
    L = Lf + kc
    print("decode B16 full cache", flush=True)
    g = torch.Generator(device=DEV).manual_seed(46)
    k = torch.empty(B, L, H, D, dtype=torch.bfloat16, device=DEV)
    v = torch.empty(B, L, H, D, dtype=torch.bfloat16, device=DEV)
    for b in range(B):      # filled row by row to bound the fp32 temporaries
        k[b].copy_(torch.randn(L, H, D, device=DEV, generator=g))
        v[b].copy_(torch.randn(L, H, D, device=DEV, generator=g))
    # queries scaled so that the logits have a standard deviation of 3: some keys dominate their row
    q = (torch.randn(B, 1, H, D, device=DEV, generator=g) * 3.0).bfloat16()
    kw = kwargs(1, kc, 1)
    cache_idx = Lf + 77
    ci = torch.tensor(cache_idx, dtype=torch.int32, device=DEV)
    out = ra.ringattention(q, k, v, None, None, ci, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    torch.cuda.synchronize()
    assert not torch.isnan(out).any()
    n_att = cache_idx + 1
    slab = 32768
    for b in range(B):
        qb = q[b, 0].float()                                    # (H, D)
        m = torch.full((H,), float("-inf"), device=DEV)
        l = torch.zeros(H, device=DEV)
        acc = torch.zeros(H, D, device=DEV)
        for s0 in range(0, n_att, slab):
            s1 = min(s0 + slab, n_att)
            sc = torch.einsum("hd,khd->hk", qb, k[b, s0:s1].float()) / D ** 0.5
            m_new = torch.maximum(m, sc.amax(dim=1))
            p = torch.exp(sc - m_new[:, None])
            corr = torch.exp(m - m_new)
            l = l * corr + p.sum(dim=1)
            acc = acc * corr[:, None] + torch.einsum("hk,khd->hd", p, v[b, s0:s1].float())
            m = m_new
        ref = acc / l[:, None]
        ma, rl = errors(out[b, 0], ref)
        assert ma <= 2e-2 and rl <= 1e-2, ("batch row", b, ma, rl)
    # one batch row through the CPU oracle (the reference's chunk loop over 513 key chunks)
    b = 5
    t0 = time.time()
    ref = O.ring_attention(q[b:b + 1].cpu(), k[b:b + 1].cpu(), v[b:b + 1].cpu(), None, None, cache_idx, 1, True,
                           oracle_kwargs(kw))
    secs = time.time() - t0
    ma, rl = assert_close(out[b:b + 1], ref, torch.bfloat16, "decode row 5 vs oracle")
    print("decode B16 row 5 vs oracle: %.1f s, max-abs %.2e rel-L2 %.2e" % (secs, ma, rl), flush=True)


@pytest.mark.parametrize("impl", ["mfma", "generic"])
def test_blockwise_q_len_differs_from_kv_len(impl):
    """_blockwise_attention_fwd / _bwd semantics with q_len != kv_len (ringattention_jax.py:101-103 takes the two
    lengths separately): 512 queries against 2048 keys, and 1024 queries against 256 keys, causal by global
    position (most of the second case's rows see every key; the first case's keys after position 511 are
    masked for every row)."""
    D, H = 128, 2
    for Sq, Skv, qc, kc in ((512, 2048, 128, 256), (1024, 256, 256, 128)):
        print("q_len != kv_len", impl, Sq, Skv, flush=True)
        q, k, v, do = make_qkv(1, Sq, H, D, dtype=torch.bfloat16, seed=Sq, Skv=Skv)
        kw = kwargs(qc, kc, 1, impl=impl)
        ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, None, None, None, 1, kw)
        out, grads = _hip(q, k, v, do, None, None, 1, kw)
        _compare("q %d kv %d %s" % (Sq, Skv, impl), out, grads, ref_out, ref_grads, 0.0)
        if impl == "mfma":                  # the same lengths in fp32, on the fp32 matrix-core kernels
            qf, kf, vf, dof = (t.float() for t in (q, k, v, do))
            ref_out, ref_grads = oracle_fwd_bwd(qf, kf, vf, dof, None, None, None, 1, kw)
            out, grads = _hip(qf, kf, vf, dof, None, None, 1, dict(kw, dtype=torch.float32))
            assert_close(out, ref_out, torch.float32, "fp32 out")
            for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
                assert_close(a, b, torch.float32, "fp32 " + name)


@pytest.mark.parametrize("impl,dtype", [("mfma", torch.bfloat16), ("generic", torch.float32), ("mfma", torch.float32)])
@pytest.mark.parametrize("cache_idx", [0, 300, 512, 1000, 1536])
def test_cache_idx_with_several_query_tokens(cache_idx, impl, dtype):
    """cache_idx with q_len > 1 (ringattention_jax.py:34-35): the query chunks start at global chunk
    cache_idx // query_chunk_size, so a block of 256 new tokens attends causally into a cache buffer of 2048
    positions; forward and backward against the oracle (the backward takes the same start, :72-73)."""
    Sq, L, H, D, qc, kc = 256, 2048, 2, 128, 128, 128
    print("cache_idx with q_len 256", cache_idx, impl, flush=True)
    q, k, v, do = make_qkv(1, Sq, H, D, dtype=dtype, seed=cache_idx + 1, Skv=L)
    kw = kwargs(qc, kc, 1, impl=impl)
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, None, None, cache_idx, 1, kw)
    for ci in (cache_idx, torch.tensor(cache_idx, dtype=torch.int32, device=DEV)):
        qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
        out = ra.ringattention(qd, kd, vd, None, None, ci, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
        out.backward(do.to(DEV))
        torch.cuda.synchronize()
        assert_close(out, ref_out, dtype, "out")
        for name, a, b in zip(("dq", "dk", "dv"), (qd.grad, kd.grad, vd.grad), ref_grads):
            assert_close(a, b, dtype, name)


def test_float32_logits_false_is_accepted():
    """float32_logits=False (ringattention_jax.py:18-19 then skips the fp32 cast of q and k): this path computes the
    logits in fp32 either way, so the result is that of float32_logits=True, and within the bf16 tolerance of the
    oracle run with the flag off."""
    B, S, H, D = 1, 1024, 2, 128
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=50)
    kw = kwargs(256, 256, 1)
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    a = ra.ringattention(qd, kd, vd, None, None, None, axis_name=None, float32_logits=False, blockwise_kwargs=kw)
    b = ra.ringattention(qd, kd, vd, None, None, None, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    assert torch.equal(a, b)
    ref = O.ring_attention(q, k, v, None, None, None, 1, False, oracle_kwargs(kw))
    # the oracle then keeps logits, running max / sum and the numerator in bf16 (2^-8 relative rounding in every
    # chunk step): it sits this far from its own fp32 run, so the bar is looser than the fp32-logit one
    ma, rl = errors(a, ref)
    assert ma <= 6e-2 and rl <= 3e-2, (ma, rl)


def test_fp32_16k_ring4_matches_oracle():
    """fp32 q, k, v on the matrix-core kernels at B1 H2 S16384 D128, ring of 4, packed documents and a bias, chunks
    512/512: the fp32 bar (max-abs 1e-4, relative L2 1e-2) at a length where every workgroup streams hundreds of
    tiles."""
    B, S, H, D, n = 1, 16384, 2, 128, 4
    print("oracle parity, fp32 16k ring 4", flush=True)
    q, k, v, do = make_qkv(B, S, H, D, dtype=torch.float32, seed=44, scale=D ** -0.25)
    seg = packed_segment_ids(B, S, 3000, seed=45)
    bias = torch.randn(1, 1, 1, S, generator=torch.Generator().manual_seed(46))
    kw = kwargs(512, 512, 1, dtype=torch.float32, impl="mfma")
    t0 = time.time()
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    secs = time.time() - t0
    out, grads = _hip(q, k, v, do, bias, seg, n, kw)
    rows = [("out",) + assert_close(out, ref_out, torch.float32, "fp32 16k out")]
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        rows.append((name,) + assert_close(a, b, torch.float32, "fp32 16k " + name))
    print("fp32 16k ring 4: oracle %.1f s;" % secs, "; ".join("%s max-abs %.2e rel-L2 %.2e" % r for r in rows), flush=True)


_SWIGLU_ORACLE = {}     # tokens -> the oracle's (y, dx, dw1, dw2, dw3) and wall time: the cases of a size share inputs


@pytest.mark.parametrize("tokens,chunk,launch,policy,tile", [
    (2048, 2048, None, "nothing_saveable", None),          # one 2048-token chunk per launch: the library picks 256 x 128
    (2048, 2048, None, "save_preactivations", 0),          # the same chunk with the 256 x 256 tile kernel forced
    (16384, 2048, 16384, "nothing_saveable", None),        # eight chunks sharing one launch: 256 x 256 tiles
    (16384, 2048, 16384, "save_preactivations", 3),        # ... and with the 256 x 128 tile kernel forced
])
def test_swiglu_llama7b_shape_matches_oracle(tokens, chunk, launch, policy, tile):
    """blockwise_feedforward over SwiGLU(4096, 11008) - the shape of BASELINE configuration 4, K = 11008 being 172
    slabs of 64 and 43 column tiles of 256 - forward and backward against the oracle's formula under fp32 autograd
    on the CPU (ringattention_jax.py:333-352): bf16 outputs of fp32-accumulated products, relative L2 <= 1e-2 and
    max-abs within 2e-2 of the output's scale."""
    from tests.test_gpu_feedforward import rel_ok
    d, f = 4096, 11008
    print("swiglu case", dict(tokens=tokens, chunk=chunk, launch=launch, policy=policy, tile=tile), flush=True)
    g = torch.Generator().manual_seed(tokens)
    x = torch.randn(1, tokens, d, generator=g).bfloat16()
    dy = torch.randn(1, tokens, d, generator=g).bfloat16()
    torch.manual_seed(4096 + tokens)                       # the weights are drawn on the device from the global stream
    ff = ra.SwiGLU(d, f, device=DEV, init_std=0.02, gemm_tile=tile)
    xd = x.to(DEV).requires_grad_(True)
    y = ra.blockwise_feedforward(ff, xd, chunk, policy=policy, launch_tokens=launch)
    y.backward(dy.to(DEV))
    torch.cuda.synchronize()
    if tokens not in _SWIGLU_ORACLE:
        t0 = time.time()
        w1, w2, w3 = (w.detach().float().cpu().requires_grad_(True) for w in (ff.w1, ff.w2, ff.w3))
        xr = x.float().requires_grad_(True)
        yr = O.blockwise_feedforward(lambda h: O.swiglu(h, w1, w2, w3), xr, chunk)
        yr.backward(dy.float())
        _SWIGLU_ORACLE.clear()                             # one size at a time: a gigabyte of gradients each
        _SWIGLU_ORACLE[tokens] = ((yr.detach(), xr.grad, w1.grad, w2.grad, w3.grad), time.time() - t0,
                                  ff.w1.detach().clone())
    ref, secs, w1_seen = _SWIGLU_ORACLE[tokens]
    assert torch.equal(w1_seen, ff.w1.detach()), "the cases of one size must share their weights"
    print("  oracle %.1f s" % secs, flush=True)
    for name, a, b in zip(("y", "dx", "dw1", "dw2", "dw3"), (y, xd.grad, ff.w1.grad, ff.w2.grad, ff.w3.grad), ref):
        ma, rl = errors(a, b)
        print("  %-3s max-abs %.3e rel-L2 %.3e (scale %.3e)" % (name, ma, rl, float(b.abs().max())), flush=True)
        rel_ok(a, b, name)
