"""Parity of the steps either side of the hot path (rope_kv_append before a decode step, rmsnorm_residual around
the FFN) with the CPU oracle.  Bars: the cache append is bitwise outside the rotated key; rotated values within one
bf16 rounding step of the oracle's fp64-angle rotation (fp32: 1e-5 relative); RMSNorm outputs and gradients
max-abs within 2e-2 of the output scale and relative L2 <= 1e-2 (bf16 in and out, fp32 arithmetic)."""
import pytest
import torch

import ringattention_amd as ra
from oracle import ringattention_oracle as O
from tests.util import errors, kwargs, oracle_kwargs

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("style", ["adjacent", "half"])
@pytest.mark.parametrize("pos", [0, 37, 262143])
def test_rope_kv_append_matches_oracle(dtype, style, pos):
    # the buffer must hold position pos: a long one gets a single batch row and head
    B, H, D = (2, 4, 128) if pos < 64 else (1, 1, 128)
    L = 64 if pos < 64 else pos + 1
    print("rope", dtype, style, pos, flush=True)
    g = torch.Generator().manual_seed(pos + 1)
    q, kn, vn = (torch.randn(B, 1, H, D, generator=g).to(dtype) for _ in range(3))
    kc, vc = torch.randn(B, L, H, D, generator=g).to(dtype), torch.randn(B, L, H, D, generator=g).to(dtype)
    qr_ref = O.rope_rotate(q.double(), pos, style=style)
    kr_ref = O.rope_rotate(kn.double(), pos, style=style)
    kd, vd = kc.to(DEV), vc.to(DEV)
    ci = torch.tensor(pos, dtype=torch.int32, device=DEV)
    qr = ra.rope_kv_append(q.to(DEV), kn.to(DEV), vn.to(DEV), kd, vd, ci, rope_style=style)
    tol = 2 ** -7 if dtype == torch.bfloat16 else 1e-5
    scale = float(q.abs().max()) * 1.5
    assert float((qr.double().cpu() - qr_ref).abs().max()) <= tol * scale
    assert float((kd[:, pos].double().cpu() - kr_ref[:, 0]).abs().max()) <= tol * scale
    assert torch.equal(vd[:, pos].cpu(), vn[:, 0])                       # the value is copied
    kd_h, vd_h = kd.cpu(), vd.cpu()                                      # every other position is untouched
    kd_h[:, pos], vd_h[:, pos] = kc[:, pos], vc[:, pos]
    assert torch.equal(kd_h, kc) and torch.equal(vd_h, vc)
    # a host position gives the same bits as the device scalar
    kd2, vd2 = kc.to(DEV), vc.to(DEV)
    qr2 = ra.rope_kv_append(q.to(DEV), kn.to(DEV), vn.to(DEV), kd2, vd2, pos, rope_style=style)
    assert torch.equal(qr2, qr) and torch.equal(kd2, kd) and torch.equal(vd2, vd)


def test_rope_kv_append_then_decode_equals_oracle_step():
    """The decode step as a model runs it: rotate + append at cache_idx, then ringattention(..., cache_idx)."""
    B, L, H, D, kc_sz, pos = 2, 512, 4, 128, 64, 300
    g = torch.Generator().manual_seed(9)
    q, kn, vn = (torch.randn(B, 1, H, D, generator=g).bfloat16() for _ in range(3))
    kc, vc = torch.randn(B, L, H, D, generator=g).bfloat16(), torch.randn(B, L, H, D, generator=g).bfloat16()
    kw = kwargs(1, kc_sz, 1)
    qr_ref, kc_ref, vc_ref = O.rope_kv_append(q.float(), kn.float(), vn.float(), kc.float(), vc.float(), pos)
    qr_ref, kc_ref = qr_ref.bfloat16(), kc_ref.bfloat16()
    ref = O.ring_attention(qr_ref, kc_ref, vc_ref.bfloat16(), None, None, pos, 1, True, oracle_kwargs(kw))
    kd, vd = kc.to(DEV), vc.to(DEV)
    ci = torch.tensor(pos, dtype=torch.int32, device=DEV)
    qr = ra.rope_kv_append(q.to(DEV), kn.to(DEV), vn.to(DEV), kd, vd, ci)
    out = ra.ringattention(qr, kd, vd, None, None, ci, axis_name=None, float32_logits=True, blockwise_kwargs=kw)
    ma, rl = errors(out, ref)
    assert ma <= 2e-2 and rl <= 1e-2


def test_rope_kv_append_rejects_bad_arguments():
    B, L, H, D = 1, 8, 2, 16
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        ra.rope_kv_append(z(B, 1, H, D), z(B, 1, H, D), z(B, 1, H, D), z(B, L, H, D), z(B, L, H, D), L)   # outside
    with pytest.raises(ValueError):
        ra.rope_kv_append(z(B, 2, H, D), z(B, 2, H, D), z(B, 2, H, D), z(B, L, H, D), z(B, L, H, D), 0)   # two tokens
    with pytest.raises(ValueError):
        ra.rope_kv_append(z(B, 1, H, D), z(B, 1, H, D), z(B, 1, H, D), z(B, L, H, D), z(B, L, H, D), 0, rope_style="x")


@pytest.mark.parametrize("shape", [(3, 40, 256), (1, 7, 4096), (2, 5, 5120), (1, 3, 8192), (1, 4, 72)])
@pytest.mark.parametrize("with_residual", [True, False])
def test_rmsnorm_residual_matches_oracle(shape, with_residual):
    B, S, d = shape
    print("rmsnorm", shape, with_residual, flush=True)
    g = torch.Generator().manual_seed(d + S)
    x = torch.randn(B, S, d, generator=g).bfloat16()
    r = torch.randn(B, S, d, generator=g).bfloat16() if with_residual else None
    w = (1.0 + 0.1 * torch.randn(d, generator=g)).bfloat16()
    dn, dres = torch.randn(B, S, d, generator=g).bfloat16(), torch.randn(B, S, d, generator=g).bfloat16()
    xr = x.float().requires_grad_(True)
    rr = r.float().requires_grad_(True) if with_residual else None
    wr = w.float().requires_grad_(True)
    y_ref, n_ref = O.rmsnorm_residual(xr, rr, wr, eps=1e-6, stream_dtype=torch.bfloat16 if with_residual else None)
    # the rounding of the stream is not differentiated: gradients are those of the unrounded sum
    y_lin, n_lin = O.rmsnorm_residual(xr, rr, wr, eps=1e-6)
    ((n_lin * dn.float()).sum() + (y_lin * dres.float()).sum()).backward()
    xd = x.to(DEV).requires_grad_(True)
    rd = r.to(DEV).requires_grad_(True) if with_residual else None
    wd = w.to(DEV).requires_grad_(True)
    y, n = ra.rmsnorm_residual(xd, rd, wd, eps=1e-6)
    ((n.float() * dn.to(DEV).float()).sum() + (y.float() * dres.to(DEV).float()).sum()).backward()

    def ok(a, b, what):
        ma, rl = errors(a, b)
        sc = max(1.0, float(b.detach().abs().max()))
        assert rl <= 1e-2 and ma <= 2e-2 * sc, "%s: max-abs %.3e (scale %.2e) rel %.3e" % (what, ma, sc, rl)

    ok(y, y_ref, "y")
    ok(n, n_ref, "normed")
    ok(xd.grad, xr.grad, "dx")
    if with_residual:
        ok(rd.grad, rr.grad, "dresidual")
    ok(wd.grad, wr.grad, "dweight")


def test_rmsnorm_rejects_unsupported_rows():
    x = torch.zeros(2, 100, dtype=torch.bfloat16, device=DEV)          # 100 is not a multiple of 8
    with pytest.raises(NotImplementedError):
        ra.rmsnorm_residual(x, None, torch.ones(100, dtype=torch.bfloat16, device=DEV))
    x = torch.zeros(2, 16384, dtype=torch.bfloat16, device=DEV)        # longer than the kernels' 8192
    with pytest.raises(NotImplementedError):
        ra.rmsnorm_residual(x, None, torch.ones(16384, dtype=torch.bfloat16, device=DEV))


def test_decode_step_replays_from_a_hip_graph():
    """The decode step (rotate + append, then attend) captured once in a HIP graph and replayed for several
    positions: cache_idx is read from device memory by both kernels, so one graph serves every step.  Each replay
    is checked against the same step run eagerly on a copy of the caches."""
    B, L, H, D, kc = 2, 1024, 4, 128, 128
    g = torch.Generator(device=DEV).manual_seed(11)
    rnd = lambda *s: torch.randn(*s, device=DEV, generator=g).bfloat16()
    k_cache, v_cache = rnd(B, L, H, D), rnd(B, L, H, D)
    q, kn, vn = rnd(B, 1, H, D), rnd(B, 1, H, D), rnd(B, 1, H, D)
    qr, out = torch.empty_like(q), torch.empty_like(q)
    ci = torch.zeros(1, dtype=torch.int32, device=DEV)
    kw = kwargs(1, kc, 1)

    ws = ra.decode_workspace(q, k_cache)       # owned by the caller: it must outlive every replay of the graph

    def step(kc_, vc_, qr_, out_):
        ra.rope_kv_append(q, kn, vn, kc_, vc_, ci, q_out=qr_)
        ra.decode_attention(qr_, kc_, vc_, None, None, ci, kw, out=out_, workspace=ws)

    ci.fill_(500)
    step(k_cache.clone(), v_cache.clone(), torch.empty_like(q), torch.empty_like(q))     # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(k_cache, v_cache, qr, out)
    for pos in (500, 501, 777, 1023, 130):
        print("graph replay at", pos, flush=True)
        ci.fill_(pos)
        q.copy_(rnd(B, 1, H, D)); kn.copy_(rnd(B, 1, H, D)); vn.copy_(rnd(B, 1, H, D))
        k_ref, v_ref = k_cache.clone(), v_cache.clone()
        qr_ref, out_ref = torch.empty_like(q), torch.empty_like(q)
        step(k_ref, v_ref, qr_ref, out_ref)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(torch.nan_to_num(out), torch.nan_to_num(out_ref))
        assert torch.equal(qr, qr_ref) and torch.equal(k_cache, k_ref) and torch.equal(v_cache, v_ref)


def test_mfma_rate_probe_computes_what_it_says():
    """The measurement probe really issues its MFMAs: with 0.5 and 0.25 everywhere an instruction adds 16 * 0.125 = 2
    to each of its 1024 results, an accumulator takes 16 instructions per iteration, and a lane sums 4 x 16 results."""
    from ringattention_amd import _lib as L
    iters, wgs = 4, 8
    sink = torch.zeros(wgs * 256, dtype=torch.float32, device=DEV)
    L.check(L.load_probe().ra_mfma_rate_probe(sink.data_ptr(), wgs, iters, 0, torch.cuda.current_stream().cuda_stream),
            "ra_mfma_rate_probe")
    torch.cuda.synchronize()
    assert bool((sink == 2.0 * 16 * iters * 64).all())
    for mode in (1, 2):
        L.check(L.load_probe().ra_mfma_rate_probe(sink.data_ptr(), wgs, iters, mode, torch.cuda.current_stream().cuda_stream),
                "ra_mfma_rate_probe")
        torch.cuda.synchronize()
        assert bool(torch.isfinite(sink).all()) and float(sink.abs().max()) > 0
