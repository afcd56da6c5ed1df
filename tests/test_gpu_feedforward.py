"""Parity of the bf16 GEMM and SwiGLU kernels and of blockwise_feedforward with the CPU oracle
(torch fp32 matmul / autograd of the same formula).  Tolerance: bf16 outputs of fp32-accumulated
products, relative L2 <= 1e-2 and max-abs within 2e-2 of the output scale."""
import pytest
import torch

import ringattention_amd as ra
from oracle import ringattention_oracle as O
from tests.util import errors

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rel_ok(got, ref, what, rel=1e-2, scaled_abs=2e-2):
    ma, rl = errors(got, ref)
    scale = float(ref.detach().float().abs().max())
    assert rl <= rel and ma <= scaled_abs * max(scale, 1.0), "%s: max-abs %.3e (scale %.3e), rel-L2 %.3e" % (
        what, ma, scale, rl)


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("shape", [(128, 128, 64), (256, 384, 192), (512, 128, 1024)])
def test_gemm_layouts(ta, tb, shape):
    M, N, K = shape
    print("gemm", ta, tb, shape, flush=True)
    g = torch.Generator().manual_seed(M + N + K)
    A = torch.randn((K, M) if ta else (M, K), generator=g).bfloat16()
    B = torch.randn((N, K) if tb else (K, N), generator=g).bfloat16()
    ref = (A.float().t() if ta else A.float()) @ (B.float().t() if tb else B.float())
    out = ra.gemm_bf16(A.to(DEV), B.to(DEV), trans_a=ta, trans_b=tb)
    rel_ok(out, ref, "bf16 out")
    acc = torch.ones(M, N, dtype=torch.float32, device=DEV)
    ra.gemm_bf16(A.to(DEV), B.to(DEV), trans_a=ta, trans_b=tb, out=acc, accumulate=True)
    assert errors(acc, ref + 1.0)[1] < 1e-5


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("tile", [0, 1, 2, 3])
@pytest.mark.parametrize("shape", [(768, 512, 320), (1280, 256, 128), (512, 384, 448), (256, 256, 64), (256, 512, 192),
                                   (512, 256, 256), (256, 256, 576)])
def test_gemm_every_tile_kernel(ta, tb, tile, shape):
    """Each tile kernel (0: 256 x 256 over four wavefronts, 1: 256 x 128 over eight, 2: 128 x 128, 3: 256 x 128 over four) on shapes whose tile
    counts are no multiple of the 8 XCDs or of the tile-row group, so the workgroup -> tile order and its
    surplus workgroups are exercised, and on K of 1 to 9 slabs of 64 (the 4-wavefront kernels rotate their LDS buffers
    every six slabs and finish with up to five single steps); ra_gemm_bf16_tile names the tile kernel that ra_gemm_bf16 would pick itself."""
    M, N, K = shape
    print("gemm tile", tile, ta, tb, shape, flush=True)
    g = torch.Generator().manual_seed(M + N + K + tile)
    A = torch.randn((K, M) if ta else (M, K), generator=g).bfloat16()
    B = torch.randn((N, K) if tb else (K, N), generator=g).bfloat16()
    ref = (A.float().t() if ta else A.float()) @ (B.float().t() if tb else B.float())
    out = ra.gemm_bf16(A.to(DEV), B.to(DEV), trans_a=ta, trans_b=tb, tile=tile)
    rel_ok(out, ref, "bf16 out")
    acc = torch.ones(M, N, dtype=torch.float32, device=DEV)
    ra.gemm_bf16(A.to(DEV), B.to(DEV), trans_a=ta, trans_b=tb, out=acc, accumulate=True, tile=tile)
    assert errors(acc, ref + 1.0)[1] < 1e-5


def test_gemm_random_shapes():
    """Sixty seeded random shapes (M, N multiples of 128 up to 1536, K of 1 to 40 slabs of 64), layouts, tile kernels
    and output modes against torch's fp32 product."""
    import random
    rnd = random.Random(7)
    for case in range(60):
        M, N, K = 128 * rnd.randint(1, 12), 128 * rnd.randint(1, 12), 64 * rnd.randint(1, 40)
        ta, tb = rnd.random() < 0.5, rnd.random() < 0.5
        tile = rnd.choice([None, 0, 1, 2, 3])
        acc = rnd.random() < 0.4
        g = torch.Generator().manual_seed(case)
        A = torch.randn((K, M) if ta else (M, K), generator=g).bfloat16().to(DEV)
        B = torch.randn((N, K) if tb else (K, N), generator=g).bfloat16().to(DEV)
        ref = (A.float().t() if ta else A.float()) @ (B.float().t() if tb else B.float())
        what = "case %d: %d x %d x %d ta %s tb %s tile %s acc %s" % (case, M, N, K, ta, tb, tile, acc)
        if acc:
            out = torch.full((M, N), 0.5, dtype=torch.float32, device=DEV)
            ra.gemm_bf16(A, B, trans_a=ta, trans_b=tb, out=out, accumulate=True, tile=tile)
            assert errors(out - 0.5, ref)[1] < 1e-5, what
        else:
            rel_ok(ra.gemm_bf16(A, B, trans_a=ta, trans_b=tb, tile=tile), ref, what)


def test_gemm_operand_beyond_two_gib():
    """A K-major operand of 2.3 GB (a weight gradient over 98304 tokens): the 4-wavefront kernels read every slab
    through a descriptor of its own, so the size of an operand does not matter; checked against fp32 sums of
    torch's products of 8192-row slices."""
    K, M, N = 98304, 11776, 256
    g = torch.Generator(device=DEV).manual_seed(5)
    A = torch.randn(K, M, device=DEV, generator=g).to(torch.bfloat16)          # stored (K, M): trans_a
    B = torch.randn(K, N, device=DEV, generator=g).to(torch.bfloat16)
    assert A.numel() * 2 > 2 ** 31
    ref = torch.zeros(M, N, dtype=torch.float32, device=DEV)
    for k0 in range(0, K, 8192):
        ref += A[k0:k0 + 8192].float().t() @ B[k0:k0 + 8192].float()
    for tile in (0, 3):
        out = torch.zeros(M, N, dtype=torch.float32, device=DEV)
        ra.gemm_bf16(A, B, trans_a=True, out=out, accumulate=True, tile=tile)
        assert errors(out, ref)[1] < 1e-5, (tile, errors(out, ref))
    # the other side: a row-wise B of 2.3 GB
    Bt = A                                                                      # as (N' = K, K' = M): stored (N, K)
    A2 = torch.randn(256, M, device=DEV, generator=g).to(torch.bfloat16)
    ref2 = A2.float() @ Bt[:16384].float().t()
    out2 = ra.gemm_bf16(A2, Bt, trans_b=True, tile=0)
    rel_ok(out2[:, :16384], ref2, "row-wise B beyond 2 GiB")


def test_gemm_rejects_ragged_shapes():
    A = torch.zeros(100, 64, dtype=torch.bfloat16, device=DEV)
    B = torch.zeros(64, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(NotImplementedError):
        ra.gemm_bf16(A, B)


@pytest.mark.parametrize("tile,shape", [(None, (256, 256, 384)), (0, (512, 256, 768)), (1, (512, 256, 768)), (3, (512, 256, 768))])
def test_swiglu_forward_backward_match_autograd(tile, shape):
    """SwiGLU forward and backward (including the two-operand-pair GEMM of dx and the fp32 accumulation of the
    weight gradients) with the library's own tile choice and with each of the large tile kernels forced."""
    T, d, f = shape
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, T, d, generator=g).bfloat16()
    dy = torch.randn(1, T, d, generator=g).bfloat16()
    ff = ra.SwiGLU(d, f, device=DEV, init_std=0.05, gemm_tile=tile)
    w1, w2, w3 = (w.detach().float().cpu().requires_grad_(True) for w in (ff.w1, ff.w2, ff.w3))
    xr = x.float().requires_grad_(True)
    yr = O.swiglu(xr, w1, w2, w3)
    yr.backward(dy.float())
    xd = x.to(DEV).requires_grad_(True)
    y = ff(xd)
    y.backward(dy.to(DEV))
    torch.cuda.synchronize()
    rel_ok(y, yr, "y")
    rel_ok(xd.grad, xr.grad, "dx")
    rel_ok(ff.w1.grad, w1.grad, "dw1")
    rel_ok(ff.w2.grad, w2.grad, "dw2")
    rel_ok(ff.w3.grad, w3.grad, "dw3")


def test_blockwise_feedforward_matches_oracle_and_unchunked():
    B, S, d, f, chunk = 2, 512, 128, 256, 128
    g = torch.Generator().manual_seed(1)
    x = torch.randn(B, S, d, generator=g).bfloat16()
    ff = ra.SwiGLU(d, f, device=DEV, init_std=0.05)
    w1, w2, w3 = (w.detach().float().cpu() for w in (ff.w1, ff.w2, ff.w3))
    ref = O.blockwise_feedforward(lambda h: O.swiglu(h, w1, w2, w3), x.float(), chunk)
    y = ra.blockwise_feedforward(ff, x.to(DEV), chunk)
    rel_ok(y, ref, "blockwise y")
    whole = ff(x.to(DEV))
    assert torch.equal(y, whole)     # token-wise: chunking does not change a single bit
    # a generic callable gets the reference's strided token groups
    seen = []

    def probe(h):
        seen.append(h.shape)
        return ff(h.contiguous())
    y2 = ra.blockwise_feedforward(probe, x.to(DEV), chunk)
    assert seen == [(B, chunk, d)] * (S // chunk)
    assert torch.equal(y2, whole)


def test_blockwise_feedforward_single_batch_scan_gradients():
    """B = 1 takes the one-node scan (weight gradients of all chunks accumulate in fp32 in the GEMM
    epilogue): forward equals the unchunked MLP bit for bit, gradients match fp32 autograd."""
    S, d, f, chunk = 1024, 128, 256, 256
    g = torch.Generator().manual_seed(5)
    x = torch.randn(1, S, d, generator=g).bfloat16()
    dy = torch.randn(1, S, d, generator=g).bfloat16()
    ff = ra.SwiGLU(d, f, device=DEV, init_std=0.05)
    xd = x.to(DEV).requires_grad_(True)
    y = ra.blockwise_feedforward(ff, xd, chunk)
    assert torch.equal(y, ff(x.to(DEV)))
    y.backward(dy.to(DEV))
    w1, w2, w3 = (w.detach().float().cpu().requires_grad_(True) for w in (ff.w1, ff.w2, ff.w3))
    xr = x.float().requires_grad_(True)
    O.swiglu(xr, w1, w2, w3).backward(dy.float())
    rel_ok(xd.grad, xr.grad, "dx")
    rel_ok(ff.w1.grad, w1.grad, "dw1")
    rel_ok(ff.w2.grad, w2.grad, "dw2")
    rel_ok(ff.w3.grad, w3.grad, "dw3")


def test_blockwise_feedforward_policies_give_the_same_bits():
    """policy="nothing_saveable" (the reference's default, ringattention_jax.py:334: the backward pass recomputes
    x w1 and x w3; also what None means) and the opt-in policy="save_preactivations" (they stay in memory) differ in
    memory and in two GEMMs per chunk, not in a single bit of y, dx or the weight gradients; nor does letting
    several chunks share a launch (launch_tokens)."""
    from ringattention_amd import feedforward as F
    S, d, f, chunk = 2048, 256, 512, 256
    g = torch.Generator().manual_seed(7)
    x = torch.randn(2, S, d, generator=g).bfloat16().to(DEV)
    dy = torch.randn(2, S, d, generator=g).bfloat16().to(DEV)
    ff = ra.SwiGLU(d, f, device=DEV, init_std=0.05)
    res = {}
    # launch_tokens 1024: several launches of four chunks, so that the kept buffers are sliced
    for policy, launch in (("nothing_saveable", None), ("save_preactivations", None), (None, None),
                           ("nothing_saveable", 1024), ("save_preactivations", 1024)):
        for prm in ff.parameters():
            prm.grad = None
        xd = x.clone().requires_grad_(True)
        y = ra.blockwise_feedforward(ff, xd, chunk, policy=policy, launch_tokens=launch)
        y.backward(dy)
        res[(policy, launch)] = (y.detach(), xd.grad, ff.w1.grad.clone(), ff.w2.grad.clone(), ff.w3.grad.clone())
    base = res[("nothing_saveable", None)]
    for key, val in res.items():
        for i, (a, b) in enumerate(zip(val, base)):
            if i >= 2 and key[1] != None:
                # weight gradients: fp32 sums over launches of another size round differently in the last bit
                assert errors(a, b)[1] < 1e-2, key
            else:
                assert torch.equal(a, b), key
    # the default is the reference's: nothing kept, one chunk per launch
    assert F._save_preactivations(None) is False and F._save_preactivations("nothing_saveable") is False
    assert F._save_preactivations("save_preactivations") is True
    assert F._slab_tokens(chunk, 16) == chunk and F._slab_tokens(chunk, 16, 1024) == 1024
    assert F._slab_tokens(chunk, 6, 1024) == 3 * chunk          # a whole number of chunks that divides the scan
    with pytest.raises(ValueError):
        ra.blockwise_feedforward(ff, x, chunk, policy="dots_saveable")
    # no gradient wanted: nothing is kept
    with torch.no_grad():
        assert torch.equal(ra.blockwise_feedforward(ff, x, chunk, policy="save_preactivations"), base[0])


def test_weight_gradients_of_grouped_launches():
    """weight_grad_chunks: the weight-gradient products of two (three, all) consecutive chunks in one launch each.
    y and dx are the same bits as with one launch per chunk; the weight gradients are the same sums in another fp32
    order (bar: relative L2 1e-2 against fp32 autograd, and 1e-3 against the per-chunk launches).  Seven chunks, so
    that the last group is short."""
    S, d, f, chunk = 7 * 256, 256, 512, 256
    g = torch.Generator().manual_seed(11)
    x = torch.randn(1, S, d, generator=g).bfloat16().to(DEV)
    dy = torch.randn(1, S, d, generator=g).bfloat16().to(DEV)
    ff = ra.SwiGLU(d, f, device=DEV, init_std=0.05)
    res = {}
    for grp in (1, 2, 3, 7, 100):
        for prm in ff.parameters():
            prm.grad = None
        xd = x.clone().requires_grad_(True)
        y = ra.blockwise_feedforward(ff, xd, chunk, weight_grad_chunks=grp)
        y.backward(dy)
        res[grp] = (y.detach(), xd.grad, ff.w1.grad.clone(), ff.w2.grad.clone(), ff.w3.grad.clone())
    w1, w2, w3 = (w.detach().float().cpu().requires_grad_(True) for w in (ff.w1, ff.w2, ff.w3))
    xr = x.float().cpu().requires_grad_(True)
    O.swiglu(xr, w1, w2, w3).backward(dy.float().cpu())
    for grp, val in res.items():
        assert torch.equal(val[0], res[1][0]) and torch.equal(val[1], res[1][1]), grp
        for i, ref in ((2, w1.grad), (3, w2.grad), (4, w3.grad)):
            rel_ok(val[i], ref, "dw group %d" % grp)
            assert errors(val[i], res[1][i])[1] < 1e-3, grp
    assert torch.equal(res[7][2], res[100][2])          # a group beyond the scan is the whole scan


@pytest.mark.parametrize("shape,tile", [((2048, 1536, 512), None), ((512, 768, 256), 0), ((512, 640, 192), 3), ((384, 256, 128), None)])
def test_gemm_pair_equals_two_launches_bitwise(shape, tile):
    """a = x w1 and b = x w3 as one launch over the tile columns of both: the bits of the two separate launches (a tile
    is computed the same whichever launch holds it), including a shape the four-wavefront kernels do not take."""
    from ringattention_amd.feedforward import gemm_bf16_pair
    M, N, K = shape
    g = torch.Generator().manual_seed(M + N)
    A = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    B1 = torch.randn(K, N, generator=g).bfloat16().to(DEV)
    B2 = torch.randn(K, N, generator=g).bfloat16().to(DEV)
    c1, c2 = gemm_bf16_pair(A, B1, B2, tile=tile)
    assert torch.equal(c1, ra.gemm_bf16(A, B1, tile=tile)) and torch.equal(c2, ra.gemm_bf16(A, B2, tile=tile))
    rel_ok(c1, A.float() @ B1.float(), "pair c1")
    rel_ok(c2, A.float() @ B2.float(), "pair c2")
