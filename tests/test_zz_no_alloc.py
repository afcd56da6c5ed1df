"""ra_decode_fwd_static, the decode entry point that allocates nothing (its split-KV partials live in a device array
inside the library), against ra_decode_fwd with a caller's workspace: both called through the C-ABI on the same
inputs.  Same kernels and the same number of key splits give the same bits; where the built-in buffer forces fewer
splits the bar is the bf16 parity tolerance (max-abs 2e-2, relative L2 1e-2)."""
import ctypes

import pytest
import torch

from ringattention_amd import _lib as L
from tests.util import errors

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _params(q, k, v, out, cache_idx, kc, num_splits):
    B, _, H, D = q.shape
    p = L.RaDecodeParams()
    p.q, p.k, p.v, p.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    p.dtype = L.RA_BF16 if q.dtype == torch.bfloat16 else L.RA_F32
    p.B, p.L, p.H, p.D = B, k.shape[1], H, D
    p.q_stride_b, p.out_stride_b = q.stride(0), out.stride(0)
    p.kv_stride_b, p.kv_stride_s = k.stride(0), k.stride(1)
    m = p.mask
    m.causal_block_size, m.query_chunk_size, m.key_chunk_size = 1, 1, kc
    m.q_chunk_idx_start, m.k_chunk_idx_start = cache_idx, 0
    m.mask_min = float(torch.finfo(torch.float32).min)
    p.num_splits = num_splits
    return p


def _both(B, Lc, H, D, kc, cache_idx, num_splits, seed, dtype=torch.bfloat16):
    print("no-alloc decode case", dict(B=B, L=Lc, H=H, D=D, cache_idx=cache_idx, num_splits=num_splits), flush=True)
    g = torch.Generator(device=DEV).manual_seed(seed)
    q = torch.randn(B, 1, H, D, device=DEV, generator=g).to(dtype)
    k = torch.randn(B, Lc, H, D, device=DEV, generator=g).to(dtype)
    v = torch.randn(B, Lc, H, D, device=DEV, generator=g).to(dtype)
    lib = L.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out_ws = torch.empty_like(q)
    ws = torch.empty(lib.ra_decode_workspace_bytes(B, Lc, H, D, num_splits), dtype=torch.uint8, device=DEV)
    p = _params(q, k, v, out_ws, cache_idx, kc, num_splits)
    p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    L.check(lib.ra_decode_fwd(ctypes.byref(p), stream), "ra_decode_fwd")
    out_st = torch.full_like(q, float("nan"))
    p2 = _params(q, k, v, out_st, cache_idx, kc, num_splits)          # workspace left null: it is ignored
    before = torch.cuda.memory_allocated()
    L.check(lib.ra_decode_fwd_static(ctypes.byref(p2), stream), "ra_decode_fwd_static")
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    return out_ws, out_st


def test_static_scratch_entry_equals_workspace_entry_twice_in_a_row():
    # first call: 16 key splits of 4 x 32 heads; second call, right after it, on a smaller input, so that the buffer
    # still holds the first call's partials beyond what the second one writes
    a_ws, a_st = _both(4, 4096, 32, 128, 128, 4000, 0, seed=21)
    assert not torch.isnan(a_st).any()
    assert torch.equal(a_ws, a_st)
    b_ws, b_st = _both(1, 1024, 8, 128, 128, 777, 0, seed=22)
    assert not torch.isnan(b_st).any()
    assert torch.equal(b_ws, b_st)
    # the first shape again: what the smaller call left behind does not leak into it
    c_ws, c_st = _both(4, 4096, 32, 128, 128, 4000, 0, seed=21)
    assert torch.equal(c_st, a_st) and torch.equal(c_ws, c_st)
    # an explicit split count, fp32 inputs, head size 64
    d_ws, d_st = _both(2, 2048, 4, 64, 64, 2047, 5, seed=23, dtype=torch.float32)
    assert torch.equal(d_ws, d_st)


def test_static_scratch_entry_lowers_the_split_count_to_fit():
    # 128 x 64 heads x (64 + 2) floats = 2.2 MB per split: the automatic choice of 8 splits needs 17 MB, the buffer
    # takes 7.  Fewer splits add the same terms in another order: parity tolerance, not bits.
    ws, st = _both(128, 2048, 64, 64, 64, 2000, 0, seed=24)
    assert not torch.isnan(st).any()
    ma, rl = errors(st, ws)
    assert ma <= 2e-2 and rl <= 1e-2, (ma, rl)


def test_static_scratch_entry_rejects_what_cannot_fit():
    lib = L.load()
    q = torch.zeros(1024, 1, 64, 128, dtype=torch.bfloat16, device=DEV)
    kv = torch.zeros(1024, 64, 64, 128, dtype=torch.bfloat16, device=DEV)
    p = _params(q, kv, kv, torch.empty_like(q), 10, 64, 0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.ra_decode_fwd_static(ctypes.byref(p), stream) == L.RA_ERR_UNSUPPORTED
    assert b"scratch" in lib.ra_last_error()


def test_static_scratch_decode_replays_from_a_graph():
    """decode_attention(static_scratch=True) after one eager warm-up call (which looks the buffer's address up),
    captured into a graph and replayed for several positions - the position sits in device memory - with eager
    work between the replays; every replay must give the bits of the workspace path."""
    import ringattention_amd as ra
    from tests.util import kwargs
    B, Lc, H, D, kc = 2, 4096, 8, 128, 128
    g = torch.Generator(device=DEV).manual_seed(31)
    q = torch.randn(B, 1, H, D, device=DEV, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Lc, H, D, device=DEV, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Lc, H, D, device=DEV, generator=g).to(torch.bfloat16)
    kw = kwargs(1, kc, 1)
    pos = torch.tensor(100, dtype=torch.int32, device=DEV)
    out = torch.empty_like(q)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ra.decode_attention(q, k, v, None, None, pos, kw, out=out, static_scratch=True)       # warm-up
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ra.decode_attention(q, k, v, None, None, pos, kw, out=out, static_scratch=True)
    for p in (100, 4095, 777, 128, 2048):
        pos.fill_(p)
        want = ra.decode_attention(q, k, v, None, None, p, kw)        # eager, workspace path, between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(want, out), p
