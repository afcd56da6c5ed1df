"""Chunk starts read from device memory (ra_mask.chunk_starts): what lax.axis_index becomes under jit
(ringattention_jax.py:31-37, :69-75).  A ring step whose starts sit in an int32 device tensor must give the bits of
the same step with the starts passed as host ints, on every kernel family, and one captured HIP graph must serve
every (device, scan step) of a ring by rewriting the two ints."""
import pytest
import torch

from ringattention_amd import ringattention_hip as R
from tests.util import kwargs, make_qkv, packed_segment_ids

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _ring_steps(n, q_len, kv_len, qc, kc):
    """(device, scan step, K/V shard, q_chunk_idx_start, k_chunk_idx_start) of a whole ring (:29-51)."""
    for idx in range(n):
        for dev in range(n):
            shard = (dev - idx) % n
            yield dev, idx, shard, dev * (q_len // qc), shard * (kv_len // kc)


def _run_ring(q, k, v, do, bias, seg, n, kw, device_starts):
    """Forward and backward of every virtual device through the one-step entry points, every step launched (also
    those in which no tile runs: with the starts on the device the host cannot know).  Returns the carries and
    gradient accumulators."""
    cfg = R._Config(kw)
    B, S, H, D = q.shape
    q_len = kv_len = S // n
    mi = R._MaskInputs(cfg, bias, seg, None, B, q.device, S)
    num = torch.empty((B, S, H, D), dtype=torch.float32, device=DEV)
    den = torch.empty((B, H, S), dtype=torch.float32, device=DEV)
    mx = torch.empty((B, H, S), dtype=torch.float32, device=DEV)
    R._carry_init(num, den, mx)
    out = torch.empty_like(q)
    starts = torch.zeros(2, dtype=torch.int32, device=DEV)

    def pass_starts(qs, ks):
        if not device_starts:
            return qs, ks
        starts.copy_(torch.tensor([qs, ks], dtype=torch.int32))
        return starts, None

    for dev, idx, shard, qs, ks in _ring_steps(n, q_len, kv_len, cfg.qc, cfg.kc):
        rq, rk = slice(dev * q_len, (dev + 1) * q_len), slice(shard * kv_len, (shard + 1) * kv_len)
        a, b = pass_starts(qs, ks)
        R._blockwise_attention_fwd(q[:, rq], k[:, rk], v[:, rk], (num[:, rq], den[:, :, rq], mx[:, :, rq]), a, b,
                                   None, None, cfg.cbs, cfg.qc, cfg.kc, _mask_inputs=mi, _cfg=cfg)
    R._finalize(num, den, out)
    dq = torch.zeros((B, S, H, D), dtype=torch.float32, device=DEV)
    dk, dv = torch.zeros_like(dq), torch.zeros_like(dq)
    delta = R._bwd_delta(do, out)
    for dev, idx, shard, qs, ks in _ring_steps(n, q_len, kv_len, cfg.qc, cfg.kc):
        rq, rk = slice(dev * q_len, (dev + 1) * q_len), slice(shard * kv_len, (shard + 1) * kv_len)
        a, b = pass_starts(qs, ks)
        R._blockwise_attention_bwd(q[:, rq], k[:, rk], v[:, rk], do[:, rq],
                                   (dq[:, rq], dk[:, rk], dv[:, rk], out[:, rq], den[:, :, rq], mx[:, :, rq]), a, b,
                                   None, None, cfg.cbs, cfg.qc, cfg.kc, _mask_inputs=mi, _cfg=cfg,
                                   _delta=delta[:, :, rq])
    torch.cuda.synchronize()
    return num, den, mx, out, dq, dk, dv


FAMILIES = [
    # dtype, D, chunk, impl, S per device
    (torch.bfloat16, 128, 128, "mfma", 256),
    (torch.bfloat16, 64, 128, "mfma", 128),
    (torch.float32, 64, 128, "mfma", 128),
    (torch.float32, 32, 32, "generic", 64),
]


@pytest.mark.parametrize("n", [2, 4, 8])
@pytest.mark.parametrize("dtype,D,chunk,impl,s_dev", FAMILIES)
@pytest.mark.parametrize("masks", ["causal", "segments+bias"])
def test_device_chunk_starts_give_the_bits_of_host_ints(n, dtype, D, chunk, impl, s_dev, masks):
    B, H, S = 1, 2, n * s_dev
    print("case", dict(n=n, dtype=str(dtype), D=D, chunk=chunk, impl=impl, S=S, masks=masks), flush=True)
    q, k, v, do = (t.to(DEV) for t in make_qkv(B, S, H, D, dtype=dtype, seed=n, scale=D ** -0.25))
    bias = seg = None
    if masks != "causal":
        bias = torch.randn(B, 1, 1, S, generator=torch.Generator().manual_seed(5)).to(DEV)
        seg = packed_segment_ids(B, S, S // 3, seed=2).to(DEV)
    kw = kwargs(chunk, chunk, 1, dtype=torch.float32, impl=impl)
    host = _run_ring(q, k, v, do, bias, seg, n, kw, device_starts=False)
    dev = _run_ring(q, k, v, do, bias, seg, n, kw, device_starts=True)
    for name, a, b in zip(("num", "den", "max", "out", "dq", "dk", "dv"), host, dev):
        assert torch.equal(a.view(torch.int32) if a.dtype == torch.float32 else a.view(torch.int16),
                           b.view(torch.int32) if b.dtype == torch.float32 else b.view(torch.int16)), name
    assert not torch.isnan(host[3]).any()


def test_one_graph_serves_every_step_of_a_ring():
    """The forward and the backward step are captured once with the starts in device memory; each (device, scan
    step) of a ring of four is then a copy of its shards into the captured buffers, two ints, and a replay.  Every
    replay is checked against the eager call with host ints."""
    n, B, H, D, s_dev, chunk = 4, 1, 2, 128, 256, 128
    S = n * s_dev
    q, k, v, do = (t.to(DEV) for t in make_qkv(B, S, H, D, dtype=torch.bfloat16, seed=3, scale=D ** -0.25))
    seg = packed_segment_ids(B, S, S // 3, seed=4).to(DEV)
    kw = kwargs(chunk, chunk, 1, dtype=torch.float32, impl="mfma")
    cfg = R._Config(kw)
    mi = R._MaskInputs(cfg, None, seg, None, B, q.device, S)
    shape = (B, s_dev, H, D)
    sq, sk, sv, sg = (torch.empty(shape, dtype=torch.bfloat16, device=DEV) for _ in range(4))
    num, dq, dk, dv = (torch.empty(shape, dtype=torch.float32, device=DEV) for _ in range(4))
    den, mx, delta = (torch.empty((B, H, s_dev), dtype=torch.float32, device=DEV) for _ in range(3))
    starts = torch.zeros(2, dtype=torch.int32, device=DEV)

    def step(a, b):
        R._blockwise_attention_fwd(sq, sk, sv, (num, den, mx), a, b, None, None, cfg.cbs, cfg.qc, cfg.kc,
                                   _mask_inputs=mi, _cfg=cfg)
        R._blockwise_attention_bwd(sq, sk, sv, sg, (dq, dk, dv, None, den, mx), a, b, None, None, cfg.cbs, cfg.qc,
                                   cfg.kc, _mask_inputs=mi, _cfg=cfg, _delta=delta)

    def load(dev, shard):
        sq.copy_(q[:, dev * s_dev:(dev + 1) * s_dev]); sg.copy_(do[:, dev * s_dev:(dev + 1) * s_dev])
        sk.copy_(k[:, shard * s_dev:(shard + 1) * s_dev]); sv.copy_(v[:, shard * s_dev:(shard + 1) * s_dev])
        R._carry_init(num, den, mx)
        for t in (dq, dk, dv):
            t.zero_()
        delta.fill_(0.25)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):           # warm-up outside the capture, on the capturing stream
        load(0, 0)
        step(starts, None)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step(starts, None)
    for dev, idx, shard, qs, ks in _ring_steps(n, s_dev, s_dev, cfg.qc, cfg.kc):
        load(dev, shard)
        step(qs, ks)                         # eager, host ints
        torch.cuda.synchronize()
        want = [t.clone() for t in (num, den, mx, dq, dk, dv)]
        load(dev, shard)
        starts.copy_(torch.tensor([qs, ks], dtype=torch.int32))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("num", "den", "max", "dq", "dk", "dv"), want, (num, den, mx, dq, dk, dv)):
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), (name, dev, idx)
