"""blockwise_feedforward (ringattention_jax.py:333-352) and the SwiGLU MLP it is used with,
over the bf16 MFMA GEMM kernels of libringattn_hip.so."""
import ctypes

import torch

from . import _lib as L
from .ringattention_hip import _stream


def _ptr(t):
    return t.data_ptr() if t is not None else None


class _SwiGLUFn(torch.autograd.Function):
    """y = (silu(x w1) * (x w3)) w2 on one chunk of tokens.  Nothing but x is kept for the backward
    pass (the reference's default policy is nothing_saveable, ringattention_jax.py:334): the
    pre-activations are recomputed.  ``gemm_tile`` is ra_swiglu_params.gemm_tile."""

    @staticmethod
    def forward(ctx, x, w1, w2, w3, gemm_tile=0):
        T, d = x.shape
        f = w1.shape[1]
        dev = x.device
        ctx.gemm_tile = gemm_tile
        a = torch.empty((T, f), dtype=torch.bfloat16, device=dev)
        b = torch.empty_like(a)
        h = torch.empty_like(a)
        y = torch.empty((T, d), dtype=torch.bfloat16, device=dev)
        p = L.RaSwigluParams()
        p.T, p.d, p.f = T, d, f
        p.x, p.w1, p.w2, p.w3 = x.data_ptr(), w1.data_ptr(), w2.data_ptr(), w3.data_ptr()
        p.a, p.b, p.h, p.y = a.data_ptr(), b.data_ptr(), h.data_ptr(), y.data_ptr()
        p.gemm_tile = gemm_tile
        L.check(L.load().ra_swiglu_fwd(ctypes.byref(p), _stream()), "ra_swiglu_fwd")
        ctx.save_for_backward(x, w1, w2, w3)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w1, w2, w3 = ctx.saved_tensors
        T, d = x.shape
        f = w1.shape[1]
        dev = x.device
        dy = dy.to(torch.bfloat16).contiguous()
        bf = dict(dtype=torch.bfloat16, device=dev)
        a, b, h, da, db = (torch.empty((T, f), **bf) for _ in range(5))
        dx = torch.empty((T, d), **bf)
        dw1 = torch.zeros((d, f), dtype=torch.float32, device=dev)
        dw3 = torch.zeros((d, f), dtype=torch.float32, device=dev)
        dw2 = torch.zeros((f, d), dtype=torch.float32, device=dev)
        p = L.RaSwigluParams()
        p.T, p.d, p.f = T, d, f
        p.x, p.w1, p.w2, p.w3 = x.data_ptr(), w1.data_ptr(), w2.data_ptr(), w3.data_ptr()
        p.a, p.b, p.h, p.y = a.data_ptr(), b.data_ptr(), h.data_ptr(), None
        p.dy, p.dx = dy.data_ptr(), dx.data_ptr()
        p.dw1, p.dw2, p.dw3 = dw1.data_ptr(), dw2.data_ptr(), dw3.data_ptr()
        p.da, p.db = da.data_ptr(), db.data_ptr()
        p.gemm_tile = ctx.gemm_tile
        L.check(L.load().ra_swiglu_bwd(ctypes.byref(p), _stream()), "ra_swiglu_bwd")
        return dx, dw1.to(w1.dtype), dw2.to(w2.dtype), dw3.to(w3.dtype), None


class _BlockwiseSwiGLUFn(torch.autograd.Function):
    """The whole scan of blockwise_feedforward over a SwiGLU MLP as one autograd node: chunk after chunk
    through the same scratch buffers; in the backward pass the weight gradients of all chunks
    accumulate in fp32 inside the GEMM epilogue and are rounded to the weights' dtype once.
    With ``save_preact`` the pre-activations x w1, x w3 of every chunk stay in memory for the backward pass
    (2 * tokens * intermediate bf16 values); otherwise they are recomputed, the reference's default policy
    (nothing_saveable, ringattention_jax.py:334).  The results are the same bits either way."""

    @staticmethod
    def forward(ctx, x, w1, w2, w3, chunk_tokens, save_preact, gemm_tile=0, dw_group=1):
        T, d = x.shape
        ctx.gemm_tile = gemm_tile
        ctx.dw_group = max(1, int(dw_group))
        f = w1.shape[1]
        bf = dict(dtype=torch.bfloat16, device=x.device)
        save_preact = bool(save_preact) and any(ctx.needs_input_grad[:4])
        rows = T if save_preact else chunk_tokens
        a, b = (torch.empty((rows, f), **bf) for _ in range(2))
        h = torch.empty((chunk_tokens, f), **bf)
        y = torch.empty((T, d), **bf)
        lib, stream = L.load(), _stream()
        p = L.RaSwigluParams()
        p.T, p.d, p.f = chunk_tokens, d, f
        p.w1, p.w2, p.w3 = w1.data_ptr(), w2.data_ptr(), w3.data_ptr()
        p.a, p.b, p.h = a.data_ptr(), b.data_ptr(), h.data_ptr()
        p.gemm_tile = gemm_tile
        for t0 in range(0, T, chunk_tokens):
            p.x, p.y = x[t0:].data_ptr(), y[t0:].data_ptr()
            if save_preact:
                p.a, p.b = a[t0:].data_ptr(), b[t0:].data_ptr()
            L.check(lib.ra_swiglu_fwd(ctypes.byref(p), stream), "ra_swiglu_fwd")
        ctx.save_for_backward(x, w1, w2, w3)
        ctx.chunk_tokens = chunk_tokens
        ctx.preact = (a, b) if save_preact else None
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w1, w2, w3 = ctx.saved_tensors
        ct = ctx.chunk_tokens
        T, d = x.shape
        f = w1.shape[1]
        dev = x.device
        dy = dy.to(torch.bfloat16).contiguous()
        bf = dict(dtype=torch.bfloat16, device=dev)
        saved = ctx.preact is not None
        a, b = ctx.preact if saved else (torch.empty((ct, f), **bf) for _ in range(2))
        ctx.preact = None
        # h, da, db of `group` consecutive launches side by side: their weight-gradient products then go out as one
        # launch each (K = group * ct), which reads and writes the fp32 accumulators once per group
        group = min(ctx.dw_group, T // ct)
        h, da, db = (torch.empty((group * ct, f), **bf) for _ in range(3))
        dx = torch.empty((T, d), **bf)
        dw1 = torch.zeros((d, f), dtype=torch.float32, device=dev)
        dw3 = torch.zeros((d, f), dtype=torch.float32, device=dev)
        dw2 = torch.zeros((f, d), dtype=torch.float32, device=dev)
        lib, stream = L.load(), _stream()
        p = L.RaSwigluParams()
        p.T, p.d, p.f = ct, d, f
        p.w1, p.w2, p.w3 = w1.data_ptr(), w2.data_ptr(), w3.data_ptr()
        p.a, p.b, p.h, p.y = a.data_ptr(), b.data_ptr(), h.data_ptr(), None
        p.dw1, p.dw2, p.dw3 = dw1.data_ptr(), dw2.data_ptr(), dw3.data_ptr()
        p.da, p.db = da.data_ptr(), db.data_ptr()
        p.preact_saved = 1 if saved else 0
        p.gemm_tile = ctx.gemm_tile
        p.defer_weight_grads = 1 if group > 1 else 0
        n_launch = T // ct
        for i in range(n_launch):
            t0, slot = i * ct, i % group
            p.T = ct
            p.x, p.dy, p.dx = x[t0:].data_ptr(), dy[t0:].data_ptr(), dx[t0:].data_ptr()
            p.h, p.da, p.db = h[slot * ct:].data_ptr(), da[slot * ct:].data_ptr(), db[slot * ct:].data_ptr()
            if saved:
                p.a, p.b = a[t0:].data_ptr(), b[t0:].data_ptr()
            L.check(lib.ra_swiglu_bwd(ctypes.byref(p), stream), "ra_swiglu_bwd")
            if group > 1 and (slot == group - 1 or i == n_launch - 1):
                first = t0 - slot * ct                 # the tokens of the launches whose h, da, db fill the slots
                p.T = (slot + 1) * ct
                p.x, p.dy = x[first:].data_ptr(), dy[first:].data_ptr()
                p.h, p.da, p.db = h.data_ptr(), da.data_ptr(), db.data_ptr()
                L.check(lib.ra_swiglu_weight_grads(ctypes.byref(p), stream), "ra_swiglu_weight_grads")
        return dx, dw1.to(w1.dtype), dw2.to(w2.dtype), dw3.to(w3.dtype), None, None, None, None


def _save_preactivations(policy):
    """What ``policy`` (ringattention_jax.py:334) means here.  "nothing_saveable" - the reference's default, by
    name or as an object of that name, and also what None means - recomputes x w1 and x w3 in the backward pass,
    so that nothing but the input of the scan outlives a chunk.  "save_preactivations" (or
    "everything_saveable") is the explicit opt-in that keeps them: 4 * tokens * intermediate bytes (2.9 GB at
    65536 x 11008) for two GEMMs less per chunk in the backward pass.  The same bits come out either way."""
    if policy is None:
        return False
    name = policy if isinstance(policy, str) else getattr(policy, "__name__", "")
    if name == "nothing_saveable":
        return False
    if name in ("save_preactivations", "everything_saveable"):
        return True
    raise ValueError("policy must be None, 'nothing_saveable' or 'save_preactivations'")


def _slab_tokens(chunk_size, n_chunks, launch_tokens=None):
    """Tokens per launch.  By default one chunk, so the scratch of a step (five (chunk_size, intermediate) bf16
    buffers) is what chunk_size implies, as in the reference's scan.  Tokens are independent in a token-wise MLP,
    so a caller with memory to spare may let consecutive chunks share a launch (``launch_tokens``): the result is
    the same, the GEMMs fill the 256 CUs in whole rounds, and the fp32 weight-gradient accumulators are read and
    written once per launch instead of once per chunk.  The largest whole number of chunks within
    ``launch_tokens`` that divides the scan is taken (16384 tokens x 11008 are 1.8 GB of scratch)."""
    if launch_tokens is None:
        return chunk_size
    g = max(1, min(n_chunks, int(launch_tokens) // chunk_size))
    while n_chunks % g:
        g -= 1
    return chunk_size * g


_TOKEN_GRID = 128       # tokens per launch are a multiple of this (rows of a GEMM tile)


def _check_swiglu_weights(ff, x):
    """The kernels read the three weights as dense bf16 (in, out) arrays on x's device: anything else (a module moved
    to fp32, a transposed view) would be read as garbage, so it is refused."""
    d, f = ff.w1.shape
    for name, w, shape in (("w1", ff.w1, (d, f)), ("w3", ff.w3, (d, f)), ("w2", ff.w2, (f, d))):
        if w.dtype != torch.bfloat16:
            raise NotImplementedError("SwiGLU kernels are bf16: %s is %s" % (name, w.dtype))
        if tuple(w.shape) != shape or not w.is_contiguous() or w.device != x.device:
            raise ValueError("SwiGLU weight %s must be a contiguous %s array on %s" % (name, shape, x.device))
    if x.shape[-1] != d:
        raise ValueError("hidden size %d of the input does not match the weights' %d" % (x.shape[-1], d))


class SwiGLU(torch.nn.Module):
    """The LLaMA-style MLP the reference's README pairs with blockwise_feedforward:
    w2(silu(x w1) * (x w3)); weights stored (in, out), bf16."""

    def __init__(self, hidden, intermediate, device=None, init_std=0.02, gemm_tile=None):
        super().__init__()
        # None: the library picks the GEMM tile kernel; 0 - 3 force one (ra_swiglu_params.gemm_tile), for tests
        self.gemm_tile = 0 if gemm_tile is None else int(gemm_tile) + 1
        mk = lambda i, o: torch.nn.Parameter(
            (torch.randn(i, o, device=device, dtype=torch.float32) * init_std).to(torch.bfloat16))
        self.w1 = mk(hidden, intermediate)
        self.w3 = mk(hidden, intermediate)
        self.w2 = mk(intermediate, hidden)

    def forward(self, hidden_states):
        shp = hidden_states.shape
        x = hidden_states.reshape(-1, shp[-1])
        if x.dtype != torch.bfloat16:
            raise NotImplementedError("SwiGLU kernels are bf16")
        if not x.is_cuda:
            raise RuntimeError("ringattention_amd runs on the GPU only")
        _check_swiglu_weights(self, x)
        T = x.shape[0]
        if T == 0:                  # nothing to launch; the zero keeps the empty result attached to its inputs
            zero = 0.0 * (self.w1.sum() + self.w2.sum() + self.w3.sum())
            return x.new_zeros(*shp[:-1], self.w2.shape[1]) + x.sum() + zero.to(x.dtype)
        if T % _TOKEN_GRID:         # the GEMM tiles want whole groups of 128 tokens: zero rows, dropped again below
            x = torch.nn.functional.pad(x, (0, 0, 0, _TOKEN_GRID - T % _TOKEN_GRID))
        y = _SwiGLUFn.apply(x.contiguous(), self.w1, self.w2, self.w3, self.gemm_tile)[:T]
        return y.reshape(*shp[:-1], y.shape[-1])


def blockwise_feedforward(feedforward, inputs, chunk_size, static_argnums=(1,), policy="nothing_saveable",
                          pre_remat=True, launch_tokens=None, weight_grad_chunks=4):
    """ringattention_jax.py:333-352: apply ``feedforward`` to ``chunk_size`` tokens at a time.

    The reference groups tokens with 'b (c n) d -> b c n d', c=chunk_size and scans over n, so step
    j sees the strided token set {ci * n + j}.  A generic callable gets exactly those groups.  A
    ``SwiGLU`` instance is token-wise, so it is fed contiguous slabs of chunk_size tokens instead:
    the same number of steps and the same result, with dense memory access (a chunk size that is not a multiple of
    128 is rounded up to one: fewer, slightly larger steps over the same tokens).  ``policy`` selects what the
    SwiGLU scan keeps for its backward pass: the reference's default ``nothing_saveable`` recomputes the
    pre-activations, ``"save_preactivations"`` is the opt-in that keeps them (see _save_preactivations).
    ``launch_tokens`` (no counterpart in the reference) lets consecutive chunks share a kernel launch and its
    scratch, see _slab_tokens; the default keeps a step's memory at what ``chunk_size`` implies.
    ``weight_grad_chunks`` (no counterpart either): in the backward pass the three weight-gradient products of that
    many consecutive launches go out together (their h, da, db are kept side by side: three more (chunk, intermediate)
    buffers per extra chunk), so the fp32 accumulators of the weights - broadcast over the scan, their gradients summed
    over chunks - are read and written once per group; forward, dx and every value of the result are unaffected but
    for the order of the fp32 sum over tokens.  1 = per launch; the default of 4 keeps the scratch of a backward step
    at 14 (chunk, intermediate) buffers instead of 5, still independent of the sequence length (at 65536 tokens of
    4096 x 11008: 61.2 ms with 1, 57.5 with 2, 55.8 with 4, 55.0 with 8).
    ``pre_remat=False`` (:335-336) rematerialises a generic callable here (torch.utils.checkpoint, per chunk) unless
    ``policy`` keeps the activations; with the default True the caller has done so, or not, as in the reference.
    ``static_argnums`` steers XLA only."""
    b, s, d = inputs.shape
    if s % chunk_size:
        raise ValueError("sequence length %d must divide by chunk_size %d" % (s, chunk_size))
    n = s // chunk_size
    if isinstance(feedforward, SwiGLU) and inputs.numel() == 0:
        return feedforward(inputs)
    if isinstance(feedforward, SwiGLU):
        if inputs.dtype != torch.bfloat16:
            raise NotImplementedError("SwiGLU kernels are bf16")
        if not inputs.is_cuda:
            raise RuntimeError("ringattention_amd runs on the GPU only")
        # contiguous slabs of chunk_size tokens (batch rows one after the other: a token-wise MLP does not see the
        # difference), one autograd node for the whole scan
        _check_swiglu_weights(feedforward, inputs)
        x2 = inputs.reshape(b * s, d)
        step, steps = chunk_size, b * n
        if chunk_size % _TOKEN_GRID:
            # a chunk size the GEMM tiles do not divide: the same tokens in steps of the next multiple of 128, the
            # last one filled up with zero rows that are dropped again (tokens are independent, zero rows add
            # nothing to the weight gradients)
            step = -(-chunk_size // _TOKEN_GRID) * _TOKEN_GRID
            steps = -(-b * s // step)
            x2 = torch.nn.functional.pad(x2, (0, 0, 0, steps * step - b * s))
        slab = _slab_tokens(step, steps, launch_tokens)
        y = _BlockwiseSwiGLUFn.apply(x2.contiguous(), feedforward.w1, feedforward.w2,
                                     feedforward.w3, slab, _save_preactivations(policy), feedforward.gemm_tile,
                                     max(1, int(weight_grad_chunks) * step // slab))
        return y[:b * s].reshape(b, s, y.shape[-1])
    fn = feedforward
    if not pre_remat and torch.is_grad_enabled():
        # :335-336: the callable has not been rematerialised by the caller, so it is here - every chunk's forward
        # pass runs again in the backward pass instead of keeping its activations - unless the policy keeps them
        try:
            keep = _save_preactivations(policy)
        except ValueError:
            keep = False            # another checkpoint policy of the reference's framework: recompute (same results)
        if not keep:
            from torch.utils.checkpoint import checkpoint
            fn = lambda h: checkpoint(feedforward, h, use_reentrant=False)
    x = inputs.reshape(b, chunk_size, n, d)
    outs = [fn(x[:, :, j, :]) for j in range(n)]
    out = torch.stack(outs, dim=2)
    return out.reshape(b, s, out.shape[-1])


def gemm_bf16(A, B, trans_a=False, trans_b=False, out_dtype=torch.bfloat16, out=None, accumulate=False, tile=None):
    """C = op(A) op(B) with the library's bf16 MFMA GEMM (used by the SwiGLU kernels; exposed for tests).
    ``tile`` 0 - 3 names the tile kernel (ra_gemm_bf16_tile); None lets the library choose."""
    M = A.shape[1] if trans_a else A.shape[0]
    K = A.shape[0] if trans_a else A.shape[1]
    N = B.shape[0] if trans_b else B.shape[1]
    if out is None:
        out = torch.zeros((M, N), dtype=out_dtype, device=A.device)
    cd = L.RA_F32 if out.dtype == torch.float32 else L.RA_BF16
    if tile is None:
        L.check(L.load().ra_gemm_bf16(A.data_ptr(), B.data_ptr(), out.data_ptr(), M, N, K, int(trans_a),
                                      int(trans_b), cd, int(accumulate), _stream()), "ra_gemm_bf16")
    else:
        L.check(L.load().ra_gemm_bf16_tile(A.data_ptr(), B.data_ptr(), out.data_ptr(), M, N, K, int(trans_a),
                                           int(trans_b), cd, int(accumulate), int(tile), _stream()),
                "ra_gemm_bf16_tile")
    return out


def gemm_bf16_pair(A, B1, B2, out1=None, out2=None, tile=None):
    """C1 = A B1 and C2 = A B2 in one launch (ra_gemm_bf16_pair: how the SwiGLU kernels compute x w1 and x w3;
    exposed for tests and the benchmark)."""
    M, K = A.shape
    N = B1.shape[1]
    if out1 is None:
        out1 = torch.empty((M, N), dtype=torch.bfloat16, device=A.device)
    if out2 is None:
        out2 = torch.empty((M, N), dtype=torch.bfloat16, device=A.device)
    L.check(L.load().ra_gemm_bf16_pair(A.data_ptr(), B1.data_ptr(), B2.data_ptr(), out1.data_ptr(), out2.data_ptr(),
                                       M, N, K, -1 if tile is None else int(tile), _stream()), "ra_gemm_bf16_pair")
    return out1, out2
