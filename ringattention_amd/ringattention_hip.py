"""Host side of the MI355X ring-attention hot path: the interface of the reference's
``ringattention/ringattention_jax.py`` over the HIP kernels of libringattn_hip.so.

Same names, argument order and meaning as the reference:

* ``ring_attention(q, k, v, attn_bias, segment_ids, cache_idx, axis_name, float32_logits,
  blockwise_kwargs)``  (ringattention_jax.py:92-97), differentiable in q, k, v;
* ``_blockwise_attention_fwd`` / ``_blockwise_attention_bwd`` (:99-179, :181-270): one ring
  step on one device, carry in / carry out;
* ``below_or_on_diag`` (:324-331).

Tensors are torch tensors in device memory (torch only owns memory and streams).  The ring over
``axis_name`` is virtual: ``ring_axis(name, size)`` declares its size, q/k/v are then the global
arrays a ``shard_map`` caller holds, and every device's program is run in turn on the one GPU
with the K/V shard that the ring would have delivered at each step.  No bytes move.
"""
import collections
import contextlib
import ctypes
import math
import warnings
import weakref

import torch

from . import _lib as L

# --------------------------------------------------------------------------- virtual ring axes
_AXES = {}


@contextlib.contextmanager
def ring_axis(axis_name, size):
    """Declare that ``axis_name`` is a ring of ``size`` virtual devices (the sp mesh axis)."""
    if size < 1:
        raise ValueError("ring size must be >= 1")
    old = _AXES.get(axis_name)
    _AXES[axis_name] = int(size)
    try:
        yield
    finally:
        if old is None:
            _AXES.pop(axis_name, None)
        else:
            _AXES[axis_name] = old


def axis_size(axis_name):
    """Counterpart of lax.psum(1, axis_name) (ringattention_jax.py:24): 1 for an undeclared axis."""
    if axis_name is None:
        return 1
    if isinstance(axis_name, int):
        return axis_name
    return _AXES.get(axis_name, 1)


# --------------------------------------------------------------------------- helpers
_DTYPES = {
    "float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16,
    "torch.float32": torch.float32, "torch.bfloat16": torch.bfloat16, "torch.float16": torch.float16,
    "<class 'jax.numpy.float32'>": torch.float32, "<class 'jax.numpy.bfloat16'>": torch.bfloat16,
}


def _as_torch_dtype(dt):
    if isinstance(dt, torch.dtype):
        return dt
    name = getattr(dt, "__name__", None) or getattr(dt, "name", None) or str(dt)
    if name in _DTYPES:
        return _DTYPES[name]
    raise ValueError("blockwise_kwargs['dtype']=%r is not float32/bfloat16/float16" % (dt,))


def _ra_dtype(t):
    if t.dtype == torch.float32:
        return L.RA_F32
    if t.dtype == torch.bfloat16:
        return L.RA_BF16
    raise NotImplementedError("q/k/v dtype %s: only float32 and bfloat16 are supported" % t.dtype)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def below_or_on_diag(r, r_blk_size, c, c_blk_size, causal_block_size):
    """ringattention_jax.py:324-331 on Python ints."""
    cq = max(causal_block_size, r_blk_size)
    ck = max(causal_block_size, c_blk_size)
    r = r // (cq // r_blk_size)
    c = c // (ck // c_blk_size)
    return ((r + 1) * cq - 1) > (c * ck)


def run_prefix_keys(q_chunk_global, qc, kc, cbs, k_chunk_idx_start, kv_len):
    """How many leading keys of a K/V shard lie in chunks that run against one query chunk.

    The skip predicate is monotone in the key chunk index, so the chunks that run are a prefix;
    the kernels use the same closed form."""
    if cbs is None or cbs <= 0:
        return kv_len
    cq, ck = max(cbs, qc), max(cbs, kc)
    r = q_chunk_global // (cq // qc)
    x = (r + 1) * cq - 1
    if x <= 0:
        return 0
    cmax = (x - 1) // ck
    climit = (cmax + 1) * (ck // kc)
    nloc = climit - k_chunk_idx_start
    if nloc <= 0:
        return 0
    return min(nloc * kc, kv_len)


_SEG_CACHE = collections.OrderedDict()    # per segment_ids tensor: [weakref, int32 ids, tile ranges, host copy]


class _Config:
    """blockwise_kwargs (ringattention_jax.py:99-100) reduced to what the kernels need."""

    def __init__(self, blockwise_kwargs):
        kw = dict(blockwise_kwargs)
        self.qc = int(kw["query_chunk_size"])
        self.kc = int(kw["key_chunk_size"])
        cbs = kw.get("causal_block_size", None)
        self.cbs = None if cbs is None else int(cbs)
        if self.cbs is not None and self.cbs < 1:
            raise ValueError("causal_block_size must be None or >= 1")
        # attention dropout (:119-123): ``dropout_rng`` is an integer seed of the Philox stream ra_dropout_keep
        # documents, not a jax.random key; the mask is a pure function of (seed, attn_pdrop, local shape)
        self.pdrop = 0.0
        self.seed = 0
        if (not kw.get("deterministic", True)) and float(kw.get("attn_pdrop", 0.0)) > 0.0:
            self.pdrop = float(kw["attn_pdrop"])
            if not self.pdrop < 1.0:
                raise ValueError("attn_pdrop must lie in [0, 1)")
            rng = kw.get("dropout_rng", None)
            if rng is None:
                raise ValueError("attention dropout needs blockwise_kwargs['dropout_rng'] (an integer seed)")
            self.seed = int(rng) & 0xFFFFFFFFFFFFFFFF
        self.dtype = _as_torch_dtype(kw.get("dtype", torch.float32))
        self.mask_min = float(torch.finfo(self.dtype).min)
        self.impl = {"auto": L.RA_IMPL_AUTO, "generic": L.RA_IMPL_GENERIC, "mfma": L.RA_IMPL_MFMA,
                     "mfma_any": L.RA_IMPL_MFMA_ANY}[kw.get("impl", "auto")]
        # measurement hook: launch one of the two backward kernels alone (ra_attn_bwd_block_part)
        self.bwd_only = {None: 0, "dq": L.RA_BWD_PART_DQ, "dkv": L.RA_BWD_PART_DKV}[kw.get("bwd_only", None)]
        self.skip_masked_tiles = kw.get("skip_masked_tiles", None)
        # "step": a scan step of all virtual devices goes out as one launch per kernel when the kernels allow;
        # "device": one launch per device and step
        # False: never reuse the int32 copy / tile ranges of a segment_ids tensor seen before (for callers that edit
        # the ids through a numpy alias or .data, which the tensor's version counter does not see)
        self.cache_segment_ids = bool(kw.get("cache_segment_ids", True))
        # False: the kernels scan the per-tile id ranges for their tile hulls instead of reading the per-run table
        # (the two give the same results; for tests)
        self.segment_hull_table = bool(kw.get("segment_hull_table", True))
        self.logit_dim = 0            # set when q, k, v were zero-padded along D: the head size that scales the logits
        self.ring_launch = kw.get("ring_launch", "step")
        if self.ring_launch not in ("step", "device"):
            raise ValueError("ring_launch must be 'step' or 'device'")
        # what the backward pass multiplies with the cotangent (:218): "fp32", the un-rounded output the reference
        # keeps as a residual (:53; 4 bytes per element next to the returned output), or "rounded", the returned
        # output itself (no extra memory; differs from the reference by the rounding of the output)
        self.output_residual = kw.get("output_residual", "fp32")
        if self.output_residual not in ("fp32", "rounded"):
            raise ValueError("output_residual must be 'fp32' or 'rounded'")
        # policy / precision / prevent_cse only steer XLA rematerialisation: the kernels always recompute
        # the probabilities in the backward pass.


class _MaskInputs:
    """attn_bias / segment_ids / cache_idx in the form ra_mask wants (device memory kept alive here)."""

    def __init__(self, cfg, attn_bias, segment_ids, cache_idx, batch, device, k_total, heads=None):
        self.bias = None
        self.bias_strides = (0, 0, 0, 0)
        if attn_bias is not None:
            if attn_bias.dim() != 4:
                raise ValueError("attn_bias must be 4-D (B, H, Q, K)")
            bb, hb, qb, kb = attn_bias.shape
            # the kernels index the bias by batch row and head: a size that is neither 1 (broadcast) nor the array's
            # own would read past its end
            if bb not in (1, batch) or (heads is not None and hb not in (1, heads)):
                raise ValueError("attn_bias batch / head dims %s must be 1 or those of q (%d, %s)"
                                 % ((bb, hb), batch, heads))
            if qb != 1 and qb < cfg.qc:
                raise ValueError("attn_bias query dim must be 1 or >= query_chunk_size")
            if kb != 1 and kb < k_total:
                raise ValueError("attn_bias key dim %d is smaller than the global key length %d" % (kb, k_total))
            # chunk_bias.astype(dtype) (ringattention_jax.py:322): values rounded to the kwargs dtype
            b = attn_bias.detach().to(device=device).to(cfg.dtype).to(torch.float32).contiguous()
            self.bias = b
            self.bias_strides = (0 if bb == 1 else b.stride(0), 0 if hb == 1 else b.stride(1),
                                 0 if qb == 1 else b.stride(2), 0 if kb == 1 else b.stride(3))
        self.seg = None
        self.seg_stride_b = 0
        self.seg_len = 0
        self.seg_mm = None
        self.seg_hull = None
        self.seg_tiles = 0
        if segment_ids is not None:
            if segment_ids.dim() != 2:
                raise ValueError("segment_ids must be 2-D (B, S)")
            if segment_ids.shape[0] not in (1, batch):
                raise ValueError("segment_ids batch dim %d must be 1 or that of q (%d)" % (segment_ids.shape[0], batch))
            # the int32 copy, the per-tile id ranges and their host copy are kept per segment_ids tensor (same
            # storage, same version counter): a later call with the tensor unchanged launches nothing for them and
            # copies nothing to the host, so it can be captured into a HIP graph.  The version counter does not see
            # edits through a numpy alias (torch.from_numpy) or through .data: such callers pass
            # blockwise_kwargs["cache_segment_ids"] = False.  Tensors made under torch.inference_mode() have no
            # version counter and are never cached.  An entry is reused on the stream that produced it, and on any
            # other stream once its host copy exists (that copy waited for the kernels that wrote the entry).
            key = None
            cur_stream = torch.cuda.current_stream(device).cuda_stream if torch.device(device).type == "cuda" else 0
            if cfg.cache_segment_ids:
                try:
                    key = (segment_ids.data_ptr(), segment_ids._version, tuple(segment_ids.shape), segment_ids.dtype,
                           str(segment_ids.device), str(device))
                except RuntimeError:          # inference tensors do not track a version counter
                    key = None
            hit = _SEG_CACHE.get(key) if key is not None else None
            if hit is not None and hit[0]() is segment_ids and (hit[4] == cur_stream or hit[3] is not None):
                _SEG_CACHE.move_to_end(key)
                self._seg_entry = hit
            else:
                self._seg_entry = self._segment_entry(segment_ids, device, cur_stream)
                if key is not None:
                    _SEG_CACHE[key] = self._seg_entry
                    while len(_SEG_CACHE) > 8:
                        _SEG_CACHE.popitem(last=False)
            s = self._seg_entry[1]
            self.seg = s
            self.seg_stride_b = 0 if s.shape[0] == 1 else s.stride(0)
            self.seg_len = s.shape[1]
            self.seg_tiles = (self.seg_len + L.RA_SEG_TILE - 1) // L.RA_SEG_TILE
            self.seg_mm = self._seg_entry[2]
            self.seg_hull = self._seg_entry[5]
        # set by a caller that knows that segment_ids covers every global position of its calls (no clamped slices):
        # the kernels may then look their tile hulls up in the per-run table instead of scanning the tile ranges
        self.seg_covers = False
        self.keep = None                   # boolean mask: ring_attention_inference (set_keep) or dropout
        self.keep_strides = (0, 0, 0, 0)
        self.keep_row0 = 0
        self.keep_k0 = 0
        self.keep_mode = L.RA_KEEP_WHERE
        self.keep_packed = None
        self._drop_base = None             # (B, H, q_len, kv_len) keep bytes of the dropout mask, if needed
        self._drop_shape = None
        self._drop_steps = {}
        self.cache_idx_host = None
        self.cache_idx_dev = None
        if cache_idx is not None:
            if isinstance(cache_idx, torch.Tensor):
                if cache_idx.is_cuda:
                    self.cache_idx_dev = cache_idx.detach().to(torch.int32).reshape(1).contiguous()
                else:
                    self.cache_idx_host = int(cache_idx)
            else:
                self.cache_idx_host = int(cache_idx)

    @staticmethod
    def _segment_entry(segment_ids, device, stream):
        """[weakref, int32 ids on the device, per-64-position (min, max) id ranges, host copy of the ranges (lazy),
        the stream that produced them, per-128-position tile hulls (ra_segment_run_hulls; None without a GPU)]."""
        s = segment_ids.detach().to(device=device, dtype=torch.int32).contiguous()
        tiles = (s.shape[1] + L.RA_SEG_TILE - 1) // L.RA_SEG_TILE
        mm = torch.empty((s.shape[0], tiles, 2), dtype=torch.int32, device=device)
        hull = None
        if s.is_cuda:
            # lets the MFMA kernels skip tiles of foreign segments
            L.check(L.load().ra_segment_tile_ranges(s.data_ptr(), s.stride(0), s.shape[0], s.shape[1],
                                                    mm.data_ptr(), _stream()), "ra_segment_tile_ranges")
            hull = torch.empty((s.shape[0], (tiles + 1) // 2, 2), dtype=torch.int32, device=device)
            L.check(L.load().ra_segment_run_hulls(mm.data_ptr(), s.shape[0], tiles, hull.data_ptr(), _stream()),
                    "ra_segment_run_hulls")
        else:                                  # host logic only (tests without a GPU): same ranges with torch ops
            pad = tiles * L.RA_SEG_TILE - s.shape[1]
            sp = torch.nn.functional.pad(s, (0, pad), mode="replicate") if pad else s
            sp = sp.view(s.shape[0], tiles, L.RA_SEG_TILE)
            mm = torch.stack((sp.amin(dim=2), sp.amax(dim=2)), dim=2).to(torch.int32)
        return [weakref.ref(segment_ids), s, mm, None, stream, hull]

    def set_keep(self, attn_mask, device, q_total, k_total):
        """attn_mask (B|1, H|1, Q|1, K_total), nonzero = attend (ringattention_inference.py:19-22).
        When both global lengths divide by 64 the mask is also packed into 64-bit words and a per-tile
        summary (ra_keep_pack), the form the MFMA kernels read."""
        if attn_mask.dim() != 4:
            raise ValueError("attn_mask must be 4-D (B, H, Q, K)")
        m = attn_mask.detach().to(device=device)
        if m.dtype == torch.bool:
            m = m.contiguous().view(torch.uint8)          # same bytes, no copy for a contiguous bool mask
        else:
            m = (m != 0).to(torch.uint8).contiguous()
        self.keep = m
        self.keep_strides = tuple(0 if m.shape[i] == 1 else m.stride(i) for i in range(4))
        self.keep_packed = None
        if q_total % 64 == 0 and k_total % 64 == 0:
            bits_k, bits_q, summ = self._pack(m, self.keep_strides, q_total, k_total)
            bm, hm = m.shape[0], m.shape[1]
            # a query row with no attended key keeps equal finfo.min logits (uniform weights): kernels must
            # not skip its fully masked tiles.  Read off the packed words (an eighth of the mask's bytes).
            row_has_key = (bits_k.view(bm, hm, k_total // 64, q_total) != 0).any(dim=2)
            self.keep_has_empty_row = not bool(row_has_key.all().item())
            self.keep_packed = (bits_k, bits_q, summ, q_total, k_total)
        else:
            self.keep_has_empty_row = bool((m.amax(dim=3) == 0).any().item())

    @staticmethod
    def _pack(m, strides, q_total, k_total):
        """ra_keep_pack of a (Bm, Hm, Q|1, K) byte mask: the 64-bit words by key tile and by query tile, and the
        per-tile summary."""
        bm, hm = m.shape[0], m.shape[1]
        words = q_total * k_total // 64
        bits_k = torch.empty((bm, hm, words), dtype=torch.int64, device=m.device)
        bits_q = torch.empty((bm, hm, words), dtype=torch.int64, device=m.device)
        summ = torch.empty((bm, hm, (q_total // 64) * (k_total // 64)), dtype=torch.uint8, device=m.device)
        L.check(L.load().ra_keep_pack(m.data_ptr(), m.stride(0), m.stride(1), strides[2], m.stride(3),
                                      bm, hm, q_total, k_total, bits_k.data_ptr(), bits_q.data_ptr(),
                                      summ.data_ptr(), _stream()), "ra_keep_pack")
        return bits_k, bits_q, summ

    def use_dropout(self, cfg, batch, heads, q_len, kv_len, q_chunk_idx_start, k_chunk_idx_start, device):
        """Points the keep mask at the dropout mask of this step (ringattention_jax.py:119-123, :311-321).

        The reference draws ONE mask of the local shape (batch, heads, q_len, kv_len) per call - the same in
        every ring step, the key being a constant of blockwise_kwargs - and slices it with dynamic_slice at the
        GLOBAL chunk offsets, which clamps: chunk j of a step whose chunk index starts at s reads the mask rows
        min((s + j) * qc, q_len - qc) ..., and likewise along the keys.  Steps that start at 0 read the mask as
        it is; every other start is served by a gathered copy, cached per (row start, key start)."""
        if self.cache_idx_host is not None or self.cache_idx_dev is not None:
            raise NotImplementedError("attention dropout together with cache_idx is not supported")
        if kv_len % 8:
            raise NotImplementedError("attention dropout needs a key length that is a multiple of 8")
        shape = (batch, heads, q_len, kv_len)
        if self._drop_shape is None:
            self._drop_shape = shape
        elif self._drop_shape != shape:
            raise ValueError("the dropout mask of this call was drawn for another shape")
        nq, nk = q_len // cfg.qc, kv_len // cfg.kc
        key = (min(q_chunk_idx_start, nq), min(k_chunk_idx_start, nk))
        aligned = q_len % 64 == 0 and kv_len % 64 == 0
        if key not in self._drop_steps and key == (0, 0) and aligned:
            # the mask as drawn, written in packed form at once (no byte array: the kernels read the words)
            words = q_len * kv_len // 64
            bits_k = torch.empty((batch, heads, words), dtype=torch.int64, device=device)
            bits_q = torch.empty((batch, heads, words), dtype=torch.int64, device=device)
            summ = torch.empty((batch, heads, words // 64), dtype=torch.uint8, device=device)
            # (only the tiles of chunk pairs that run under the causal block size: nothing else is read)
            L.check(L.load().ra_dropout_keep_packed(cfg.seed, cfg.pdrop, batch, heads, q_len, kv_len,
                                                    bits_k.data_ptr(), bits_q.data_ptr(), summ.data_ptr(),
                                                    cfg.cbs or 0, cfg.qc, cfg.kc, 0, 0, _stream()),
                    "ra_dropout_keep_packed")
            self._drop_steps[key] = (None, (bits_k, bits_q, summ, q_len, kv_len))
        if key not in self._drop_steps:
            if self._drop_base is None:
                base = torch.empty(shape, dtype=torch.uint8, device=device)
                L.check(L.load().ra_dropout_keep(cfg.seed, cfg.pdrop, batch, heads, q_len, kv_len, base.data_ptr(),
                                                 _stream()), "ra_dropout_keep")
                self._drop_base = base
            m = self._drop_base
            if key[0] != 0:
                starts = torch.clamp((key[0] + torch.arange(nq, device=device)) * cfg.qc, max=q_len - cfg.qc)
                m = m.index_select(2, (starts[:, None] + torch.arange(cfg.qc, device=device)).reshape(-1))
            if key[1] != 0:
                starts = torch.clamp((key[1] + torch.arange(nk, device=device)) * cfg.kc, max=kv_len - cfg.kc)
                m = m.index_select(3, (starts[:, None] + torch.arange(cfg.kc, device=device)).reshape(-1))
            packed = None
            if aligned:
                packed = self._pack(m, m.stride(), q_len, kv_len) + (q_len, kv_len)
                m = None if key != (0, 0) else m          # the gathered bytes are not needed once packed
            self._drop_steps[key] = (m, packed)
        self.keep, self.keep_packed = self._drop_steps[key]
        self.keep_strides = self.keep.stride() if self.keep is not None else (0, 0, 0, 0)
        self.keep_row0 = 0
        self.keep_k0 = k_chunk_idx_start * cfg.kc
        self.keep_mode = L.RA_KEEP_DROPOUT

    def fill(self, cfg, q_chunk_idx_start, k_chunk_idx_start, skip, chunk_starts=None):
        m = L.RaMask()
        if chunk_starts is not None:            # int32[2] in device memory: the kernels read the starts there
            self._chunk_starts = chunk_starts   # kept alive with the mask inputs
            m.chunk_starts = chunk_starts.data_ptr()
            q_chunk_idx_start = k_chunk_idx_start = 0
        m.bias = self.bias.data_ptr() if self.bias is not None else None
        m.bias_stride_b, m.bias_stride_h, m.bias_stride_q, m.bias_stride_k = self.bias_strides
        m.segment_ids = self.seg.data_ptr() if self.seg is not None else None
        m.seg_stride_b = self.seg_stride_b
        m.seg_len = self.seg_len
        m.causal_block_size = 0 if cfg.cbs is None else cfg.cbs
        m.query_chunk_size = cfg.qc
        m.key_chunk_size = cfg.kc
        m.q_chunk_idx_start = q_chunk_idx_start
        m.k_chunk_idx_start = k_chunk_idx_start
        m.cache_idx = self.cache_idx_dev.data_ptr() if self.cache_idx_dev is not None else None
        m.mask_min = cfg.mask_min
        m.skip_masked_tiles = 1 if skip else 0
        m.seg_tile_minmax = self.seg_mm.data_ptr() if self.seg_mm is not None else None
        m.seg_tiles = self.seg_tiles
        if self.seg_hull is not None and self.seg_covers and chunk_starts is None:
            m.seg_run_hulls = self.seg_hull.data_ptr()
            m.seg_runs = (self.seg_tiles + 1) // 2
        if self.keep is not None or self.keep_packed is not None:
            if self.keep is not None:
                m.keep = self.keep.data_ptr() + self.keep_row0 * self.keep_strides[2]
                m.keep_stride_b, m.keep_stride_h, m.keep_stride_q, m.keep_stride_k = self.keep_strides
            if self.keep_packed is not None:
                bits_k, bits_q, summ, q_total, k_total = self.keep_packed
                m.keep_bits_k, m.keep_bits_q, m.keep_summary = bits_k.data_ptr(), bits_q.data_ptr(), summ.data_ptr()
                m.keep_pack_stride_b = 0 if bits_k.shape[0] == 1 else bits_k.stride(0)
                m.keep_pack_stride_h = 0 if bits_k.shape[1] == 1 else bits_k.stride(1)
                m.keep_sum_stride_b = 0 if summ.shape[0] == 1 else summ.stride(0)
                m.keep_sum_stride_h = 0 if summ.shape[1] == 1 else summ.stride(1)
                m.keep_q_total, m.keep_k_total, m.keep_q0 = q_total, k_total, self.keep_row0
            m.keep_k0 = self.keep_k0
            m.keep_mode = self.keep_mode
        return m

    def segments_meet(self, q_lo, q_hi, k_lo, k_hi):
        """False when no batch row has a segment id present both in global query positions
        [q_lo, q_hi) and in global key positions [k_lo, k_hi) (conservative: id ranges are compared).
        Costs one device->host copy of the per-tile ranges per segment_ids tensor (kept while it is unchanged)."""
        if self.seg_mm is None:
            return True
        if self._seg_entry[3] is None:
            self._seg_entry[3] = self.seg_mm.cpu().numpy()
        mm = self._seg_entry[3]
        t = L.RA_SEG_TILE
        qs = mm[:, q_lo // t:max(q_lo // t + 1, -(-q_hi // t))]
        ks = mm[:, k_lo // t:max(k_lo // t + 1, -(-k_hi // t))]
        q_min, q_max = qs[..., 0].min(axis=1), qs[..., 1].max(axis=1)
        k_min, k_max = ks[..., 0].min(axis=1), ks[..., 1].max(axis=1)
        return bool(((k_max >= q_min) & (k_min <= q_max)).any())


def _check_qkv(q, k, v):
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise RuntimeError("ringattention_amd runs on the GPU only: q, k, v must be device tensors")
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4 or v.shape != k.shape:
        raise ValueError("q, k, v must be (B, S, H, D) with k.shape == v.shape")
    if q.shape[0] != k.shape[0] or q.shape[2:] != k.shape[2:]:
        raise ValueError("q and k must agree in batch, heads and head size")
    if not (q.dtype == k.dtype == v.dtype):
        raise ValueError("q, k, v must share a dtype")


def _row_dense(t):
    """(B, S, H, D) with the last three dims laid out as one dense row of H * D elements per position."""
    return t.stride(3) == 1 and t.stride(2) == t.shape[3] and t.stride(1) == t.shape[2] * t.shape[3]


def _rows(t):
    """(stride_b, stride_s) of a (B, S, H, D) tensor whose last two dims are dense."""
    if t.stride(3) != 1 or t.stride(2) != t.shape[3]:
        raise ValueError("tensor must be dense in its last two (H, D) dims")
    return t.stride(0), t.stride(1)


# --------------------------------------------------------------------------- which kernels ran
_FAMILY_NAMES = {L.RA_FAMILY_GENERIC: "generic", L.RA_FAMILY_MFMA_BF16: "mfma_bf16", L.RA_FAMILY_MFMA_F32: "mfma_f32",
                 L.RA_FAMILY_MFMA_BF16_ANY: "mfma_bf16_any"}
_LAST_FAMILY = {"forward": None, "backward": None}
_WARNED = set()
_GENERIC_WARN_PAIRS = 1 << 28         # B * H * q_len * kv_len from which the vector-ALU kernels take seconds


def kernel_family_of_last_call():
    """{"forward": ..., "backward": ...}: the kernel family ("mfma_bf16", "mfma_f32", "mfma_bf16_any" - the
    matrix-core kernels that evaluate the mask element by element -, "generic") that the last attention launch of
    each direction ran on - what blockwise_kwargs["impl"] = "auto" (the default) chose."""
    return dict(_LAST_FAMILY)


def _note_family(direction, fam, cfg, q, k, mi):
    _LAST_FAMILY[direction] = _FAMILY_NAMES.get(fam)
    if fam != L.RA_FAMILY_GENERIC or cfg.impl != L.RA_IMPL_AUTO:
        return
    B, Sq, H, D = q.shape
    if B * H * Sq * k.shape[1] < _GENERIC_WARN_PAIRS:
        return
    why = []
    if q.dtype not in (torch.bfloat16, torch.float32):
        why.append("dtype %s" % q.dtype)
    if D not in (64, 128):
        why.append("head size %d (64 and 128 are taken as they are, smaller ones zero-padded)" % D)
    if cfg.qc % 128 or cfg.kc % 128:
        why.append("chunk sizes (%d, %d) that are no multiples of 128 and cannot be re-chunked (odd sizes under a "
                   "causal mask, a ragged shard, dropout)" % (cfg.qc, cfg.kc))
    if mi.bias is not None and mi.bias_strides[2] != 0:
        why.append("a bias with one row per query")
    if mi.keep is not None and mi.keep_packed is None:
        why.append("a boolean mask whose lengths are no multiples of 64")
    key = (direction, tuple(why))
    if key in _WARNED:
        return
    _WARNED.add(key)
    warnings.warn("ringattention_amd: this %s call runs on the generic vector-ALU kernels, about a hundred times "
                  "slower than the matrix-core kernels at this size, because of %s"
                  % (direction, "; ".join(why) or "its strides or alignment"), RuntimeWarning, stacklevel=4)


# --------------------------------------------------------------------------- one ring step
def _device_chunk_starts(q_chunk_idx_start, k_chunk_idx_start, device):
    """The chunk starts as the kernels take them from device memory (ra_mask.chunk_starts), or None when both are
    Python ints.  Under jit the reference computes them from lax.axis_index (:31-37, :69-75), a traced value; the
    counterpart here is a device tensor: either one int32 tensor of two elements passed as q_chunk_idx_start (with
    k_chunk_idx_start None: no kernel is launched to pack them, so the call can be captured into a HIP graph and
    replayed with other values in the tensor), or two scalars of which at least one is a device tensor."""
    qt, kt = isinstance(q_chunk_idx_start, torch.Tensor), isinstance(k_chunk_idx_start, torch.Tensor)
    if not qt and not kt:
        return None
    if qt and k_chunk_idx_start is None:
        cs = q_chunk_idx_start
        if cs.numel() != 2 or cs.dtype != torch.int32 or not cs.is_cuda or not cs.is_contiguous():
            raise ValueError("chunk starts in one tensor: a contiguous int32 device tensor of two elements")
        return cs.reshape(2)
    parts = [t.to(device=device, dtype=torch.int32).reshape(1) if isinstance(t, torch.Tensor)
             else torch.tensor([int(t)], dtype=torch.int32, device=device) for t in (q_chunk_idx_start, k_chunk_idx_start)]
    return torch.cat(parts)


def _blockwise_attention_fwd(q, k, v, carry, q_chunk_idx_start, k_chunk_idx_start, bias, segment_ids,
                             causal_block_size, query_chunk_size, key_chunk_size, deterministic=True,
                             dropout_rng=None, attn_pdrop=0.0, dtype=torch.float32, policy=None,
                             precision=None, prevent_cse=True, cache_idx=None, _mask_inputs=None,
                             _cfg=None, _carry_is_initial=False, _out=None, _out_f32=None, **extra):
    """ringattention_jax.py:99-179.  ``carry`` = (numerator (B,Sq,H,D), denominator (B,H,Sq),
    max_score (B,H,Sq)), fp32, updated IN PLACE and returned.  With ``_out`` (B,Sq,H,D in q's dtype) the step is
    the last one of its device: out = numerator / denominator (:52) is written there instead of the numerator,
    which may then be None if the carry is initial; ``_out_f32`` (fp32, the strides of ``_out``) takes the same
    quotient before it is rounded (the residual of :53)."""
    cfg = _cfg or _Config(dict(causal_block_size=causal_block_size, query_chunk_size=query_chunk_size,
                               key_chunk_size=key_chunk_size, deterministic=deterministic,
                               attn_pdrop=attn_pdrop, dtype=dtype, **extra))
    _check_qkv(q, k, v)
    B, Sq, H, D = q.shape
    Skv = k.shape[1]
    starts_dev = _device_chunk_starts(q_chunk_idx_start, k_chunk_idx_start, q.device)
    if starts_dev is not None:
        q_chunk_idx_start = k_chunk_idx_start = 0      # unknown to the host: nothing below may depend on them
        if cfg.pdrop > 0.0:
            raise NotImplementedError("attention dropout needs chunk starts the host knows")
    mi = _mask_inputs or _MaskInputs(cfg, bias, segment_ids, cache_idx, B, q.device,
                                     (k_chunk_idx_start * cfg.kc + Skv) if starts_dev is None else 0, H)
    num, den, mx = carry
    p = L.RaAttnFwdParams()
    p.q, p.k, p.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    p.dtype = _ra_dtype(q)
    p.B, p.Sq, p.Skv, p.H, p.D = B, Sq, Skv, H, D
    p.q_stride_b, p.q_stride_s = _rows(q)
    p.kv_stride_b, p.kv_stride_s = _rows(k)
    if _rows(v) != _rows(k):
        raise ValueError("k and v must share strides")
    if num is not None:
        p.numerator = num.data_ptr()
        p.num_stride_b, p.num_stride_s = _rows(num)
    else:
        p.num_stride_b, p.num_stride_s = Sq * H * D, H * D
    if _out is not None:
        if _out.dtype != q.dtype:
            raise ValueError("out must have the dtype of q")
        p.out = _out.data_ptr()
        p.out_stride_b, p.out_stride_s = _rows(_out)
        if _out_f32 is not None:
            if _out_f32.dtype != torch.float32 or _rows(_out_f32) != _rows(_out):
                raise ValueError("out_f32 must be fp32 with the strides of out")
            p.out_f32 = _out_f32.data_ptr()
    p.denominator, p.max_score = den.data_ptr(), mx.data_ptr()
    if den.stride() != mx.stride() or den.stride(2) != 1:
        raise ValueError("denominator / max_score must share strides and be dense in the last dim")
    p.stat_stride_b, p.stat_stride_h = den.stride(0), den.stride(1)
    if mi.cache_idx_host is not None:
        q_chunk_idx_start = mi.cache_idx_host // cfg.qc                    # :35
    skip = cfg.skip_masked_tiles
    if skip is None:
        skip = cfg.qc >= 2 and cache_idx is None
    if cfg.pdrop > 0.0:
        mi.use_dropout(cfg, B, H, Sq, Skv, q_chunk_idx_start, k_chunk_idx_start, q.device)
        skip = False        # a row may lose every allowed key: its masked tiles then carry its (uniform) weights
    p.mask = mi.fill(cfg, q_chunk_idx_start, k_chunk_idx_start, skip, starts_dev)
    p.impl = cfg.impl
    p.logit_dim = cfg.logit_dim
    p.carry_is_initial = 1 if _carry_is_initial else 0
    _note_family("forward", L.load().ra_attn_fwd_family(ctypes.byref(p)), cfg, q, k, mi)
    L.check(L.load().ra_attn_fwd_block(ctypes.byref(p), _stream()), "ra_attn_fwd_block")
    return num, den, mx


def _blockwise_attention_bwd(q, k, v, g, carry, q_chunk_idx_start, k_chunk_idx_start, bias, segment_ids,
                             causal_block_size, query_chunk_size, key_chunk_size, deterministic=True,
                             dropout_rng=None, attn_pdrop=0.0, dtype=torch.float32, policy=None,
                             precision=None, prevent_cse=True, cache_idx=None, _mask_inputs=None,
                             _cfg=None, _delta=None, _grads_initial=0, _dq_out=None, _dkv_out=None, **extra):
    """ringattention_jax.py:181-270.  ``carry`` = (dq, dk, dv, output, denominator, max_score); the
    fp32 accumulators dq, dk, dv are added into IN PLACE and returned.  ``_grads_initial`` (RA_GRAD_INIT_*) marks
    accumulators that hold zeros by definition (not read; may be None with the matching output); ``_dq_out`` /
    ``_dkv_out = (dk_out, dv_out)`` in q's dtype mark the last call that adds into them: the sum is written there
    (the cast of :89) and the accumulator is left alone."""
    cfg = _cfg or _Config(dict(causal_block_size=causal_block_size, query_chunk_size=query_chunk_size,
                               key_chunk_size=key_chunk_size, deterministic=deterministic,
                               attn_pdrop=attn_pdrop, dtype=dtype, **extra))
    _check_qkv(q, k, v)
    B, Sq, H, D = q.shape
    Skv = k.shape[1]
    starts_dev = _device_chunk_starts(q_chunk_idx_start, k_chunk_idx_start, q.device)
    if starts_dev is not None:
        q_chunk_idx_start = k_chunk_idx_start = 0
        if cfg.pdrop > 0.0:
            raise NotImplementedError("attention dropout needs chunk starts the host knows")
    mi = _mask_inputs or _MaskInputs(cfg, bias, segment_ids, cache_idx, B, q.device,
                                     (k_chunk_idx_start * cfg.kc + Skv) if starts_dev is None else 0, H)
    dq, dk, dv, output, den, mx = carry
    if g.dtype != q.dtype:
        g = g.to(q.dtype)
    if _rows(g) != _rows(q):
        g = g.contiguous()
        if _rows(g) != _rows(q):
            raise ValueError("g must share q's strides")
    delta = _delta if _delta is not None else _bwd_delta(g, output)
    p = L.RaAttnBwdParams()
    p.q, p.k, p.v, p.g = q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr()
    p.dtype = _ra_dtype(q)
    p.B, p.Sq, p.Skv, p.H, p.D = B, Sq, Skv, H, D
    p.q_stride_b, p.q_stride_s = _rows(q)
    p.kv_stride_b, p.kv_stride_s = _rows(k)
    p.delta, p.denominator, p.max_score = delta.data_ptr(), den.data_ptr(), mx.data_ptr()
    if not (delta.stride() == den.stride() == mx.stride()):
        raise ValueError("delta / denominator / max_score must share strides")
    p.stat_stride_b, p.stat_stride_h = den.stride(0), den.stride(1)
    if dq is not None:
        p.dq = dq.data_ptr()
        p.dq_stride_b, p.dq_stride_s = _rows(dq)
    else:
        p.dq_stride_b, p.dq_stride_s = Sq * H * D, H * D
    if dk is not None:
        p.dk, p.dv = dk.data_ptr(), dv.data_ptr()
        p.dkv_stride_b, p.dkv_stride_s = _rows(dk)
        if _rows(dv) != _rows(dk):
            raise ValueError("dk and dv must share strides")
    else:
        p.dkv_stride_b, p.dkv_stride_s = Skv * H * D, H * D
    p.grads_are_initial = _grads_initial
    if _dq_out is not None:
        if _dq_out.dtype != q.dtype:
            raise ValueError("dq_out must have the dtype of q")
        p.dq_out = _dq_out.data_ptr()
        p.dq_out_stride_b, p.dq_out_stride_s = _rows(_dq_out)
    if _dkv_out is not None:
        dko, dvo = _dkv_out
        if dko.dtype != q.dtype or dvo.dtype != q.dtype or _rows(dko) != _rows(dvo):
            raise ValueError("dk_out and dv_out must have the dtype of q and share strides")
        p.dk_out, p.dv_out = dko.data_ptr(), dvo.data_ptr()
        p.dkv_out_stride_b, p.dkv_out_stride_s = _rows(dko)
    if mi.cache_idx_host is not None:
        q_chunk_idx_start = mi.cache_idx_host // cfg.qc
    skip = cfg.skip_masked_tiles
    if skip is None:
        skip = cfg.qc >= 2 and cache_idx is None
    if cfg.pdrop > 0.0:
        mi.use_dropout(cfg, B, H, Sq, Skv, q_chunk_idx_start, k_chunk_idx_start, q.device)
        skip = False
    p.mask = mi.fill(cfg, q_chunk_idx_start, k_chunk_idx_start, skip, starts_dev)
    p.impl = cfg.impl
    p.logit_dim = cfg.logit_dim
    _note_family("backward", L.load().ra_attn_bwd_family(ctypes.byref(p)), cfg, q, k, mi)
    if cfg.bwd_only:
        L.check(L.load().ra_attn_bwd_block_part(ctypes.byref(p), cfg.bwd_only, _stream()), "ra_attn_bwd_block_part")
    else:
        L.check(L.load().ra_attn_bwd_block(ctypes.byref(p), _stream()), "ra_attn_bwd_block")
    return dq, dk, dv


def _bwd_delta(g, output):
    """dl_part of ringattention_jax.py:218: sum_d g * output, (B, H, Sq) fp32.  ``output`` is the forward output in
    g's dtype or, as in the reference (:53), un-rounded in fp32."""
    B, Sq, H, D = g.shape
    if output.dtype not in (g.dtype, torch.float32):
        output = output.to(g.dtype)
    if _rows(output) != _rows(g):
        output = output.contiguous()
        g = g.contiguous()
    delta = torch.empty((B, H, Sq), dtype=torch.float32, device=g.device)
    sb, ss = _rows(g)
    L.check(L.load().ra_attn_bwd_delta(g.data_ptr(), output.data_ptr(), _ra_dtype(g), _ra_dtype(output), sb, ss,
                                       delta.data_ptr(), delta.stride(0), delta.stride(1), B, Sq, H, D, _stream()),
            "ra_attn_bwd_delta")
    return delta


def _finalize(num, den, out):
    B, Sq, H, D = num.shape
    nb, ns = _rows(num)
    ob, os_ = _rows(out)
    L.check(L.load().ra_attn_finalize(num.data_ptr(), nb, ns, den.data_ptr(), den.stride(0), den.stride(1),
                                      out.data_ptr(), _ra_dtype(out), ob, os_, B, Sq, H, D, _stream()),
            "ra_attn_finalize")


def _carry_init(num, den, mx):
    B, Sq, H, D = num.shape
    nb, ns = _rows(num)
    L.check(L.load().ra_attn_carry_init(num.data_ptr(), nb, ns, den.data_ptr(), mx.data_ptr(), den.stride(0),
                                        den.stride(1), B, Sq, H, D, _stream()), "ra_attn_carry_init")


# --------------------------------------------------------------------------- the ring
def _q_start(cfg, mi, dev, q_len):
    if mi.cache_idx_host is not None:
        return mi.cache_idx_host // cfg.qc                                   # :35
    if mi.cache_idx_dev is not None:
        return 0            # resolved on the device from the cache_idx scalar
    return dev * (q_len // cfg.qc)                                           # :32-33


def _step_runs(cfg, mi, q_start, q_len, k_start, kv_len):
    """False when the skip predicate drops every tile of this ring step (whole future shards), or -
    with skip_masked_tiles - when no segment id is shared between the query and the key shard."""
    if mi.cache_idx_dev is not None:
        return True
    if cfg.cbs is not None:
        last_q_chunk = q_start + q_len // cfg.qc - 1
        if run_prefix_keys(last_q_chunk, cfg.qc, cfg.kc, cfg.cbs, k_start, kv_len) <= 0:
            return False
    if cfg.skip_masked_tiles and mi.seg_mm is not None:
        return mi.segments_meet(q_start * cfg.qc, q_start * cfg.qc + q_len, k_start * cfg.kc,
                                k_start * cfg.kc + kv_len)
    return True


def _ring_attention_fwd(q, k, v, attn_bias, segment_ids, cache_idx, axis_name, float32_logits, blockwise_kwargs):
    """ringattention_jax.py:17-53 for every device of the virtual ring.

    Logits, softmax statistics and the carry are always fp32 (what float32_logits=True asks for;
    with False the reference computes them in the input dtype, which this path exceeds).
    Returns (out, residuals)."""
    cfg = _Config(blockwise_kwargs)
    _check_qkv(q, k, v)
    # the kernels take any batch stride, rows of H * D elements one after the other; k and v share theirs; the
    # cotangent arrives dense and shares q's strides, so q is dense too.  Any other view (a slice of a fused q/k/v
    # projection, a transposed (B, H, S, D) array, the first positions of a longer q) is copied once
    q = q.contiguous()
    k, v = (t if _row_dense(t) else t.contiguous() for t in (k, v))
    if k.stride(0) != v.stride(0):
        k, v = k.contiguous(), v.contiguous()
    n = axis_size(axis_name)
    B, q_total, H, D = q.shape
    kv_total = k.shape[1]
    if q_total % n or kv_total % n:
        raise ValueError("sequence lengths must divide by the ring size %d" % n)
    q_len, kv_len = q_total // n, kv_total // n
    if q_len % cfg.qc or kv_len % cfg.kc:
        raise ValueError("per-device lengths (%d, %d) must divide by the chunk sizes (%d, %d)"
                         % (q_len, kv_len, cfg.qc, cfg.kc))
    mi = _MaskInputs(cfg, attn_bias, segment_ids, cache_idx, B, q.device, kv_total, H)
    mi.seg_covers = (mi.seg is not None and cache_idx is None and mi.seg_len >= max(q_total, kv_total)
                     and cfg.segment_hull_table)
    if cfg.skip_masked_tiles is None:
        cfg.skip_masked_tiles = bool(cfg.qc >= 2 and cache_idx is None and q_total == kv_total)
    if cfg.pdrop > 0.0:
        if cache_idx is not None:
            raise NotImplementedError("attention dropout together with cache_idx is not supported")
        cfg.skip_masked_tiles = False      # dropout can leave a row without any allowed key
    _fit_chunks_to_mfma_grid(cfg, mi, q, q_len, kv_len, q_total, kv_total)
    d_true = D
    pad_to = _padded_head_size(cfg, mi, q)
    if pad_to:
        # a head size the matrix-core kernels do not tile: q, k, v zero-padded along D (the products are those of the
        # un-padded rows), the logits still divided by sqrt of the original head size (:118)
        q, k, v = (torch.nn.functional.pad(t, (0, pad_to - D)) for t in (q, k, v))
        cfg.logit_dim = D
        D = pad_to
    den = torch.empty((B, H, q_total), dtype=torch.float32, device=q.device)         # :23
    mx = torch.empty((B, H, q_total), dtype=torch.float32, device=q.device)          # :49
    out = torch.empty((B, q_total, H, D), dtype=v.dtype, device=q.device)
    # the residual `output` of :53 is the quotient before it is rounded to v's dtype
    out32 = None
    if cfg.output_residual == "fp32" and out.dtype != torch.float32:
        out32 = torch.empty((B, q_total, H, D), dtype=torch.float32, device=q.device)
    plan = _ring_plan(cfg, mi, n, q_len, kv_len)
    # the numerator carry (:22) only exists between the steps of a device: its first step starts it (nothing is
    # read), its last step writes out = numerator / denominator (:52) instead
    num = None
    if any(len(steps) > 1 for steps in plan.values()):
        num = torch.empty((B, q_total, H, D), dtype=torch.float32, device=q.device)
    whole = _ring_step_launches(cfg, mi, n) and q.dtype == torch.bfloat16      # those entry points take bf16 only
    for idx in range(n):                    # the scan of :29-51; all devices run a step side by side
        devs = [dev for dev in range(n) if idx in plan[dev]]
        if whole and devs:
            whole = _fwd_ring_step(q, k, v, (num, den, mx), out, out32, cfg, mi, n, idx, plan, devs)
            if whole:
                continue
        for dev in devs:
            qs = slice(dev * q_len, (dev + 1) * q_len)
            q_start, k_blk, k_start = plan[dev][idx]
            ks = slice(k_blk * kv_len, (k_blk + 1) * kv_len)
            carry = (num[:, qs] if num is not None else None, den[:, :, qs], mx[:, :, qs])
            _blockwise_attention_fwd(q[:, qs], k[:, ks], v[:, ks], carry, q_start, k_start, None, None,
                                     cfg.cbs, cfg.qc, cfg.kc, _mask_inputs=mi, _cfg=cfg,
                                     _carry_is_initial=idx == min(plan[dev]), cache_idx=cache_idx,
                                     _out=out[:, qs] if idx == max(plan[dev]) else None,
                                     _out_f32=out32[:, qs] if out32 is not None and idx == max(plan[dev]) else None)
    for dev in range(n):
        if not plan[dev]:                   # no tile runs for this device: 0 / 0
            qs = slice(dev * q_len, (dev + 1) * q_len)
            carry = (num[:, qs] if num is not None else torch.empty((B, q_len, H, D), dtype=torch.float32,
                                                                    device=q.device), den[:, :, qs], mx[:, :, qs])
            _carry_init(*carry)
            _finalize(carry[0], carry[1], out[:, qs])
            if out32 is not None:
                _finalize(carry[0], carry[1], out32[:, qs])
    del num
    res = (out if out32 is None else out32, q, k, v, mi, cfg, n, den, mx)
    if D != d_true:
        out = out[..., :d_true].contiguous()
    return out, res


def _padded_head_size(cfg, mi, q):
    """The head size to zero-pad q, k, v to (the products are those of the un-padded rows; the logits keep the scale
    of the original head size), or 0 when the kernels take the head size as it is.  The tiled matrix-core kernels take
    64 and 128; a bf16 call that leaves their grid (chunk sizes off the 128-grid, a per-row bias, an unpacked boolean
    mask, a head size above 128) goes to the matrix-core kernels that evaluate the mask element by element, which
    take 128 and 256; what is left - fp32 inputs off the grid, attention dropout there, the generic kernels asked for
    by name - runs on the generic kernels, which take 32, 64, 128 and 256."""
    D = q.shape[3]
    if D > 256:
        raise NotImplementedError("head size %d: the kernels take head sizes up to 256" % D)
    generic = (cfg.impl in (L.RA_IMPL_GENERIC, L.RA_IMPL_MFMA_ANY) or D > 128
               or q.dtype not in (torch.bfloat16, torch.float32)
               or cfg.qc % 128 or cfg.kc % 128 or (mi.bias is not None and mi.bias_strides[2] != 0)
               or (mi.keep is not None and mi.keep_packed is None))
    if generic and q.dtype == torch.bfloat16 and cfg.impl != L.RA_IMPL_GENERIC and cfg.pdrop == 0.0:
        to = 128 if D <= 128 else 256       # the matrix-core kernels that evaluate the mask element by element
    elif generic:
        to = next(s for s in (32, 64, 128, 256) if D <= s)
    else:
        to = 64 if D <= 64 else 128
    return 0 if to == D else to


def _fit_chunks_to_mfma_grid(cfg, mi, q, q_len, kv_len, q_total, kv_total, grid=128):
    """Chunk sizes the MFMA kernels do not tile (they want multiples of 128) are replaced by 128 where that cannot
    change the result.  The chunk sizes enter the reference's result in four places only: which chunk pairs run
    (below_or_on_diag, :324-331), the clamped slices of segment_ids (:286-295) and of the dropout mask (:311-320),
    and the rows of a per-row bias (:279-283).  With causal_block_size 1 and even chunk sizes - or a block size that
    divides both chunk sizes - a chunk pair that does not run holds causally masked pairs only (its last row lies
    before its first key, and a tie is impossible), and a masked pair weighs exp(finfo.min - max) = 0 exactly as
    long as its row has an unmasked key, which is what skip_masked_tiles already asks for; so both chunkings sum
    over the same pairs.  Without a causal block size every chunk pair runs.  The slices are not clamped when the
    segment ids cover every position, there is no dropout here, and a per-row bias takes the generic kernels."""
    if cfg.impl in (L.RA_IMPL_GENERIC, L.RA_IMPL_MFMA_ANY) or q.dtype not in (torch.bfloat16, torch.float32) \
            or q.shape[3] > 128:
        return
    if cfg.qc % grid == 0 and cfg.kc % grid == 0:
        return
    if q_len % grid or kv_len % grid or cfg.pdrop > 0.0 or not cfg.skip_masked_tiles:
        return
    if mi.cache_idx_host is not None or mi.cache_idx_dev is not None or mi.keep is not None:
        return
    if mi.bias is not None and mi.bias_strides[2] != 0:
        return
    if mi.seg is not None and mi.seg_len < max(q_total, kv_total):
        return
    if cfg.cbs is not None:
        if cfg.cbs == 1:
            if cfg.qc % 2 or cfg.kc % 2:
                return
        elif cfg.qc % cfg.cbs or cfg.kc % cfg.cbs or grid % cfg.cbs:
            return
    cfg.qc = cfg.kc = grid


def _ring_plan(cfg, mi, n, q_len, kv_len):
    """For every device of the virtual ring the scan steps that run: {dev: {idx: (q_chunk_idx_start, index of the
    K/V shard that has arrived (:36), k_chunk_idx_start (:37))}}, idx ascending (:50-51)."""
    plan = {}
    for dev in range(n):
        steps = {}
        for idx in range(n):
            k_blk = (dev - idx) % n
            k_start = k_blk * (kv_len // cfg.kc)
            q_start = _q_start(cfg, mi, dev, q_len)
            if _step_runs(cfg, mi, q_start, q_len, k_start, kv_len):
                steps[idx] = (q_start, k_blk, k_start)
        plan[dev] = steps
    return plan


def _ring_step_launches(cfg, mi, n):
    """Whether a scan step of all devices may go out as one launch per kernel (ra_attn_*_ring_step): a ring of 2 to
    64 devices, the MFMA kernels, no boolean / dropout mask, no cache_idx.  blockwise_kwargs["ring_launch"] =
    "device" keeps one launch per device."""
    return (1 < n <= 64 and cfg.ring_launch != "device" and cfg.impl in (L.RA_IMPL_AUTO, L.RA_IMPL_MFMA) and cfg.pdrop == 0.0
            and mi.keep is None and mi.keep_packed is None and mi.cache_idx_host is None and mi.cache_idx_dev is None)


def _ring_bits(devs):
    bits = 0
    for d in devs:
        bits |= 1 << d
    return bits


def _fwd_ring_step(q, k, v, carry, out, out32, cfg, mi, n, idx, plan, devs):
    """Scan step idx of every device in `devs` as one launch; False when the shape does not fit the MFMA kernels
    (nothing was launched then)."""
    num, den, mx = carry
    B, q_total, H, D = q.shape
    p = L.RaAttnFwdParams()
    p.q, p.k, p.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    p.dtype = _ra_dtype(q)
    p.B, p.Sq, p.Skv, p.H, p.D = B, q_total, k.shape[1], H, D
    p.q_stride_b, p.q_stride_s = _rows(q)
    p.kv_stride_b, p.kv_stride_s = _rows(k)
    if _rows(v) != _rows(k):
        raise ValueError("k and v must share strides")
    if num is not None:
        p.numerator = num.data_ptr()
        p.num_stride_b, p.num_stride_s = _rows(num)
    else:
        p.num_stride_b, p.num_stride_s = q_total * H * D, H * D
    p.out = out.data_ptr()
    p.out_stride_b, p.out_stride_s = _rows(out)
    if out32 is not None:
        p.out_f32 = out32.data_ptr()
    p.denominator, p.max_score = den.data_ptr(), mx.data_ptr()
    p.stat_stride_b, p.stat_stride_h = den.stride(0), den.stride(1)
    p.mask = mi.fill(cfg, 0, 0, cfg.skip_masked_tiles)
    p.impl = cfg.impl
    p.logit_dim = cfg.logit_dim
    r = L.RaRingStep()
    r.n_dev, r.idx = n, idx
    r.run = _ring_bits(devs)
    r.first = _ring_bits(d for d in devs if idx == min(plan[d]))
    r.last = _ring_bits(d for d in devs if idx == max(plan[d]))
    rc = L.load().ra_attn_fwd_ring_step(ctypes.byref(p), ctypes.byref(r), _stream())
    if rc == L.RA_ERR_UNSUPPORTED and cfg.impl == L.RA_IMPL_AUTO:
        return False
    L.check(rc, "ra_attn_fwd_ring_step")
    _LAST_FAMILY["forward"] = "mfma_bf16"
    return True


def _ring_attention_bwd(res, g):
    """ringattention_jax.py:55-90 for every device of the virtual ring; returns dq, dk, dv in the
    primal dtype (accumulated in fp32)."""
    out, q, k, v, mi, cfg, n, den, mx = res
    B, q_total, H, D = q.shape
    kv_total = k.shape[1]
    q_len, kv_len = q_total // n, kv_total // n
    d_true = g.shape[3]
    if d_true != D:             # q, k, v were zero-padded along D in the forward pass: the cotangent follows
        g = torch.nn.functional.pad(g, (0, D - d_true))
    g = g.to(q.dtype).contiguous()
    delta = _bwd_delta(g, out)
    plan = _ring_plan(cfg, mi, n, q_len, kv_len)
    # the scan steps that add into each K/V shard's dk, dv (they ride with the shard, :85-86): shard s is with
    # device (s + idx) mod n in step idx
    shard_steps = {s: [idx for idx in range(n) if idx in plan[(s + idx) % n]] for s in range(n)}
    # fp32 accumulators (:61-63) exist only where more than one call adds into a gradient: the first call starts
    # them (nothing is read, so no zero fill), the last one writes the sum in the primal dtype (:89)
    dq_out = torch.empty((B, q_total, H, D), dtype=q.dtype, device=q.device)
    dk_out = torch.empty((B, kv_total, H, D), dtype=k.dtype, device=q.device)
    dv_out = torch.empty((B, kv_total, H, D), dtype=v.dtype, device=q.device)
    dq = dk = dv = None
    if any(len(steps) > 1 for steps in plan.values()):
        dq = torch.empty((B, q_total, H, D), dtype=torch.float32, device=q.device)
    if any(len(steps) > 1 for steps in shard_steps.values()):
        dk = torch.empty((B, kv_total, H, D), dtype=torch.float32, device=q.device)
        dv = torch.empty((B, kv_total, H, D), dtype=torch.float32, device=q.device)
    whole = _ring_step_launches(cfg, mi, n) and q.dtype == torch.bfloat16      # those entry points take bf16 only
    for idx in range(n):                    # the scan of :65-88
        devs = [dev for dev in range(n) if idx in plan[dev]]
        if whole and devs:
            whole = _bwd_ring_step(q, k, v, g, delta, den, mx, (dq, dk, dv), (dq_out, dk_out, dv_out), cfg, mi, n,
                                   idx, plan, shard_steps, devs)
            if whole:
                continue
        for dev in devs:
            qs = slice(dev * q_len, (dev + 1) * q_len)
            q_start, k_blk, k_start = plan[dev][idx]
            ks = slice(k_blk * kv_len, (k_blk + 1) * kv_len)
            initial = (L.RA_GRAD_INIT_DQ if idx == min(plan[dev]) else 0) | (
                L.RA_GRAD_INIT_DKV if idx == shard_steps[k_blk][0] else 0)
            last_dq = idx == max(plan[dev])
            last_dkv = idx == shard_steps[k_blk][-1]
            _blockwise_attention_bwd(q[:, qs], k[:, ks], v[:, ks], g[:, qs],
                                     (dq[:, qs] if dq is not None else None, dk[:, ks] if dk is not None else None,
                                      dv[:, ks] if dv is not None else None, out[:, qs], den[:, :, qs], mx[:, :, qs]),
                                     q_start, k_start, None, None, cfg.cbs, cfg.qc, cfg.kc,
                                     _mask_inputs=mi, _cfg=cfg, _delta=delta[:, :, qs], _grads_initial=initial,
                                     _dq_out=dq_out[:, qs] if last_dq else None,
                                     _dkv_out=(dk_out[:, ks], dv_out[:, ks]) if last_dkv else None)
    for dev in range(n):
        if not plan[dev]:
            dq_out[:, dev * q_len:(dev + 1) * q_len].zero_()
    for s in range(n):
        if not shard_steps[s]:
            ks = slice(s * kv_len, (s + 1) * kv_len)
            dk_out[:, ks].zero_()
            dv_out[:, ks].zero_()
    if d_true != D:
        dq_out, dk_out, dv_out = (t[..., :d_true].contiguous() for t in (dq_out, dk_out, dv_out))
    return dq_out, dk_out, dv_out


def _bwd_ring_step(q, k, v, g, delta, den, mx, acc, outs, cfg, mi, n, idx, plan, shard_steps, devs):
    """Scan step idx of the backward pass of every device in `devs` as one launch per kernel; False when the shape
    does not fit the MFMA kernels (nothing was launched then)."""
    dq, dk, dv = acc
    dq_out, dk_out, dv_out = outs
    B, q_total, H, D = q.shape
    kv_total = k.shape[1]
    if _rows(g) != _rows(q):
        raise ValueError("g must share q's strides")
    p = L.RaAttnBwdParams()
    p.q, p.k, p.v, p.g = q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr()
    p.dtype = _ra_dtype(q)
    p.B, p.Sq, p.Skv, p.H, p.D = B, q_total, kv_total, H, D
    p.q_stride_b, p.q_stride_s = _rows(q)
    p.kv_stride_b, p.kv_stride_s = _rows(k)
    p.delta, p.denominator, p.max_score = delta.data_ptr(), den.data_ptr(), mx.data_ptr()
    if not (delta.stride() == den.stride() == mx.stride()):
        raise ValueError("delta / denominator / max_score must share strides")
    p.stat_stride_b, p.stat_stride_h = den.stride(0), den.stride(1)
    if dq is not None:
        p.dq = dq.data_ptr()
        p.dq_stride_b, p.dq_stride_s = _rows(dq)
    else:
        p.dq_stride_b, p.dq_stride_s = q_total * H * D, H * D
    if dk is not None:
        p.dk, p.dv = dk.data_ptr(), dv.data_ptr()
        p.dkv_stride_b, p.dkv_stride_s = _rows(dk)
    else:
        p.dkv_stride_b, p.dkv_stride_s = kv_total * H * D, H * D
    p.dq_out = dq_out.data_ptr()
    p.dq_out_stride_b, p.dq_out_stride_s = _rows(dq_out)
    p.dk_out, p.dv_out = dk_out.data_ptr(), dv_out.data_ptr()
    p.dkv_out_stride_b, p.dkv_out_stride_s = _rows(dk_out)
    p.mask = mi.fill(cfg, 0, 0, cfg.skip_masked_tiles)
    p.impl = cfg.impl
    p.logit_dim = cfg.logit_dim
    r = L.RaRingStep()
    r.n_dev, r.idx = n, idx
    r.run = _ring_bits(devs)
    r.first = _ring_bits(d for d in devs if idx == min(plan[d]))
    r.last = _ring_bits(d for d in devs if idx == max(plan[d]))
    shards = [(d - idx) % n for d in devs]
    r.kv_first = _ring_bits(s for s in shards if idx == shard_steps[s][0])
    r.kv_last = _ring_bits(s for s in shards if idx == shard_steps[s][-1])
    if cfg.bwd_only:      # measurement hook: one of the two kernels alone
        rc = L.load().ra_attn_bwd_ring_step_part(ctypes.byref(p), ctypes.byref(r), cfg.bwd_only, _stream())
    else:
        rc = L.load().ra_attn_bwd_ring_step(ctypes.byref(p), ctypes.byref(r), _stream())
    if rc == L.RA_ERR_UNSUPPORTED and cfg.impl == L.RA_IMPL_AUTO:
        return False
    L.check(rc, "ra_attn_bwd_ring_step")
    _LAST_FAMILY["backward"] = "mfma_bf16"
    return True


class _RingAttentionFn(torch.autograd.Function):
    """custom_vjp of ringattention_jax.py:92-97: cotangents for q, k, v only (:90)."""

    @staticmethod
    def forward(ctx, q, k, v, attn_bias, segment_ids, cache_idx, axis_name, float32_logits, blockwise_kwargs):
        out, res = _ring_attention_fwd(q, k, v, attn_bias, segment_ids, cache_idx, axis_name, float32_logits,
                                       blockwise_kwargs)
        _save_residuals(ctx, res)
        return out

    @staticmethod
    def backward(ctx, g):
        dq, dk, dv = _ring_attention_bwd(_saved_residuals(ctx), g)
        return dq, dk, dv, None, None, None, None, None, None


def _save_residuals(ctx, res):
    """The tensors of the residuals (:53) go through save_for_backward - autograd then checks that none was edited
    in place before the backward pass, frees them with the graph, and `out -> grad_fn -> ctx -> out` is no reference
    cycle; the mask inputs and the configuration are plain attributes."""
    out, q, k, v, mi, cfg, n, den, mx = res
    ctx.save_for_backward(out, q, k, v, den, mx)
    ctx.ra_extra = (mi, cfg, n)


def _saved_residuals(ctx):
    out, q, k, v, den, mx = ctx.saved_tensors
    mi, cfg, n = ctx.ra_extra
    return out, q, k, v, mi, cfg, n, den, mx


_DECODE_HEAD_SIZES = (32, 40, 64, 80, 96, 112, 128, 160, 192, 256)     # what decode_split_kernel is instantiated for


def _pad_lengths_to_mfma_grid(q, k, v, attn_bias, segment_ids, cache_idx, n, axis_name, float32_logits,
                              blockwise_kwargs, grid=128):
    """One device, equal query and key lengths that are no multiple of 128 (a prompt of 5000 tokens in chunks of
    500): the matrix-core kernels tile 128 positions, so such a call would take the vector kernels, a few hundred times
    slower.  Where the chunking cannot change the result (the conditions of _fit_chunks_to_mfma_grid) the call is
    made on arrays padded to the next multiple of 128 instead, in chunks of 128, and the result cut back:
    the padded keys are masked for every real row - they lie behind it under a causal mask, and carry a segment id
    of their own otherwise - so each real row sums over exactly its own pairs, and the padded rows, whose output is
    dropped, get no cotangent.  Returns the result, or None when the call is left as it is."""
    kw = dict(blockwise_kwargs)
    B, S, H, D = q.shape
    if n != 1 or cache_idx is not None or k.shape[1] != S or S % grid == 0 or D > 128:
        return None
    if q.dtype not in (torch.bfloat16, torch.float32) or kw.get("impl", "auto") in ("generic", "mfma_any"):
        return None
    if kw.get("skip_masked_tiles", None) is False or kw.get("_padded", False):
        return None
    if (not kw.get("deterministic", True)) and float(kw.get("attn_pdrop", 0.0)) > 0.0:
        return None                    # the dropout mask is drawn for the shape of the call
    qc, kc, cbs = int(kw["query_chunk_size"]), int(kw["key_chunk_size"]), kw.get("causal_block_size", None)
    if S % qc or S % kc:
        return None                    # refused further down, with the reference's message
    if cbs is not None:
        cbs = int(cbs)
        if (cbs == 1 and (qc % 2 or kc % 2)) or (cbs > 1 and (qc % cbs or kc % cbs or grid % cbs)):
            return None
    if attn_bias is not None and (attn_bias.dim() != 4 or attn_bias.shape[2] != 1 or attn_bias.shape[3] != S):
        return None
    if segment_ids is not None and (segment_ids.dim() != 2 or segment_ids.shape[1] != S):
        return None
    if cbs is None and segment_ids is None and attn_bias is not None:
        return None                    # the segment ids added below would switch the clamp of the bias on (:299)
    pad = grid - S % grid
    qp, kp, vp = (torch.nn.functional.pad(t, (0, 0, 0, 0, 0, pad)) for t in (q, k, v))
    bias_p = None if attn_bias is None else torch.nn.functional.pad(attn_bias.detach(), (0, pad))
    seg_p = segment_ids
    if cbs is None or segment_ids is not None:
        # without a causal mask only a segment id of their own keeps the padded keys away from the real rows
        ids = segment_ids.detach().to(torch.int32) if segment_ids is not None else \
            torch.zeros((1, S), dtype=torch.int32, device=q.device)
        own = (ids.max() + 1).reshape(1, 1).expand(ids.shape[0], pad)
        seg_p = torch.cat((ids, own), dim=1)
    kw.update(query_chunk_size=grid, key_chunk_size=grid, skip_masked_tiles=True, _padded=True)
    out = ring_attention(qp, kp, vp, bias_p, seg_p, None, axis_name, float32_logits, kw)
    return out[:, :S].contiguous()


def ring_attention(q, k, v, attn_bias, segment_ids, cache_idx, axis_name, float32_logits, blockwise_kwargs):
    """Drop-in for ringattention_jax.py:92-97 (exported as ``ringattention``).

    q, k, v: (B, S, H, D) device tensors, bf16, fp32 or fp16 (computed on fp32 copies); with a declared ring axis they are the global
    arrays and the sequence axis is split over the virtual devices.  attn_bias (B|1, H|1, 1, K_total)
    and segment_ids (B|1, S_total) are global / replicated, as in the reference's shard_map specs.
    One query token with cache_idx set takes the streaming decode kernel."""
    # (a head size the streaming kernel is not built for takes the blockwise kernels below, like a call that wants
    # gradients)
    _check_qkv(q, k, v)
    if q.dtype == torch.float16 and k.dtype == torch.float16 and v.dtype == torch.float16:
        # float16 inputs: with float32_logits the reference casts q and k to fp32 (:18-19) and the products with v
        # promote to fp32 as well, so computing on exact fp32 copies (the fp32 matrix-core kernels) and rounding the
        # output - and, through autograd, the gradients - to float16 is its arithmetic; twice the memory of a native
        # float16 path, which the kernels do not have
        out = ring_attention(q.float(), k.float(), v.float(), attn_bias, segment_ids, cache_idx, axis_name,
                             float32_logits, blockwise_kwargs)
        return out.to(torch.float16)
    if q.numel() == 0 or k.numel() == 0:
        # nothing to launch: an empty result, or - queries without a single key - the 0 / 0 of :52; the product
        # with zero keeps the result attached to its inputs for autograd
        _check_qkv(q, k, v)
        fill = float("nan") if q.numel() else 0.0
        return torch.full_like(q, fill) + 0.0 * (q.sum() + k.sum() + v.sum()).to(q.dtype)
    n = axis_size(axis_name)
    padded = _pad_lengths_to_mfma_grid(q, k, v, attn_bias, segment_ids, cache_idx, n, axis_name, float32_logits,
                                       blockwise_kwargs)
    if padded is not None:
        return padded
    if cache_idx is not None and q.shape[1] == n and q.shape[3] in _DECODE_HEAD_SIZES and not (
            torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)) \
            and int(dict(blockwise_kwargs)["query_chunk_size"]) == 1:
        from .decode import decode_attention, decode_attention_ring
        if n == 1:
            return decode_attention(q, k, v, attn_bias, segment_ids, cache_idx, blockwise_kwargs)
        # one query token per virtual device and the cache sharded over the ring: every shard is streamed with
        # the split kernel and merged into the device's carry
        if k.shape[1] % n == 0 and (k.shape[1] // n) % int(dict(blockwise_kwargs)["key_chunk_size"]) == 0:
            return decode_attention_ring(q, k, v, attn_bias, segment_ids, cache_idx, blockwise_kwargs, n)
    return _RingAttentionFn.apply(q, k, v, attn_bias, segment_ids, cache_idx, axis_name, float32_logits,
                                  blockwise_kwargs)
