"""ctypes binding of libringattn_hip.so (the C-ABI declared in include/ringattn_hip.h).

The library is the only compute path: loading fails loudly when it has not been built, and
nothing here falls back to torch ops.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libringattn_hip.so")

RA_ABI_VERSION = 2          # include/ringattn_hip.h; load() refuses a library built for another one
RA_OK, RA_ERR_INVALID, RA_ERR_UNSUPPORTED, RA_ERR_LAUNCH = 0, 1, 2, 3
RA_F32, RA_BF16 = 0, 1
RA_IMPL_AUTO, RA_IMPL_GENERIC, RA_IMPL_MFMA, RA_IMPL_MFMA_ANY = 0, 1, 2, 3
RA_BWD_PART_DQ, RA_BWD_PART_DKV = 1, 2          # include/ringattn_hip_measure.h
RA_DECODE_STATIC_SCRATCH_BYTES = 16 * 1024 * 1024
RA_SEG_TILE = 64
RA_KEEP_WHERE, RA_KEEP_DROPOUT = 0, 1
RA_GRAD_INIT_DQ, RA_GRAD_INIT_DKV = 1, 2
RA_FAMILY_GENERIC, RA_FAMILY_MFMA_BF16, RA_FAMILY_MFMA_F32, RA_FAMILY_MFMA_BF16_ANY = 1, 2, 3, 4

i32, i64, f32, vp = C.c_int32, C.c_int64, C.c_float, C.c_void_p


class RaMask(C.Structure):
    _fields_ = [
        ("bias", vp), ("bias_stride_b", i64), ("bias_stride_h", i64), ("bias_stride_q", i64),
        ("bias_stride_k", i64), ("segment_ids", vp), ("seg_stride_b", i64), ("seg_len", i32),
        ("causal_block_size", i32), ("query_chunk_size", i32), ("key_chunk_size", i32),
        ("q_chunk_idx_start", i32), ("k_chunk_idx_start", i32), ("cache_idx", vp), ("chunk_starts", vp),
        ("mask_min", f32),
        ("skip_masked_tiles", i32), ("seg_tile_minmax", vp), ("seg_tiles", i32),
        ("seg_run_hulls", vp), ("seg_runs", i32),
        ("keep", vp), ("keep_stride_b", i64), ("keep_stride_h", i64), ("keep_stride_q", i64),
        ("keep_stride_k", i64),
        ("keep_bits_k", vp), ("keep_bits_q", vp), ("keep_summary", vp),
        ("keep_pack_stride_b", i64), ("keep_pack_stride_h", i64), ("keep_sum_stride_b", i64),
        ("keep_sum_stride_h", i64), ("keep_q_total", i32), ("keep_k_total", i32), ("keep_q0", i32),
        ("keep_k0", i32), ("keep_mode", i32),
    ]


class RaAttnFwdParams(C.Structure):
    _fields_ = [
        ("q", vp), ("k", vp), ("v", vp), ("dtype", i32),
        ("B", i32), ("Sq", i32), ("Skv", i32), ("H", i32), ("D", i32),
        ("q_stride_b", i64), ("q_stride_s", i64), ("kv_stride_b", i64), ("kv_stride_s", i64),
        ("numerator", vp), ("num_stride_b", i64), ("num_stride_s", i64),
        ("denominator", vp), ("max_score", vp), ("stat_stride_b", i64), ("stat_stride_h", i64),
        ("mask", RaMask), ("impl", i32), ("carry_is_initial", i32),
        ("out", vp), ("out_stride_b", i64), ("out_stride_s", i64), ("logit_dim", i32), ("out_f32", vp),
    ]


class RaAttnBwdParams(C.Structure):
    _fields_ = [
        ("q", vp), ("k", vp), ("v", vp), ("g", vp), ("dtype", i32),
        ("B", i32), ("Sq", i32), ("Skv", i32), ("H", i32), ("D", i32),
        ("q_stride_b", i64), ("q_stride_s", i64), ("kv_stride_b", i64), ("kv_stride_s", i64),
        ("delta", vp), ("denominator", vp), ("max_score", vp), ("stat_stride_b", i64), ("stat_stride_h", i64),
        ("dq", vp), ("dq_stride_b", i64), ("dq_stride_s", i64),
        ("dk", vp), ("dv", vp), ("dkv_stride_b", i64), ("dkv_stride_s", i64),
        ("mask", RaMask), ("impl", i32), ("grads_are_initial", i32),
        ("dq_out", vp), ("dq_out_stride_b", i64), ("dq_out_stride_s", i64),
        ("dk_out", vp), ("dv_out", vp), ("dkv_out_stride_b", i64), ("dkv_out_stride_s", i64), ("logit_dim", i32),
    ]


class RaRingStep(C.Structure):
    _fields_ = [
        ("n_dev", i32), ("idx", i32), ("run", C.c_uint64), ("first", C.c_uint64), ("last", C.c_uint64),
        ("kv_first", C.c_uint64), ("kv_last", C.c_uint64),
    ]


class RaDecodeParams(C.Structure):
    _fields_ = [
        ("q", vp), ("k", vp), ("v", vp), ("out", vp), ("dtype", i32),
        ("B", i32), ("L", i32), ("H", i32), ("D", i32),
        ("q_stride_b", i64), ("kv_stride_b", i64), ("kv_stride_s", i64), ("out_stride_b", i64),
        ("mask", RaMask), ("workspace", vp), ("workspace_bytes", C.c_size_t), ("num_splits", i32),
        ("carry_numerator", vp), ("carry_denominator", vp), ("carry_max_score", vp),
        ("carry_num_stride_b", i64), ("carry_stat_stride_b", i64), ("carry_is_initial", i32),
    ]


class RaSwigluParams(C.Structure):
    _fields_ = [
        ("T", i32), ("d", i32), ("f", i32),
        ("x", vp), ("w1", vp), ("w2", vp), ("w3", vp),
        ("a", vp), ("b", vp), ("h", vp), ("y", vp),
        ("dy", vp), ("dx", vp), ("dw1", vp), ("dw2", vp), ("dw3", vp), ("da", vp), ("db", vp),
        ("preact_saved", i32), ("defer_weight_grads", i32), ("gemm_tile", i32),
    ]


class RaRopeAppendParams(C.Structure):
    _fields_ = [
        ("q", vp), ("q_out", vp), ("k_new", vp), ("v_new", vp), ("k_cache", vp), ("v_cache", vp),
        ("cache_idx", vp), ("cache_idx_host", i32), ("dtype", i32),
        ("B", i32), ("L", i32), ("H", i32), ("D", i32),
        ("q_stride_b", i64), ("q_out_stride_b", i64), ("new_stride_b", i64), ("cache_stride_b", i64),
        ("cache_stride_s", i64), ("rope_theta", f32), ("rope_style", i32),
    ]


class RaRmsnormParams(C.Structure):
    _fields_ = [
        ("T", i64), ("d", i32), ("eps", f32),
        ("x", vp), ("residual", vp), ("weight", vp),
        ("y", vp), ("normed", vp), ("rstd", vp),
        ("d_normed", vp), ("d_residual", vp),
        ("d_y", vp), ("d_weight", vp), ("dw_workspace", vp), ("dw_workspace_bytes", C.c_size_t),
    ]


# every symbol include/ringattn_hip.h and include/ringattn_hip_measure.h declare: (name, restype, argtypes)
SYMBOLS = {
    "ra_segment_tile_ranges": (C.c_int, [vp, i64, i32, i32, vp, vp]),
    "ra_segment_run_hulls": (C.c_int, [vp, i32, i32, vp, vp]),
    "ra_keep_pack": (C.c_int, [vp, i64, i64, i64, i64, i32, i32, i32, i32, vp, vp, vp, vp]),
    "ra_dropout_keep": (C.c_int, [C.c_uint64, f32, i32, i32, i32, i32, vp, vp]),
    "ra_dropout_keep_packed": (C.c_int, [C.c_uint64, f32, i32, i32, i32, i32, vp, vp, vp, i32, i32, i32, i32, i32, vp]),
    "ra_attn_carry_init": (C.c_int, [vp, i64, i64, vp, vp, i64, i64, i32, i32, i32, i32, vp]),
    "ra_attn_fwd_block": (C.c_int, [C.POINTER(RaAttnFwdParams), vp]),
    "ra_attn_fwd_family": (C.c_int, [C.POINTER(RaAttnFwdParams)]),
    "ra_attn_bwd_family": (C.c_int, [C.POINTER(RaAttnBwdParams)]),
    "ra_attn_finalize": (C.c_int, [vp, i64, i64, vp, i64, i64, vp, i32, i64, i64, i32, i32, i32, i32, vp]),
    "ra_attn_bwd_delta": (C.c_int, [vp, vp, i32, i32, i64, i64, vp, i64, i64, i32, i32, i32, i32, vp]),
    "ra_attn_bwd_block": (C.c_int, [C.POINTER(RaAttnBwdParams), vp]),
    "ra_attn_fwd_ring_step": (C.c_int, [C.POINTER(RaAttnFwdParams), C.POINTER(RaRingStep), vp]),
    "ra_attn_bwd_ring_step": (C.c_int, [C.POINTER(RaAttnBwdParams), C.POINTER(RaRingStep), vp]),
    "ra_decode_workspace_bytes": (C.c_size_t, [i32, i32, i32, i32, i32]),
    "ra_decode_auto_splits": (C.c_int, [i32, i32, i32, i32, i32]),
    "ra_decode_fwd": (C.c_int, [C.POINTER(RaDecodeParams), vp]),
    "ra_decode_fwd_static": (C.c_int, [C.POINTER(RaDecodeParams), vp]),
    "ra_swiglu_fwd": (C.c_int, [C.POINTER(RaSwigluParams), vp]),
    "ra_swiglu_bwd": (C.c_int, [C.POINTER(RaSwigluParams), vp]),
    "ra_swiglu_weight_grads": (C.c_int, [C.POINTER(RaSwigluParams), vp]),
    "ra_gemm_bf16": (C.c_int, [vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, vp]),
    "ra_rope_kv_append": (C.c_int, [C.POINTER(RaRopeAppendParams), vp]),
    "ra_rmsnorm_workspace_bytes": (C.c_size_t, [i64, i32]),
    "ra_rmsnorm_fwd": (C.c_int, [C.POINTER(RaRmsnormParams), vp]),
    "ra_rmsnorm_bwd": (C.c_int, [C.POINTER(RaRmsnormParams), vp]),
    "ra_last_error": (C.c_char_p, []),
    "ra_version": (C.c_int, []),
    # measurement / test hooks
    "ra_attn_bwd_block_part": (C.c_int, [C.POINTER(RaAttnBwdParams), i32, vp]),
    "ra_attn_bwd_ring_step_part": (C.c_int, [C.POINTER(RaAttnBwdParams), C.POINTER(RaRingStep), i32, vp]),
    "ra_gemm_bf16_pair": (C.c_int, [vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]),
    "ra_gemm_bf16_tile": (C.c_int, [vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, i32, vp]),
}
# libringattn_probe.so: the MFMA rate probe of the benchmark, kept out of the product library
PROBE_LIB_PATH = os.path.join(_HERE, "libringattn_probe.so")
PROBE_SYMBOLS = {
    "ra_mfma_rate_probe": (C.c_int, [vp, i32, i32, i32, vp]),
}
_probe = None


def load_probe():
    """The measurement library (ringattn_hip_measure.h: ra_mfma_rate_probe); raises if it has not been built."""
    global _probe
    if _probe is None:
        if not os.path.exists(PROBE_LIB_PATH):
            raise RuntimeError("ringattention_amd: %s is missing. Build it with `python -m ringattention_amd.build`."
                               % PROBE_LIB_PATH)
        lib = C.CDLL(PROBE_LIB_PATH)
        for name, (res, args) in PROBE_SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _probe = lib
    return _probe

_lib = None


def load():
    """Load the shared library once; raise if it is missing (there is no fallback path)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "ringattention_amd: %s is missing. Build it with `python -m ringattention_amd.build` "
            "(hipcc, gfx950); there is no non-HIP fallback." % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.ra_version() != RA_ABI_VERSION:
        raise RuntimeError("ringattention_amd: %s speaks interface version %d, this binding version %d; rebuild it "
                           "with `python -m ringattention_amd.build`" % (LIB_PATH, lib.ra_version(), RA_ABI_VERSION))
    _lib = lib
    return lib


def check(rc, what):
    if rc == RA_OK:
        return
    msg = load().ra_last_error().decode()
    if rc == RA_ERR_UNSUPPORTED:
        raise NotImplementedError("%s: %s" % (what, msg))
    if rc == RA_ERR_INVALID:
        raise ValueError("%s: %s" % (what, msg))
    raise RuntimeError("%s: %s (code %d)" % (what, msg, rc))
