"""CPU tests of the host side: the C-ABI library loads and exports every declared symbol, the
closed-form run prefix equals the reference predicate, argument checking raises like the reference."""
import os
import re

import pytest
import torch

import ringattention_amd as ra
from ringattention_amd import _lib
from oracle import ringattention_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    declared = set()
    for name in ("ringattn_hip.h", "ringattn_hip_measure.h"):
        header = open(os.path.join(ROOT, "include", name)).read()
        header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
        declared |= set(re.findall(r"\b(ra_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations parsed"
    assert declared == set(_lib.SYMBOLS) | set(_lib.PROBE_SYMBOLS), declared ^ (set(_lib.SYMBOLS) | set(_lib.PROBE_SYMBOLS))
    lib, probe = _lib.load(), _lib.load_probe()
    for name in declared:
        assert getattr(probe if name in _lib.PROBE_SYMBOLS else lib, name) is not None
    with pytest.raises(AttributeError):           # the probe is measurement code: not in the product library
        lib.ra_mfma_rate_probe
    macro = int(re.search(r"#define\s+RA_ABI_VERSION\s+(\d+)", open(os.path.join(ROOT, "include", "ringattn_hip.h")).read()).group(1))
    assert lib.ra_version() == macro == _lib.RA_ABI_VERSION


def test_struct_sizes_match_a_c_compiler(tmp_path):
    import ctypes
    import subprocess
    src = tmp_path / "sz.c"
    src.write_text('#include <stdio.h>\n#include "%s"\nint main(){printf("%%zu %%zu %%zu %%zu %%zu %%zu %%zu %%zu\\n",'
                   'sizeof(ra_mask),sizeof(ra_attn_fwd_params),sizeof(ra_attn_bwd_params),'
                   'sizeof(ra_decode_params),sizeof(ra_swiglu_params),sizeof(ra_rope_append_params),'
                   'sizeof(ra_rmsnorm_params),sizeof(ra_ring_step));return 0;}\n'
                   % os.path.join(ROOT, "include", "ringattn_hip.h"))
    exe = tmp_path / "sz"
    subprocess.check_call(["gcc", str(src), "-o", str(exe)])
    sizes = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    mine = [ctypes.sizeof(c) for c in (_lib.RaMask, _lib.RaAttnFwdParams, _lib.RaAttnBwdParams,
                                       _lib.RaDecodeParams, _lib.RaSwigluParams, _lib.RaRopeAppendParams,
                                       _lib.RaRmsnormParams, _lib.RaRingStep)]
    assert sizes == mine


@pytest.mark.parametrize("qc,kc,cbs", [(1, 1, 1), (1, 8, 1), (2, 2, 1), (4, 8, 1), (8, 4, 1), (4, 4, 8),
                                       (4, 4, 2), (2, 8, 4), (8, 2, 16), (3, 5, 1), (512, 512, 1)])
def test_run_prefix_equals_predicate(qc, kc, cbs):
    nkv = 12
    for k_start in (0, 3, 7):
        for r in range(0, 20):
            runs = [bool(O.below_or_on_diag(r, qc, k_start + c, kc, cbs)) for c in range(nkv)]
            # monotone: a prefix of the key chunks runs
            n_run = sum(runs)
            assert runs == [True] * n_run + [False] * (nkv - n_run)
            assert ra.run_prefix_keys(r, qc, kc, cbs, k_start, nkv * kc) == n_run * kc
            assert bool(ra.below_or_on_diag(r, qc, k_start, kc, cbs)) == runs[0]


def test_ring_axis_registry():
    assert ra.axis_size("sp") == 1
    with ra.ring_axis("sp", 8):
        assert ra.axis_size("sp") == 8
        with ra.ring_axis("sp", 2):
            assert ra.axis_size("sp") == 2
        assert ra.axis_size("sp") == 8
    assert ra.axis_size("sp") == 1
    assert ra.axis_size(None) == 1


def test_cpu_tensors_are_refused():
    q = torch.zeros(1, 8, 1, 64)
    kw = dict(causal_block_size=1, query_chunk_size=4, key_chunk_size=4, dtype=torch.float32)
    with pytest.raises(RuntimeError):
        ra.ringattention(q, q, q, None, None, None, "sp", True, kw)


def test_dropout_configuration():
    from ringattention_amd.ringattention_hip import _Config
    base = dict(causal_block_size=1, query_chunk_size=4, key_chunk_size=4, dtype=torch.float32)
    cfg = _Config(dict(base, deterministic=False, attn_pdrop=0.1, dropout_rng=(1 << 40) + 3))
    assert cfg.pdrop == 0.1 and cfg.seed == (1 << 40) + 3
    assert _Config(dict(base, deterministic=True, attn_pdrop=0.1)).pdrop == 0.0        # :119: both conditions
    assert _Config(dict(base, deterministic=False, attn_pdrop=0.0)).pdrop == 0.0
    with pytest.raises(ValueError):
        _Config(dict(base, deterministic=False, attn_pdrop=0.1))                         # no dropout_rng
    with pytest.raises(ValueError):
        _Config(dict(base, deterministic=False, attn_pdrop=1.0, dropout_rng=0))


def test_invalid_arguments_return_codes_without_gpu():
    import ctypes
    lib = _lib.load()
    assert lib.ra_attn_fwd_block(None, None) == _lib.RA_ERR_INVALID
    assert b"null" in lib.ra_last_error()
    p = _lib.RaAttnFwdParams()
    assert lib.ra_attn_fwd_block(ctypes.byref(p), None) == _lib.RA_ERR_INVALID
    assert lib.ra_decode_fwd(None, None) == _lib.RA_ERR_INVALID
    assert lib.ra_decode_workspace_bytes(16, 1024, 32, 128, 4) == 16 * 32 * 4 * 130 * 4
    # the entry point that allocates nothing refuses what its built-in buffer cannot hold, before any device call
    assert lib.ra_decode_fwd_static(None, None) == _lib.RA_ERR_INVALID
    d = _lib.RaDecodeParams()
    d.q = d.k = d.v = d.out = 16
    d.dtype, d.B, d.L, d.H, d.D = _lib.RA_BF16, 1024, 512, 64, 128       # 1024 * 64 * 130 * 4 bytes > 16 MiB
    d.mask.query_chunk_size, d.mask.key_chunk_size = 1, 512
    assert lib.ra_decode_fwd_static(ctypes.byref(d), None) == _lib.RA_ERR_UNSUPPORTED
    assert b"scratch" in lib.ra_last_error()
    d.D = 96
    assert lib.ra_decode_fwd_static(ctypes.byref(d), None) == _lib.RA_ERR_UNSUPPORTED
    # measurement hooks validate too
    assert lib.ra_attn_bwd_block_part(None, 3, None) == _lib.RA_ERR_INVALID
    assert lib.ra_gemm_bf16_tile(one_ := ctypes.c_void_p(16), one_, one_, 128, 128, 64, 0, 0, 1, 0, 7, None) == _lib.RA_ERR_INVALID
    assert _lib.load_probe().ra_mfma_rate_probe(None, 1, 1, 0, None) == _lib.RA_ERR_INVALID
    assert _lib.load_probe().ra_mfma_rate_probe(ctypes.c_void_p(16), 1, 1, 3, None) == _lib.RA_ERR_INVALID
    # ra_keep_pack validates before touching the device
    assert lib.ra_keep_pack(None, 0, 0, 0, 1, 1, 1, 64, 64, None, None, None, None) == _lib.RA_ERR_INVALID
    one = ctypes.c_void_p(16)      # any non-null address: the shape check comes before any use
    assert lib.ra_keep_pack(one, 0, 0, 100, 1, 1, 1, 100, 64, one, one, one, None) == _lib.RA_ERR_UNSUPPORTED
    assert b"multiples of 64" in lib.ra_last_error()
    # the steps either side of the path validate before launching too
    assert lib.ra_rope_kv_append(None, None) == _lib.RA_ERR_INVALID
    r = _lib.RaRopeAppendParams()
    r.q = r.q_out = r.k_new = r.v_new = r.k_cache = r.v_cache = 16
    r.dtype, r.B, r.L, r.H, r.D, r.cache_idx_host = _lib.RA_BF16, 1, 8, 2, 15, 0
    assert lib.ra_rope_kv_append(ctypes.byref(r), None) == _lib.RA_ERR_INVALID and b"even" in lib.ra_last_error()
    r.D, r.cache_idx_host = 16, 8
    assert lib.ra_rope_kv_append(ctypes.byref(r), None) == _lib.RA_ERR_INVALID and b"outside" in lib.ra_last_error()
    n = _lib.RaRmsnormParams()
    n.T, n.d = 4, 100
    assert lib.ra_rmsnorm_fwd(ctypes.byref(n), None) == _lib.RA_ERR_UNSUPPORTED
    assert lib.ra_rmsnorm_workspace_bytes(65536, 4096) == 4096 * 4096 * 4


# --- chunk sizes off the 128-grid: what _fit_chunks_to_mfma_grid relies on, by brute force against the predicate
@pytest.mark.parametrize("qc,kc,cbs", [(64, 64, 1), (192, 64, 1), (32, 96, 1), (96, 96, 1), (2, 6, 1), (64, 192, 32),
                                       (24, 8, 4), (128, 128, 1), (128, 128, 32)])
def test_a_chunk_pair_that_does_not_run_holds_masked_pairs_only(qc, kc, cbs):
    """Even chunk sizes under causal_block_size 1, or a block size that divides both: every causally allowed pair
    (q // cbs >= k // cbs) lies in a chunk pair that below_or_on_diag lets run, so two such chunkings sum over the
    same pairs."""
    S = 384
    for q in range(S):
        ks = torch.arange(0, S)
        allowed = (q // cbs) >= (ks // cbs)
        runs = torch.tensor([bool(O.below_or_on_diag(q // qc, qc, int(k) // kc, kc, cbs)) for k in range(0, S, kc)])
        runs = runs.repeat_interleave(kc)[:S]
        assert bool((runs | ~allowed).all()), (q, qc, kc, cbs)


def test_odd_chunk_sizes_can_drop_an_allowed_pair():
    """What keeps odd sizes away from the remapping: with query chunks of 3 and key chunks of 2 the causally allowed
    pair (q, k) = (2, 2) sits in key chunk 1 (keys 2-3), which does not run for query chunk 0 (rows 0-2): the
    predicate compares the last row with the first key strictly (ringattention_jax.py:331)."""
    assert not O.below_or_on_diag(0, 3, 1, 2, 1)
    assert 2 // 1 >= 2 // 1


class _FakeMaskInputs:
    cache_idx_host = cache_idx_dev = keep = bias = seg = None
    bias_strides = (0, 0, 0, 0)
    seg_len = 0


@pytest.mark.parametrize("qc,kc,cbs,skip,expect", [
    (64, 64, 1, True, 128), (192, 64, 1, True, 128), (3, 3, 1, True, 3), (64, 64, 1, False, 64),
    (384, 192, None, True, 128), (64, 192, 32, True, 128), (64, 192, 48, True, 64), (256, 256, 1, True, 256)])
def test_fit_chunks_to_mfma_grid_decisions(qc, kc, cbs, skip, expect):
    from ringattention_amd import ringattention_hip as rh
    for dtype in (torch.bfloat16, torch.float32):           # both matrix-core families tile on the same grid
        cfg = rh._Config(dict(query_chunk_size=qc, key_chunk_size=kc, causal_block_size=cbs))
        cfg.skip_masked_tiles = skip
        q = torch.zeros(1, 1, 1, 128, dtype=dtype)
        rh._fit_chunks_to_mfma_grid(cfg, _FakeMaskInputs(), q, 768, 768, 768, 768)
        assert cfg.qc == expect, (cfg.qc, cfg.kc)
        if expect == 128:
            assert cfg.kc == 128
    cfg = rh._Config(dict(query_chunk_size=qc, key_chunk_size=kc, causal_block_size=cbs))
    cfg.skip_masked_tiles = skip
    rh._fit_chunks_to_mfma_grid(cfg, _FakeMaskInputs(), torch.zeros(1, 1, 1, 256, dtype=torch.bfloat16), 768, 768, 768, 768)
    assert (cfg.qc, cfg.kc) == (qc, kc)                      # head size 256: the vector kernels, chunk sizes untouched
    # head sizes below 128 are zero-padded to 64 / 128 for the matrix-core kernels, so they re-chunk like those
    cfg = rh._Config(dict(query_chunk_size=qc, key_chunk_size=kc, causal_block_size=cbs))
    cfg.skip_masked_tiles = skip
    q32 = torch.zeros(1, 1, 1, 32, dtype=torch.bfloat16)
    rh._fit_chunks_to_mfma_grid(cfg, _FakeMaskInputs(), q32, 768, 768, 768, 768)
    assert cfg.qc == expect
    on_grid = cfg.qc % 128 == 0 and cfg.kc % 128 == 0
    # on the matrix-core grid 32 is padded to 64; off it a bf16 call takes the matrix-core kernels that evaluate the
    # mask element by element (head size 128 or 256), an fp32 call the vector kernels (they tile 32)
    assert rh._padded_head_size(cfg, _FakeMaskInputs(), q32) == (64 if on_grid else 128)
    assert rh._padded_head_size(cfg, _FakeMaskInputs(), q32.float()) == (64 if on_grid else 0)
    # 96 is tiled by no family: 128 either way; above 128 the element-wise and the vector kernels' 256
    assert rh._padded_head_size(cfg, _FakeMaskInputs(), torch.zeros(1, 1, 1, 96, dtype=torch.float32)) == 128
    assert rh._padded_head_size(cfg, _FakeMaskInputs(), torch.zeros(1, 1, 1, 40, dtype=torch.bfloat16)) == (64 if on_grid else 128)
    assert rh._padded_head_size(cfg, _FakeMaskInputs(), torch.zeros(1, 1, 1, 40, dtype=torch.float32)) == 64
    assert rh._padded_head_size(cfg, _FakeMaskInputs(), torch.zeros(1, 1, 1, 160, dtype=torch.bfloat16)) == 256
    assert rh._padded_head_size(cfg, _FakeMaskInputs(), torch.zeros(1, 1, 1, 256, dtype=torch.bfloat16)) == 0
    assert rh._padded_head_size(cfg, _FakeMaskInputs(), torch.zeros(1, 1, 1, 16, dtype=torch.float32)) == (64 if on_grid else 32)
    # the vector kernels asked for by name, or attention dropout: their head sizes
    cfg_g = rh._Config(dict(query_chunk_size=cfg.qc, key_chunk_size=cfg.kc, causal_block_size=cbs, impl="generic"))
    assert rh._padded_head_size(cfg_g, _FakeMaskInputs(), q32) == 0
    with pytest.raises(NotImplementedError):
        rh._padded_head_size(cfg, _FakeMaskInputs(), torch.zeros(1, 1, 1, 272, dtype=torch.bfloat16))
    assert rh._padded_head_size(cfg, _FakeMaskInputs(), torch.zeros(1, 1, 1, 128, dtype=torch.bfloat16)) == 0


def test_output_residual_option():
    from ringattention_amd.ringattention_hip import _Config
    base = dict(causal_block_size=1, query_chunk_size=128, key_chunk_size=128)
    assert _Config(base).output_residual == "fp32"                          # the reference's residual (:53)
    assert _Config(dict(base, output_residual="rounded")).output_residual == "rounded"
    with pytest.raises(ValueError):
        _Config(dict(base, output_residual="bf16"))


def test_mask_inputs_accept_segment_ids_made_under_inference_mode():
    """Inference tensors have no version counter: the per-tensor cache of the int32 ids and tile ranges is bypassed
    for them instead of raising, and the ranges equal those of an ordinary tensor."""
    from ringattention_amd import ringattention_hip as R
    cfg = R._Config(dict(query_chunk_size=128, key_chunk_size=128, causal_block_size=1))
    ids = torch.arange(300) // 70
    with torch.inference_mode():
        seg = ids.clone().reshape(1, -1)
        with pytest.raises(RuntimeError):
            seg._version
        mi = R._MaskInputs(cfg, None, seg, None, 1, "cpu", 300)
    ref = R._MaskInputs(cfg, None, ids.reshape(1, -1), None, 1, "cpu", 300)
    assert torch.equal(mi.seg_mm, ref.seg_mm) and torch.equal(mi.seg, ref.seg)
    assert mi.seg_mm.shape == (1, 5, 2)
    assert mi.seg_mm[0, 1].tolist() == [0, 1] and mi.seg_mm[0, 4].tolist() == [3, 4]
    assert mi.segments_meet(0, 64, 256, 300) is False and mi.segments_meet(0, 128, 64, 128) is True


def test_segment_cache_follows_the_version_counter_and_the_opt_out():
    from ringattention_amd import ringattention_hip as R
    cfg = R._Config(dict(query_chunk_size=128, key_chunk_size=128, causal_block_size=1))
    seg = (torch.arange(256) // 100).reshape(1, -1)
    a = R._MaskInputs(cfg, None, seg, None, 1, "cpu", 256)
    b = R._MaskInputs(cfg, None, seg, None, 1, "cpu", 256)
    assert a._seg_entry is b._seg_entry                  # unchanged tensor: one entry
    seg[0, 0] = 7                                        # in-place edit bumps the version: recomputed
    c = R._MaskInputs(cfg, None, seg, None, 1, "cpu", 256)
    assert c._seg_entry is not a._seg_entry and c.seg_mm[0, 0].tolist() == [0, 7]
    seg.numpy()[0, 1] = 9                                # an edit the counter does not see needs the opt-out
    cfg2 = R._Config(dict(query_chunk_size=128, key_chunk_size=128, causal_block_size=1, cache_segment_ids=False))
    d = R._MaskInputs(cfg2, None, seg, None, 1, "cpu", 256)
    assert d.seg_mm[0, 0].tolist() == [0, 9]


def test_bias_and_segment_ids_must_broadcast_or_match_batch_and_heads():
    """The kernels index attn_bias by batch row and head and segment_ids by batch row: a dim that is neither 1 nor the
    array's own would be read past its end, so the host refuses it before anything is launched."""
    from ringattention_amd import ringattention_hip as rh
    cfg = rh._Config(dict(query_chunk_size=8, key_chunk_size=8, causal_block_size=1, cache_segment_ids=False))
    ok_bias = torch.zeros(1, 4, 1, 64)
    rh._MaskInputs(cfg, ok_bias, torch.zeros(1, 64, dtype=torch.int32), None, 3, "cpu", 64, 4)
    rh._MaskInputs(cfg, torch.zeros(3, 1, 1, 64), torch.zeros(3, 64, dtype=torch.int32), None, 3, "cpu", 64, 4)
    for bad_bias in (torch.zeros(2, 1, 1, 64), torch.zeros(1, 3, 1, 64)):
        with pytest.raises(ValueError):
            rh._MaskInputs(cfg, bad_bias, None, None, 3, "cpu", 64, 4)
    with pytest.raises(ValueError):
        rh._MaskInputs(cfg, None, torch.zeros(2, 64, dtype=torch.int32), None, 3, "cpu", 64, 4)


def test_blockwise_feedforward_generic_callable_groups_and_remat():
    """A callable that is not the library's SwiGLU (ringattention_jax.py:333-352): the scan hands it the reference's
    strided token groups {c * n + j} ('b (c n) d -> b c n d'); with pre_remat=False it is rematerialised per chunk
    (its forward pass runs again in the backward pass), with the default True it is called once per chunk.  Same
    values and gradients either way, equal to the un-chunked call.  Runs on the CPU: no kernel of the library is
    involved."""
    import ringattention_amd as ra
    torch.manual_seed(0)
    mlp = torch.nn.Sequential(torch.nn.Linear(16, 48), torch.nn.GELU(), torch.nn.Linear(48, 16))
    calls = []

    def ff(h):
        calls.append(tuple(h.shape))
        return mlp(h)
    x = torch.randn(2, 24, 16, requires_grad=True)
    ref = mlp(x)
    ref.square().sum().backward()
    gx, gw = x.grad.clone(), mlp[0].weight.grad.clone()
    for pre_remat, n_calls in ((True, 4), (False, 8)):
        x.grad = None
        mlp.zero_grad()
        calls.clear()
        y = ra.blockwise_feedforward(ff, x, 6, pre_remat=pre_remat)
        assert torch.allclose(y, ref, atol=1e-6)
        y.square().sum().backward()
        assert calls[:4] == [(2, 6, 16)] * 4 and len(calls) == n_calls
        assert torch.allclose(x.grad, gx, atol=1e-5) and torch.allclose(mlp[0].weight.grad, gw, atol=1e-5)
    # the groups are strided: step j sees tokens j, n + j, 2 n + j, ...
    seen = []
    ra.blockwise_feedforward(lambda h: (seen.append(h[0, :, 0].clone()), h)[1], torch.arange(24.).reshape(1, 24, 1), 6)
    assert torch.equal(seen[1], torch.tensor([1., 5., 9., 13., 17., 21.]))
    # a policy that keeps the activations switches the rematerialisation off again
    calls.clear()
    ra.blockwise_feedforward(ff, x, 6, pre_remat=False, policy="everything_saveable").sum().backward()
    assert len(calls) == 4


def test_swiglu_weights_must_be_dense_bf16():
    """A module moved to fp32 or given a transposed weight would be read as garbage by kernels that take raw bf16
    pointers: refused before anything is launched (the check runs on the host; no GPU needed)."""
    from ringattention_amd import feedforward as F
    ff = F.SwiGLU(128, 256, device="cpu")
    x = torch.zeros(4, 128, dtype=torch.bfloat16)
    F._check_swiglu_weights(ff, x)
    with pytest.raises(ValueError):
        F._check_swiglu_weights(ff, torch.zeros(4, 64, dtype=torch.bfloat16))
    ff.w2.data = ff.w2.data.t().contiguous().t()
    with pytest.raises(ValueError):
        F._check_swiglu_weights(ff, x)
    with pytest.raises(NotImplementedError):
        F._check_swiglu_weights(F.SwiGLU(128, 256, device="cpu").float(), x)
