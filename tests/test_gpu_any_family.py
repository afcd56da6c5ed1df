"""The matrix-core kernels that evaluate the mask element by element (blockwise_kwargs["impl"] = "mfma_any") against the
CPU oracle: the random configurations of test_gpu_random_configs with bf16 inputs."""
import pytest
import torch

import ringattention_amd as ra
from tests.test_gpu_attention import run_hip
from tests.test_gpu_random_configs import OFFSET, draw
from tests.util import assert_close_scaled, kwargs, make_qkv, oracle_fwd_bwd, packed_segment_ids

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(OFFSET, OFFSET + 160))
def test_random_configuration_on_the_elementwise_matrix_core_kernels(seed):
    c = draw(seed)
    c["dtype"] = torch.bfloat16
    print("any case", seed, c, flush=True)
    n, B, H, D = c["n"], c["B"], c["H"], c["D"]
    S, Skv = n * c["q_len"], n * c["kv_len"]
    q, k, v, do = make_qkv(B, S, H, D, dtype=c["dtype"], seed=seed, Skv=Skv, scale=c["qk_std"])
    g = torch.Generator().manual_seed(seed + 500)
    bias = None
    if c["bias"] == "key":
        bias = torch.randn(1, 1, 1, Skv, generator=g)
    elif c["bias"] == "head":
        bias = torch.randn(B, H, 1, Skv, generator=g)
    elif c["bias"] == "row":
        bias = torch.randn(1, H, c["qc"], Skv, generator=g)
    elif c["bias"] == "pad":
        keep = torch.arange(Skv)[None, :] < torch.randint(1, Skv + 1, (B, 1), generator=g)
        bias = torch.where(keep, 0.0, torch.finfo(c["kw_dtype"]).min).reshape(B, 1, 1, Skv)
    seg = None
    if c["seg"] in ("docs", "relabelled"):
        seg = packed_segment_ids(B, max(S, Skv), max(4, S // 5), seed=seed + 7)
    elif c["seg"] == "one":
        seg = torch.zeros(B, max(S, Skv), dtype=torch.int32)
    if c["seg"] == "relabelled":
        table = torch.randint(-3, 4, (int(seg.max()) + 1,), generator=g, dtype=torch.int32)
        seg = table[seg[:1].long()]
    if c["bias"] == "pad" and c["seg"] in ("docs", "relabelled"):
        seg = None
    kw = kwargs(c["qc"], c["kc"], c["cbs"], dtype=c["kw_dtype"], impl="mfma_any")
    ref_out, ref_grads = oracle_fwd_bwd(q, k, v, do, bias, seg, None, n, kw)
    out, grads = run_hip(q, k, v, do, bias, seg, None, n, kw)
    fam = ra.kernel_family_of_last_call()
    print("  family", fam, flush=True)
    assert fam == {"forward": "mfma_bf16_any", "backward": "mfma_bf16_any"}, fam
    assert_close_scaled(out, ref_out, torch.bfloat16, "out")
    for name, a, b in zip(("dq", "dk", "dv"), grads, ref_grads):
        assert_close_scaled(a, b, torch.bfloat16, name)
