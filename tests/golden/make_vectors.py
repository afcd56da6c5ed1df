"""Writes tests/golden/oracle_vectors.npz: small seeded inputs with the outputs of THIS repository's CPU oracle
(oracle/ringattention_oracle.py) at the time of writing.

The reference holds no golden vectors and its runtime (JAX) is not installed, so these are not reference outputs:
they freeze the oracle's results once it had passed every check of tests/test_oracle.py, so that a later change of
the oracle or of the HIP path that moves a number shows up.  Run from the repository root:
    python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from oracle import ringattention_oracle as O   # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def kwargs(qc, kc, cbs, drop_permille=0, seed=None):
    return dict(causal_block_size=cbs, deterministic=drop_permille == 0, dropout_rng=seed,
                attn_pdrop=drop_permille / 1000.0, query_chunk_size=qc,
                key_chunk_size=kc, dtype=torch.float32, policy=None, precision=None, prevent_cse=True)


def bf16_exact(t):
    """Inputs are rounded to bf16-representable values, so the bf16 kernels see exactly what the oracle saw."""
    return t.to(torch.bfloat16).float()


def store(t):
    """bf16-exact float inputs are stored as their upper 16 bits; everything else as it is."""
    t = t.detach()
    if t.dtype == torch.float32 and torch.equal(t, t.to(torch.bfloat16).float()):
        return t.to(torch.bfloat16).view(torch.int16).numpy()
    return t.numpy()


def cases():
    """name -> (inputs dict, config dict).  Everything needed to rebuild the call is stored with the outputs."""
    out = {}
    g = torch.Generator().manual_seed(2024)
    B, S, H, D = 1, 64, 1, 64
    q, k, v, do = (bf16_exact(torch.randn(B, S, H, D, generator=g)) for _ in range(4))
    bias = torch.randn(1, 1, 1, S, generator=g)
    seg = torch.tensor([[0] * 20 + [1] * 25 + [2] * 19], dtype=torch.int32)
    out["ring2_causal_bias_segments"] = (dict(q=q, k=k, v=v, do=do, bias=bias, seg=seg), dict(qc=16, kc=16, cbs=1, n=2))
    out["one_device_causal_block4"] = (dict(q=q, k=k, v=v, do=do), dict(qc=8, kc=16, cbs=4, n=1))
    # attention dropout (rate 0.3, the documented Philox stream seeded with 1234), two devices: the second one
    # reads the mask through the clamped slices
    out["ring2_causal_dropout"] = (dict(q=q, k=k, v=v, do=do), dict(qc=16, kc=16, cbs=1, n=2, drop_permille=300,
                                                                    seed=1234))
    qd = bf16_exact(torch.randn(2, 1, H, D, generator=g))
    kd, vd = bf16_exact(torch.randn(2, 96, H, D, generator=g)), bf16_exact(torch.randn(2, 96, H, D, generator=g))
    out["decode_cache_idx_70"] = (dict(q=qd, k=kd, v=vd), dict(qc=1, kc=32, cbs=1, n=1, cache_idx=70))
    return out


def run_case(inp, cfg):
    kw = kwargs(cfg["qc"], cfg["kc"], cfg["cbs"], cfg.get("drop_permille", 0), cfg.get("seed"))
    out, res = O.ring_attention_fwd(inp["q"], inp["k"], inp["v"], inp.get("bias"), inp.get("seg"), cfg.get("cache_idx"),
                                    cfg["n"], True, kw)
    r = {"out": out}
    if "do" in inp:
        dq, dk, dv = O.ring_attention_bwd(cfg["n"], True, kw, res, inp["do"])
        r.update(dq=dq, dk=dk, dv=dv)
    return r


def main():
    blob = {}
    for name, (inp, cfg) in cases().items():
        for k_, t in inp.items():
            blob["%s/in/%s" % (name, k_)] = store(t)
        for k_, val in cfg.items():
            blob["%s/cfg/%s" % (name, k_)] = np.asarray(val)
        for k_, t in run_case(inp, cfg).items():
            blob["%s/out/%s" % (name, k_)] = t.detach().float().numpy()
    # inference ring: boolean mask (B, 1, Q, K_total), two devices
    g = torch.Generator().manual_seed(7)
    q, k, v, do = (bf16_exact(torch.randn(1, 64, 1, 64, generator=g)) for _ in range(4))
    mask = torch.rand(1, 1, 64, 64, generator=g) > 0.3
    mask[..., 0] = True
    out, res = O.ring_attention_inference_fwd(q, k, v, mask, 2)
    dq, dk, dv = O.ring_attention_inference_bwd(2, res, do)
    for k_, t in dict(q=q, k=k, v=v, do=do, mask=mask).items():
        blob["inference_ring2/in/%s" % k_] = store(t)
    for k_, t in dict(out=out, dq=dq, dk=dk, dv=dv).items():
        blob["inference_ring2/out/%s" % k_] = t.detach().float().numpy()
    # SwiGLU feed-forward in chunks (too small for the GPU kernels' 128-multiples: an oracle-only vector)
    x = bf16_exact(torch.randn(2, 32, 16, generator=g)).requires_grad_(True)
    w1, w3 = (bf16_exact(torch.randn(16, 24, generator=g) * 0.2).requires_grad_(True) for _ in range(2))
    w2 = bf16_exact(torch.randn(24, 16, generator=g) * 0.2).requires_grad_(True)
    dy = bf16_exact(torch.randn(2, 32, 16, generator=g))
    y = O.blockwise_feedforward(lambda h: O.swiglu(h, w1, w2, w3), x, 8)
    y.backward(dy)
    for k_, t in dict(x=x, w1=w1, w2=w2, w3=w3, dy=dy).items():
        blob["ffn_chunk8/in/%s" % k_] = store(t)
    for k_, t in dict(y=y, dx=x.grad, dw1=w1.grad, dw2=w2.grad, dw3=w3.grad).items():
        blob["ffn_chunk8/out/%s" % k_] = t.detach().numpy()
    path = os.path.join(HERE, "oracle_vectors.npz")
    np.savez_compressed(path, **blob)
    print(path, "%.0f KB" % (os.path.getsize(path) / 1024), len(blob), "arrays")


if __name__ == "__main__":
    main()
