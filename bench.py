#!/usr/bin/env python3
"""Benchmark of the ring-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload attn32k|ring131k|ffn|decode|inference|copy|decode_step|rmsnorm|dropout32k|c1|mfma_probe|vendor_sdpa]

One step = one pass of the hot path over one batch of synthetic input already resident in HBM.
Default workload ``attn32k`` is the configuration the headline metric is quoted on: blockwise
causal attention forward+backward, bf16, B=1 H=32 S=32768 D=128, chunks 512/512.  Prints ONE JSON
line with the throughput, the roofline figures of the dominant kernel (timed live with events on
the launch stream) and a CPU baseline (the CPU oracle timed on a bounded slice of the workload).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6      # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3        # MI355X dense fp32 MFMA
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E


def _measured(profile, kind):
    """Figures that only a ``rocprofv3 --pmc`` run can give (HBM bytes per launch, MFMA busy share), read from the
    summary committed under profiles/: lines ``<kind> <kernel> <value>`` after lines ``source <path> sha256=<hex>``
    naming the kernel sources the run was made with.  A figure is reported only while every one of those sources
    still hashes to the recorded value; once a kernel source has changed the table is stale and this returns {}."""
    import hashlib
    path = os.path.join(ROOT, "profiles", profile)
    out, ok = {}, True
    try:
        for line in open(path):
            w = line.split()
            if len(w) == 3 and w[0] == "source" and w[2].startswith("sha256="):
                try:
                    ok = ok and hashlib.sha256(open(os.path.join(ROOT, w[1]), "rb").read()).hexdigest() == w[2][7:]
                except OSError:
                    ok = False
            elif len(w) == 3 and w[0] == kind:
                out[w[1]] = float(w[2])
    except OSError:
        return {}
    return out if ok else {}


TRAFFIC_PROFILE = "hbm_traffic_pmc.txt"
MFMA_PROFILE = "mfma_utilisation_pmc.txt"


def _kwargs(qc, kc, cbs=1, **extra):
    import torch
    kw = dict(causal_block_size=cbs, deterministic=True, dropout_rng=None, attn_pdrop=0.0,
              query_chunk_size=qc, key_chunk_size=kc, dtype=torch.float32, policy=None, precision=None,
              prevent_cse=True)
    kw.update(extra)
    return kw


def _note(msg):
    """A line on stderr: a sign of life from runs whose steps take many seconds (the JSON line stays alone on stdout)."""
    print("[bench] " + msg, file=sys.stderr, flush=True)


def _time_steps(fn, steps, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if steps <= 2:          # a handful of long steps: say so as they finish (the wait costs nothing next to them)
        for i in range(steps):
            t1 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            if time.perf_counter() - t1 > 5.0:
                _note("step %d of %d: %.1f s" % (i + 1, steps, time.perf_counter() - t1))
    else:
        for _ in range(steps):
            fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def _event_ms(fn, reps):
    """Average duration of ``fn`` (which launches on torch's current stream) from events on that stream.  A call
    that takes seconds is repeated once, not ``reps`` times."""
    import torch
    t0 = time.perf_counter()
    fn()
    torch.cuda.synchronize()
    if time.perf_counter() - t0 > 2.0:
        _note("a launch of %.1f s: timed once more" % (time.perf_counter() - t0))
        reps = 1
    total = 0.0
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        total += e0.elapsed_time(e1)
    return total / reps


def _gpu_sysfs_dirs():
    """sysfs device directories of the GPU this process uses (matched by PCI address where torch gives one; else
    every card)."""
    import glob
    import torch
    dirs = sorted(os.path.dirname(f) for f in glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
    try:
        pr = torch.cuda.get_device_properties(0)
        addr = "%04x:%02x:%02x" % (getattr(pr, "pci_domain_id", 0), pr.pci_bus_id, pr.pci_device_id)
        mine = [d for d in dirs if addr in os.path.realpath(d)]
        if mine:
            return mine
    except Exception:
        pass
    return dirs


def _read_int(path):
    try:
        return int(open(path).read().split()[0])
    except (OSError, ValueError, IndexError):
        return None


def _sclk_under_load(fn, seconds=2.0):
    """Shader clock in MHz (the level the driver marks current in sysfs pp_dpm_sclk, what rocm-smi --showclocks
    prints) and board power in W (hwmon power1_input / power1_average, next to the limit in power1_cap) sampled from
    a thread while ``fn`` runs back to back for ``seconds``: median, min and max of the samples taken under load, or
    None where the files are not readable.  Plain file reads: no child process is started.  The nominal peak figures
    assume 2400 MHz; the samples of the first half second (the ramp from idle) are left out of the power figures."""
    import glob
    import re
    import threading
    import torch
    dirs = _gpu_sysfs_dirs()
    if not dirs:
        return None
    files = [os.path.join(d, "pp_dpm_sclk") for d in dirs]
    pfiles = [p for d in dirs for p in glob.glob(os.path.join(d, "hwmon/hwmon*/power1_input")) +
              glob.glob(os.path.join(d, "hwmon/hwmon*/power1_average"))][:1]
    cap = _read_int(pfiles[0].rsplit("/", 1)[0] + "/power1_cap") if pfiles else None
    samples, watts, stop = [], [], threading.Event()
    t0 = time.perf_counter()

    def poll():
        while not stop.is_set():
            best = 0
            for f in files:
                try:
                    m = re.search(r"(\d+)Mhz \*", open(f).read())
                except OSError:
                    m = None
                if m:
                    best = max(best, int(m.group(1)))
            if best:
                samples.append(best)
            w = _read_int(pfiles[0]) if pfiles else None
            if w and time.perf_counter() - t0 > 0.5:
                watts.append(w * 1e-6)
            stop.wait(0.1)

    th = threading.Thread(target=poll, daemon=True)
    th.start()
    while time.perf_counter() - t0 < seconds:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()
    stop.set()
    th.join(timeout=10)
    busy = sorted(x for x in samples if x > 500)
    if not busy:
        return None
    res = {"median": busy[len(busy) // 2], "min": busy[0], "max": busy[-1], "samples": len(busy)}
    if watts:
        watts.sort()
        res["power_w"] = {"median": round(watts[len(watts) // 2], 1), "max": round(watts[-1], 1),
                          "cap": round(cap * 1e-6, 1) if cap else None}
    return res


def _packed_segments(S, mean_len, seed, device):
    import numpy as np
    import torch
    rng = np.random.default_rng(seed)
    lens = []
    tot = 0
    while tot < S:
        ln = int(rng.geometric(1.0 / mean_len))
        lens.append(ln)
        tot += ln
    ids = np.repeat(np.arange(len(lens)), lens)[:S].astype(np.int32)
    lens[-1] -= tot - S
    return torch.from_numpy(ids).reshape(1, S).to(device), lens


# --------------------------------------------------------------------------- attention workloads
def bench_attention(args, ring, dropout=False, c1=False):
    import torch
    import ringattention_amd as ra
    from ringattention_amd import ringattention_hip as rh
    dev = "cuda:0"
    D, H, B = 128, 32, 1
    if args.head_dim:
        D, H = args.head_dim, 32 * 128 // args.head_dim      # the same model width
    if ring:
        S, n, name = 131072, 8, "ring131k"
    else:
        S, n, name = 32768, 1, "attn32k"
    if dropout:
        name = "dropout32k"
    if c1:
        # the reference's own CPU-runnable configuration: B1 H8 S2048 D64 fp32, N(0,1) inputs, a zero bias, one document
        S, n, name, D, H = 2048, 1, "c1", 64, 8
        args = argparse.Namespace(**dict(vars(args), dtype="fp32", inputs="unit"))
    if args.seq_len:
        S = args.seq_len
    if args.batch:
        B = args.batch
    g = torch.Generator(device=dev).manual_seed(0)
    # q, k, v ~ N(0,1) / sqrt(D) is the input the configuration names; it makes the logits tiny (std 0.008).  The
    # other choices give the logits a standard deviation of 0.09 (q, k scaled D^-0.25) or 1 (unscaled q, k)
    qk_scale = {"baseline": D ** -0.5, "d-quarter": D ** -0.25, "unit": 1.0}[args.inputs]
    v_scale = D ** -0.5 if args.inputs == "baseline" else 1.0
    fp32 = getattr(args, "dtype", "bf16") == "fp32"
    tdt = torch.float32 if fp32 else torch.bfloat16
    peak = PEAK_F32_TFLOPS if fp32 else PEAK_BF16_TFLOPS
    # (a head size above 128: the matrix-core kernels that evaluate the mask element by element)
    sfx = "_f32_kernel" if fp32 else ("_any_kernel" if D > 128 else "_ws_kernel")
    mk = lambda sc: (torch.randn(B, S, H, D, device=dev, generator=g) * sc).to(tdt)
    q, k, v = mk(qk_scale).requires_grad_(True), mk(qk_scale).requires_grad_(True), mk(v_scale).requires_grad_(True)
    do = torch.randn(B, S, H, D, device=dev, generator=g).to(tdt)
    bias = seg = None
    pairs = S * (S + 1) / 2
    if ring:
        bias = torch.randn(1, 1, 1, S, device=dev, generator=g)
        seg, lens = _packed_segments(S, 4096, 0, dev)
        pairs = float(sum(l * (l + 1) / 2 for l in lens))
    if c1:
        bias = torch.zeros(1, 1, 1, S, device=dev)
        seg = torch.zeros(1, S, dtype=torch.int32, device=dev)
    kw = _kwargs(512, 512, 1)
    if fp32:
        kw["dtype"] = torch.float32
    pdrop = 0.1
    if dropout:
        # attention dropout: a fresh seed every step, so drawing and packing the mask is part of the step; only the
        # pairs that are kept count as work
        kw.update(deterministic=False, attn_pdrop=pdrop, dropout_rng=0)
        pairs *= 1.0 - pdrop
    flops_fwd = 4.0 * D * pairs * B * H
    flops_bwd = 10.0 * D * pairs * B * H
    seed = [0]

    def step():
        q.grad = k.grad = v.grad = None
        seed[0] += 1
        kws = dict(kw, dropout_rng=seed[0]) if dropout else kw
        with ra.ring_axis("sp", n):
            out = ra.ringattention(q, k, v, bias, seg, None, axis_name="sp", float32_logits=True, blockwise_kwargs=kws)
            out.backward(do)

    ms = _time_steps(step, args.steps, args.warmup)
    value = (flops_fwd + flops_bwd) / (ms * 1e-3) / 1e12

    # --- per-kernel durations (events on the launch stream), N=1 shape of one ring step
    roof = None
    kern = {}
    sclk = None
    if not ring and not c1:
        with torch.no_grad():
            cfg = rh._Config(kw)
            mi = rh._MaskInputs(cfg, None, None, None, B, q.device, S)
            # the launches of the step: one ring step that is the first and the last of its device, so there is no
            # fp32 numerator or gradient array: out and dq / dk / dv are written once, in bf16
            from ringattention_amd import _lib as L
            den = torch.empty(B, H, S, dtype=torch.float32, device=dev)
            mx = torch.empty(B, H, S, dtype=torch.float32, device=dev)
            qd, kd, vd = q.detach(), k.detach(), v.detach()
            out = torch.empty_like(qd)
            # the fp32 residual the step keeps next to a bf16 output
            out32 = torch.empty(qd.shape, dtype=torch.float32, device=dev) if not fp32 else None
            fwd = lambda: rh._blockwise_attention_fwd(qd, kd, vd, (None, den, mx), 0, 0, None, None, 1, 512, 512,
                                                      _mask_inputs=mi, _cfg=cfg, _carry_is_initial=True, _out=out,
                                                      _out_f32=out32)
            fwd()            # under dropout the first call draws and packs the mask, which stays with mi
            kern["attn_fwd" + sfx] = (_event_ms(fwd, 5), flops_fwd)
            delta = rh._bwd_delta(do, out32 if out32 is not None else out)
            dq_o, dk_o, dv_o = (torch.empty_like(qd) for _ in range(3))
            for which, share in (("dkv", 8.0), ("dq", 2.0)):
                cfg1 = rh._Config(dict(kw, bwd_only=which))
                bw = lambda: rh._blockwise_attention_bwd(qd, kd, vd, do, (None, None, None, out, den, mx), 0, 0, None,
                                                         None, 1, 512, 512, _mask_inputs=mi, _cfg=cfg1, _delta=delta,
                                                         _grads_initial=L.RA_GRAD_INIT_DQ | L.RA_GRAD_INIT_DKV,
                                                         _dq_out=dq_o, _dkv_out=(dk_o, dv_o))
                kern["attn_bwd_%s%s" % (which, sfx)] = (_event_ms(bw, 5), share * D * pairs * B * H)
                if which == "dkv" and not (args.no_extras or dropout):
                    sclk = _sclk_under_load(bw)       # the clock the dominant kernel actually runs at
            if dropout:
                def draw():
                    m2 = rh._MaskInputs(cfg, None, None, None, B, q.device, S)
                    m2.use_dropout(cfg, B, H, S, S, 0, 0, q.device)
                del mi
                mask_ms = _event_ms(draw, 3)
        traffic, util = _measured(TRAFFIC_PROFILE, "traffic"), _measured(MFMA_PROFILE, "mfma_util")
        dom = max(kern, key=lambda n_: kern[n_][0])
        dms, dfl = kern[dom]
        ach = dfl / (dms * 1e-3) / 1e12
        roof = {"bound": "mfma", "kernel": dom, "achieved": round(ach, 1), "peak": peak,
                "unit": "TFLOP/s", "frac": round(ach / peak, 4),
                "traffic": traffic.get(dom) if S == 32768 and args.inputs == "baseline" else None,
                "traffic_source": ("profiles/" + TRAFFIC_PROFILE
                                   if traffic.get(dom) and S == 32768 and args.inputs == "baseline" else None),
                "mfma_util_pmc": ({"kernel": util.get(dom), "step": util.get("attn32k_step"),
                                   "source": "profiles/" + MFMA_PROFILE}
                                  if S == 32768 and not dropout and util.get(dom) else None),
                "kernel_ms": {n_: round(t, 3) for n_, (t, _) in kern.items()},
                "kernel_tflops": {n_: round(f / (t * 1e-3) / 1e12, 1) for n_, (t, f) in kern.items()}}
        if sclk:
            # the published peak assumes 2400 MHz; what the same matrix pipes can do at the clock the kernel runs at
            roof["power_w_under_load"] = sclk.pop("power_w", None)
            roof["sclk_mhz_under_load"] = sclk
            roof["frac_of_peak_at_sclk"] = round(ach / (peak * sclk["median"] / 2400.0), 4)
        if dropout:
            roof["traffic"] = None
            roof["mask_draw_and_pack_ms"] = round(mask_ms, 3)
    if ring:
        # per kernel: the sum of its launches over the scan steps of one pass (two steps have work: every device
        # against its own shard, then the documents that straddle a shard boundary), events on the launch stream
        import copy
        with torch.no_grad(), ra.ring_axis("sp", n):
            qd, kd, vd = q.detach(), k.detach(), v.detach()
            fwd = lambda: rh._ring_attention_fwd(qd, kd, vd, bias, seg, None, "sp", True, kw)
            res = fwd()[1]
            kern["attn_fwd_ws_kernel"] = (_event_ms(fwd, 3), flops_fwd)
            t_delta = _event_ms(lambda: rh._bwd_delta(do, res[0]), 3)
            for which, share in (("dkv", 8.0), ("dq", 2.0)):
                cfg_p = copy.copy(res[5])
                cfg_p.bwd_only = {"dq": 1, "dkv": 2}[which]        # RA_BWD_PART_*
                res_p = res[:5] + (cfg_p,) + res[6:]
                t = _event_ms(lambda: rh._ring_attention_bwd(res_p, do), 3) - t_delta
                kern["attn_bwd_%s_ws_kernel" % which] = (t, share * D * pairs * B * H)
            del res, res_p
        util = _measured(MFMA_PROFILE, "mfma_util")
        dom = max(kern, key=lambda n_: kern[n_][0])
        dms, dfl = kern[dom]
        ach = dfl / (dms * 1e-3) / 1e12
        ring_traffic = _measured(TRAFFIC_PROFILE, "traffic").get("ring131k:" + dom) if S == 131072 else None
        roof = {"bound": "mfma", "kernel": dom, "achieved": round(ach, 1), "peak": peak, "unit": "TFLOP/s",
                "frac": round(ach / peak, 4), "traffic": ring_traffic,
                "traffic_source": "profiles/" + TRAFFIC_PROFILE if ring_traffic else None,
                "scope": "the kernel's launches of one pass summed (one per scan step with work, host launch gaps "
                         "included), FLOP of unmasked pairs: 8*D per pair for dK/dV, 2*D for dQ, 4*D forward",
                "mfma_util_pmc": ({"kernel": util.get("ring131k:" + dom), "step": util.get("ring131k_step"),
                                   "source": "profiles/" + MFMA_PROFILE}
                                  if S == 131072 and util.get("ring131k:" + dom) else None),
                "kernel_ms": {n_: round(t, 3) for n_, (t, _) in kern.items()},
                "kernel_tflops": {n_: round(f / (t * 1e-3) / 1e12, 1) for n_, (t, f) in kern.items()}}
        if not args.no_extras:
            # clock and board power over whole steps: what tells a power-limited step from a stall-limited one
            whole = _sclk_under_load(step)
            if whole:
                roof["power_w_under_load"] = whole.pop("power_w", None)
                roof["sclk_mhz_under_load"] = whole
    if c1:
        roof = {"bound": "mfma", "kernel": None, "achieved": round(value, 2), "peak": peak, "unit": "TFLOP/s",
                "frac": round(value / peak, 4), "traffic": None,
                "scope": "whole step: 128 forward and dQ workgroups on 256 CUs, launch-bound"}
    cpu = None
    if c1 and not args.no_cpu:
        cpu = cpu_baseline_c1(q.detach().cpu(), k.detach().cpu(), v.detach().cpu(), do.cpu(), kw)
    elif ring and not args.no_cpu:
        cpu = cpu_baseline_ring(lens)
    elif not (args.no_cpu or dropout):
        cpu = cpu_baseline_attention()
    del q, k, v, do
    pct_key = "pct_f32_mfma_peak" if fp32 else "pct_bf16_mfma_peak"
    return {
        "metric": "attn_fwd_bwd_tflops", "value": round(value, 2), "unit": "TFLOP/s", "ms_per_step": round(ms, 3),
        "dtype": "f32" if fp32 else "bf16", pct_key: round(100 * value / peak, 2),
        "config": {"workload": name, "B": B, "H": H, "S": S, "D": D, "causal_block_size": 1,
                   "query_chunk_size": 512, "key_chunk_size": 512, "virtual_ring": n,
                   "segment_ids": seg is not None, "bias": bias is not None, "attn_pdrop": pdrop if dropout else 0.0,
                   "inputs": {"baseline": "q, k, v ~ N(0,1)/sqrt(D), dO ~ N(0,1)",
                              "d-quarter": "q, k ~ N(0,1) * D^-0.25, v, dO ~ N(0,1)",
                              "unit": "q, k, v, dO ~ N(0,1)"}[args.inputs],
                   "flop_convention": "4*D fwd + 10*D bwd per unmasked (q,k) pair per head"},
        "roofline": roof, "cpu_baseline": cpu,
    }


def cpu_baseline_c1(q, k, v, do, kw):
    """The CPU oracle on the whole of the reference's CPU-runnable configuration, forward + backward."""
    import torch
    from oracle import ringattention_oracle as O
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    S, H, D = q.shape[1], q.shape[2], q.shape[3]
    bias, seg = torch.zeros(1, 1, 1, S), torch.zeros(1, S, dtype=torch.int32)
    reps, t0 = 0, time.perf_counter()
    while reps < 3 or time.perf_counter() - t0 < 10.0:
        out, res = O.ring_attention_fwd(q, k, v, bias, seg, None, 1, True, kw)
        O.ring_attention_bwd(1, True, kw, res, do)
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    flops = 14.0 * D * (S * (S + 1) / 2) * H
    return {"value": round(flops / dt / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": "the whole configuration, fwd+bwd, %d repetitions of %.3f s" % (reps, dt)}


def cpu_baseline_attention():
    """The CPU oracle (torch-CPU fp32, the reference's loop structure) on 8 of the 32 heads of the
    attn32k workload at full S=32768: forward + backward, fp32 logits, chunks 512/512."""
    import torch
    from oracle import ringattention_oracle as O
    S, D, Hc = 32768, 128, 8
    cores = os.cpu_count() or 1
    cores = min(cores, 16)
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)
    q, k, v, do = (torch.randn(1, S, Hc, D, generator=g) * (D ** -0.5 if i < 2 else 1.0) for i in range(4))
    kw = _kwargs(512, 512, 1)
    t0 = time.perf_counter()
    out, res = O.ring_attention_fwd(q, k, v, None, None, None, 1, True, kw)
    O.ring_attention_bwd(1, True, kw, res, do)
    dt = time.perf_counter() - t0
    flops = 14.0 * D * (S * (S + 1) / 2) * Hc
    return {"value": round(flops / dt / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": "8 heads (of 32) at full S=32768, fwd+bwd, %.1f s" % dt}


def cpu_baseline_ring(lens):
    """The CPU oracle on a slice of the ring131k workload: one head (of 32) over the first 65536 positions (of
    131072) as a ring of four shards of 16384, the same packed documents and a per-key bias, forward + backward."""
    import numpy as np
    import torch
    from oracle import ringattention_oracle as O
    S, D, n = 65536, 128, 4
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)
    q, k, v, do = (torch.randn(1, S, 1, D, generator=g) * (D ** -0.5 if i < 3 else 1.0) for i in range(4))
    bias = torch.randn(1, 1, 1, S, generator=g)
    ids = np.repeat(np.arange(len(lens)), lens)[:S].astype(np.int32)
    seg = torch.from_numpy(ids).reshape(1, S)
    cut = np.bincount(ids).astype(np.float64)                    # document lengths inside the slice
    pairs = float((cut * (cut + 1) / 2).sum())
    kw = _kwargs(512, 512, 1)
    t0 = time.perf_counter()
    out, res = O.ring_attention_fwd(q, k, v, bias, seg, None, n, True, kw)
    O.ring_attention_bwd(n, True, kw, res, do)
    dt = time.perf_counter() - t0
    return {"value": round(14.0 * D * pairs / dt / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": "1 head (of 32), the first 65536 positions (of 131072) as a ring of 4, documents + bias, "
                      "fwd+bwd, FLOP of unmasked pairs, %.1f s" % dt}


# --------------------------------------------------------------------------- decode workload
def bench_decode(args, steps=0):
    import torch
    import ringattention_amd as ra
    dev = "cuda:0"
    B, H, D, kc = 16, 32, 128, 512
    Lf = args.seq_len or 262144
    L = Lf + kc
    k = torch.empty(B, L, H, D, dtype=torch.bfloat16, device=dev)
    v = torch.empty(B, L, H, D, dtype=torch.bfloat16, device=dev)
    g = torch.Generator(device=dev).manual_seed(0)
    for b in range(B):      # filled batch row by batch row to bound the fp32 temporaries
        k[b].copy_(torch.randn(L, H, D, device=dev, generator=g))
        v[b].copy_(torch.randn(L, H, D, device=dev, generator=g))
    q = torch.randn(B, 1, H, D, device=dev, generator=g).to(torch.bfloat16)
    out = torch.empty_like(q)
    kw = _kwargs(1, kc, 1)
    ci = torch.zeros(1, dtype=torch.int32, device=dev)
    state = {"t": 0}

    def step():
        ci.fill_(Lf + state["t"] % 64)      # one new token per step, read by the kernel from device memory
        state["t"] += 1
        ra.decode_attention(q, k, v, None, None, ci, kw, out=out)

    ms = _time_steps(step, args.steps, args.warmup)
    bytes_step = 2.0 * B * (Lf + 1) * H * D * 2
    value = bytes_step / (ms * 1e-3) / 1e9
    # events around the whole step: the fill of the position scalar, the split kernel and the combine pass that merges
    # its partials (0.05 GB); the split kernel is 98.9 % of that by the kernel trace
    kms = _event_ms(step, 5)
    ach = bytes_step / (kms * 1e-3) / 1e9
    cpu = None
    if not args.no_cpu:
        from oracle import ringattention_oracle as O
        cores = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(cores)
        Bc, Lc, steps_c = 2, 262144, 4
        gq = torch.Generator().manual_seed(0)
        qc_ = torch.randn(Bc, 1, H, D, generator=gq).to(torch.bfloat16)
        blk = torch.randn(1, 4096, H, D, generator=gq).to(torch.bfloat16)        # one random slab, tiled:
        kc_ = blk.repeat(Bc, (Lc + kc) // 4096 + 1, 1, 1)[:, :Lc + kc].contiguous()   # values do not matter for timing
        vc_ = kc_.flip(1).contiguous()
        t0 = time.perf_counter()
        for t_ in range(steps_c):
            O.ring_attention(qc_, kc_, vc_, None, None, Lc + 1 + t_, 1, True, _kwargs(1, kc, 1))
        dt = time.perf_counter() - t0
        cpu = {"value": round(steps_c * 2.0 * Bc * (Lc + 2) * H * D * 2 / dt / 1e9, 3), "unit": "GB/s", "cores": cores,
               "kind": "port", "sample": "B=2 (of 16), full cache 262144, %d steps, %.1f s" % (steps_c, dt)}
    return {
        "metric": "decode_hbm_gbs", "value": round(value, 1), "unit": "GB/s", "ms_per_step": round(ms, 3),
        "dtype": "bf16", "pct_hbm_peak": round(100 * value / PEAK_HBM_GBS, 2),
        "steps": steps or args.steps,
        "config": {"workload": "decode", "B": B, "H": H, "D": D, "cache_len": Lf, "key_chunk_size": kc,
                   "query_chunk_size": 1, "bytes_per_step": bytes_step},
        "roofline": {"bound": "hbm", "kernel": "decode_split_kernel + decode_combine_kernel", "achieved": round(ach, 1),
                     "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(ach / PEAK_HBM_GBS, 4),
                     "scope": "algorithmic bytes of a step / events around the whole step on the launch stream "
                              "(position fill + split kernel + combine kernel)",
                     "traffic": (_measured(TRAFFIC_PROFILE, "traffic").get("decode_split_kernel")
                                 if (B, Lf) == (16, 262144) else None),
                     "traffic_source": "profiles/" + TRAFFIC_PROFILE},
        "cpu_baseline": cpu,
    }


# --------------------------------------------------------------------------- feed-forward workload
def bench_ffn(args):
    import torch
    import ringattention_amd as ra
    dev = "cuda:0"
    T, d, f, chunk = args.seq_len or 65536, 4096, 11008, 2048
    g = torch.Generator(device=dev).manual_seed(0)
    ff = ra.SwiGLU(d, f, device=dev)
    x = torch.randn(1, T, d, device=dev, generator=g).to(torch.bfloat16).requires_grad_(True)
    dy = torch.randn(1, T, d, device=dev, generator=g).to(torch.bfloat16)

    def step():
        x.grad = None
        for p in ff.parameters():
            p.grad = None
        y = ra.blockwise_feedforward(ff, x, chunk, policy=args.ffn_policy, launch_tokens=args.ffn_launch_tokens or None,
                                     weight_grad_chunks=args.ffn_weight_grad_chunks)
        y.backward(dy)

    ms = _time_steps(step, args.steps, args.warmup)
    kept = ra.feedforward._save_preactivations(args.ffn_policy)
    flops = 18.0 * T * d * f
    shared = None
    if not args.ffn_launch_tokens and not args.no_extras:
        # the same step with consecutive chunks sharing launches of 16384 tokens (same result, 1.8 GB of scratch)
        def step_shared():
            x.grad = None
            for p in ff.parameters():
                p.grad = None
            ra.blockwise_feedforward(ff, x, chunk, policy=args.ffn_policy, launch_tokens=16384,
                                     weight_grad_chunks=args.ffn_weight_grad_chunks).backward(dy)
        ms_sh = _time_steps(step_shared, args.steps, args.warmup)
        shared = {"tokens_per_launch": ra.feedforward._slab_tokens(chunk, T // chunk, 16384),
                  "ms_per_step": round(ms_sh, 3), "value": round(flops / (ms_sh * 1e-3) / 1e12, 2), "unit": "TFLOP/s"}
    value = flops / (ms * 1e-3) / 1e12
    # dominant kernel: the launch that computes a = x w1 and b = x w3 together over the tile columns of both (a third
    # of the step's time by the kernel trace), timed alone on one launch's tokens
    from ringattention_amd.feedforward import gemm_bf16_pair
    slab = ra.feedforward._slab_tokens(chunk, T // chunk, args.ffn_launch_tokens or None)
    xs = x.detach()[0, :slab]
    a_out = torch.empty(slab, f, dtype=torch.bfloat16, device=dev)
    b_out = torch.empty(slab, f, dtype=torch.bfloat16, device=dev)
    pair = lambda: gemm_bf16_pair(xs, ff.w1.detach(), ff.w3.detach(), a_out, b_out)
    gemm_ms = _event_ms(pair, 5)
    gemm_tf = 4.0 * slab * d * f / (gemm_ms * 1e-3) / 1e12
    # the tile kernel the library picks for the pair (slab, 2 f): 256 x 256 or 256 x 128 over four wavefronts, whichever
    # takes fewer rounds of 256 CUs weighted by the cost of a round (1.72 : 1); the shapes here divide both
    r256 = math.ceil((slab // 256) * (2 * f // 256) / 256.0) * 1.72
    r128 = math.ceil((slab // 256) * (2 * f // 128) / 256.0) * 1.0
    gemm_name = "gemm_bf16_w4_kernel<false, false, %d>" % (256 if r256 <= r128 else 128)
    sclk = None if args.no_extras else _sclk_under_load(pair)
    cpu = None
    if not args.no_cpu:
        from oracle import ringattention_oracle as O
        cores = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(cores)
        Tc = 2048
        gc = torch.Generator().manual_seed(0)
        xc = torch.randn(1, Tc, d, generator=gc, requires_grad=True)
        w1, w3 = (torch.randn(d, f, generator=gc) * 0.02).requires_grad_(True), (torch.randn(d, f, generator=gc) * 0.02).requires_grad_(True)
        w2 = (torch.randn(f, d, generator=gc) * 0.02).requires_grad_(True)
        t0 = time.perf_counter()
        y = O.blockwise_feedforward(lambda h_: O.swiglu(h_, w1, w2, w3), xc, Tc)
        y.backward(torch.ones_like(y))
        dt = time.perf_counter() - t0
        cpu = {"value": round(18.0 * Tc * d * f / dt / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
               "sample": "one chunk of 2048 tokens (of 65536), fwd+bwd fp32, %.1f s" % dt}
    return {
        "metric": "swiglu_ffn_fwd_bwd_tflops", "value": round(value, 2), "unit": "TFLOP/s", "ms_per_step": round(ms, 3),
        "dtype": "bf16", "pct_bf16_mfma_peak": round(100 * value / PEAK_BF16_TFLOPS, 2),
        "config": {"workload": "ffn", "tokens": T, "hidden": d, "intermediate": f, "chunk_size": chunk,
                   "tokens_per_launch": slab, "weight_grad_chunks": args.ffn_weight_grad_chunks,
                   "policy": args.ffn_policy, "preactivations": "kept (%.1f GB)" % (4e-9 * T * f) if kept else "recomputed",
                   "flop_convention": "6*T*d*f fwd + 12*T*d*f bwd, recompute not counted"},
        "launch_tokens_16384": shared,
        "roofline": {"bound": "mfma", "kernel": "%s (a = x w1 and b = x w3 of one launch of %d tokens)" % (gemm_name, slab),
                     "achieved": round(gemm_tf, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(gemm_tf / PEAK_BF16_TFLOPS, 4),
                     "traffic": (_measured(TRAFFIC_PROFILE, "traffic").get(
                                     "gemm_bf16_w4_kernel<false,false,256>" if slab == 16384
                                     else "ffn2048:gemm_bf16_w4_kernel<false,false,256>")
                                 if T == 65536 and slab in (2048, 16384) else None),
                     "traffic_source": "profiles/" + TRAFFIC_PROFILE,
                     "mfma_util_pmc": {"kernel": (_measured(MFMA_PROFILE, "mfma_util").get(
                                           "gemm_bf16_w4_kernel<false,false,256>" if slab == 16384
                                           else "ffn2048:gemm_bf16_w4_kernel<false,false,256>")
                                                  if T == 65536 and slab in (2048, 16384) else None),
                                       "source": "profiles/" + MFMA_PROFILE},
                     "kernel_ms": {gemm_name: round(gemm_ms, 3)},
                     "power_w_under_load": sclk.pop("power_w", None) if sclk else None,
                     "sclk_mhz_under_load": sclk,
                     "frac_of_peak_at_sclk": (round(gemm_tf / (PEAK_BF16_TFLOPS * sclk["median"] / 2400.0), 4)
                                              if sclk else None)},
        "cpu_baseline": cpu,
    }


# --------------------------------------------------------------------------- steps either side of the path
def bench_decode_step(args):
    """A decode step as a model runs it: rotate + append the new token at cache_idx, then attend over the cache."""
    import torch
    import ringattention_amd as ra
    dev = "cuda:0"
    B, H, D, kc = 16, 32, 128, 512
    Lf = args.seq_len or 262144
    L = Lf + kc
    k = torch.empty(B, L, H, D, dtype=torch.bfloat16, device=dev)
    v = torch.empty(B, L, H, D, dtype=torch.bfloat16, device=dev)
    g = torch.Generator(device=dev).manual_seed(0)
    for b in range(B):
        k[b].copy_(torch.randn(L, H, D, device=dev, generator=g))
        v[b].copy_(torch.randn(L, H, D, device=dev, generator=g))
    q, kn, vn = (torch.randn(B, 1, H, D, device=dev, generator=g).to(torch.bfloat16) for _ in range(3))
    qr, out = torch.empty_like(q), torch.empty_like(q)
    kw = _kwargs(1, kc, 1)
    ci = torch.zeros(1, dtype=torch.int32, device=dev)
    state = {"t": 0}

    def prologue():
        ra.rope_kv_append(q, kn, vn, k, v, ci, q_out=qr)

    def step():
        ci.fill_(Lf + state["t"] % 64)
        state["t"] += 1
        prologue()
        ra.decode_attention(qr, k, v, None, None, ci, kw, out=out)

    ms = _time_steps(step, args.steps, args.warmup)
    bytes_step = 2.0 * B * (Lf + 1) * H * D * 2
    value = bytes_step / (ms * 1e-3) / 1e9
    pro_ms = _event_ms(prologue, 20)
    pro_bytes = 7.0 * B * H * D * 2          # q, k_new, v_new in; q_out, cache K and V rows out
    cpu = None
    if not args.no_cpu:
        from oracle import ringattention_oracle as O
        gq = torch.Generator().manual_seed(0)
        qc_, knc, vnc = (torch.randn(B, 1, H, D, generator=gq) for _ in range(3))
        kcc, vcc = torch.zeros(B, 64, H, D), torch.zeros(B, 64, H, D)
        t0 = time.perf_counter()
        reps = 200
        for _ in range(reps):
            O.rope_kv_append(qc_, knc, vnc, kcc, vcc, 37)
        dt = time.perf_counter() - t0
        cpu = {"value": round(reps / dt, 1), "unit": "prologues/s", "cores": 1, "kind": "port",
               "sample": "rotate + append of B=16 H=32 D=128 into a 64-position buffer, %d calls, %.2f s" % (reps, dt)}
    return {
        "metric": "decode_step_hbm_gbs", "value": round(value, 1), "unit": "GB/s", "ms_per_step": round(ms, 3),
        "dtype": "bf16", "pct_hbm_peak": round(100 * value / PEAK_HBM_GBS, 2),
        "config": {"workload": "decode_step", "B": B, "H": H, "D": D, "cache_len": Lf, "key_chunk_size": kc,
                   "rope_theta": 10000.0, "bytes_per_step": bytes_step},
        "roofline": {"bound": "hbm", "kernel": "rope_kv_append_kernel", "achieved": round(pro_bytes / (pro_ms * 1e-3) / 1e9, 2),
                     "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(pro_bytes / (pro_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 6),
                     "traffic": None, "kernel_ms": {"rope_kv_append_kernel": round(pro_ms, 4)},
                     "note": "917 KB per call: the launch, not the memory system, bounds this kernel"},
        "cpu_baseline": cpu,
    }


def bench_rmsnorm(args):
    """residual add + RMSNorm, forward and backward, over the FFN workload's activations (65536 x 4096, bf16)."""
    import torch
    import ringattention_amd as ra
    dev = "cuda:0"
    T, d = args.seq_len or 65536, 4096
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(1, T, d, device=dev, generator=g).to(torch.bfloat16).requires_grad_(True)
    r = torch.randn(1, T, d, device=dev, generator=g).to(torch.bfloat16).requires_grad_(True)
    w = torch.ones(d, device=dev, dtype=torch.bfloat16).requires_grad_(True)
    dn = torch.randn(1, T, d, device=dev, generator=g).to(torch.bfloat16)
    dres = torch.randn(1, T, d, device=dev, generator=g).to(torch.bfloat16)

    def fwd():
        return ra.rmsnorm_residual(x, r, w)

    def step():
        x.grad = r.grad = w.grad = None
        y, n = fwd()
        torch.autograd.backward((y, n), (dres, dn))

    ms = _time_steps(step, args.steps, args.warmup)
    bytes_step = 8.0 * T * d * 2            # forward: x, r in, y, n out; backward: dn, y, dres in, dy out
    value = bytes_step / (ms * 1e-3) / 1e9
    with torch.no_grad():
        f_ms = _event_ms(fwd, 5)
    ach = 4.0 * T * d * 2 / (f_ms * 1e-3) / 1e9
    cpu = None
    if not args.no_cpu:
        from oracle import ringattention_oracle as O
        cores = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(cores)
        Tc = 8192
        gc = torch.Generator().manual_seed(0)
        xc = torch.randn(Tc, d, generator=gc, requires_grad=True)
        rc = torch.randn(Tc, d, generator=gc, requires_grad=True)
        wc = torch.ones(d, requires_grad=True)
        t0 = time.perf_counter()
        reps = 5
        for _ in range(reps):
            yc, nc = O.rmsnorm_residual(xc, rc, wc)
            (yc.sum() + nc.sum()).backward()
        dt = time.perf_counter() - t0
        cpu = {"value": round(reps * 8.0 * Tc * d * 2 / dt / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": "8192 rows (of 65536), fwd+bwd fp32, %d repeats, %.1f s; bytes counted as for bf16" % (reps, dt)}
    return {
        "metric": "rmsnorm_residual_fwd_bwd_gbs", "value": round(value, 1), "unit": "GB/s", "ms_per_step": round(ms, 3),
        "dtype": "bf16", "pct_hbm_peak": round(100 * value / PEAK_HBM_GBS, 2),
        "config": {"workload": "rmsnorm", "tokens": T, "hidden": d, "bytes_per_step": bytes_step},
        "roofline": {"bound": "hbm", "kernel": "rmsnorm_fwd_kernel", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(ach / PEAK_HBM_GBS, 4),
                     "traffic": _measured(TRAFFIC_PROFILE, "traffic").get("rmsnorm_fwd_kernel") if T == 65536 else None,
                     "kernel_ms": {"rmsnorm_fwd_kernel": round(f_ms, 4)}},
        "cpu_baseline": cpu,
    }


# --------------------------------------------------------------------------- calibration copy
def bench_copy(args):
    """A plain 1 GiB device-to-device copy: the kernel of known size that the FETCH_SIZE / WRITE_SIZE
    counters of a ``rocprofv3 --pmc`` run are scaled by (it reads and writes exactly 2**30 bytes)."""
    import torch
    n = 1 << 28
    src = torch.empty(n, dtype=torch.float32, device="cuda:0").normal_()
    dst = torch.empty_like(src)
    ms = _time_steps(lambda: dst.copy_(src), args.steps, args.warmup)
    gbs = 2.0 * n * 4 / (ms * 1e-3) / 1e9
    return {"metric": "device_copy_gbs", "value": round(gbs, 1), "unit": "GB/s", "ms_per_step": round(ms, 3),
            "dtype": "u8", "config": {"workload": "copy", "bytes_read": n * 4, "bytes_written": n * 4},
            "roofline": {"bound": "hbm", "kernel": "copyBuffer", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": 2.0 * n * 4},
            "cpu_baseline": None}


# --------------------------------------------------------------------------- boolean-mask ring (inference twin)
def bench_inference(args):
    """ring_attention_inference on a causal + key-padding boolean mask, forward + backward, bf16 inputs,
    2 virtual shards: the MFMA kernels with the mask in packed form (ra_keep_pack, inside the timed step)."""
    import torch
    import ringattention_amd as ra
    dev = "cuda:0"
    B, H, D, n = 1, 32, 128, 2
    S = args.seq_len or 32768
    g = torch.Generator(device=dev).manual_seed(0)
    mk = lambda: (torch.randn(B, S, H, D, device=dev, generator=g) * D ** -0.5).to(torch.bfloat16)
    q, k, v = mk().requires_grad_(True), mk().requires_grad_(True), mk().requires_grad_(True)
    do = torch.randn(B, S, H, D, device=dev, generator=g).to(torch.bfloat16)
    mask = torch.tril(torch.ones(S, S, dtype=torch.bool, device=dev))
    mask[:, S - S // 16:] = False                      # the last sixteenth of the keys is padding
    mask[:, 0] = True
    mask = mask.reshape(1, 1, S, S)
    pairs = float(mask.sum().item())

    def step():
        q.grad = k.grad = v.grad = None
        with ra.ring_axis("sp", n):
            out = ra.ringattention_inference(q, k, v, mask, "sp", True)
            out.backward(do)

    ms = _time_steps(step, args.steps, args.warmup)
    flops = 14.0 * D * pairs * B * H
    value = flops / (ms * 1e-3) / 1e12
    return {"metric": "inference_attn_fwd_bwd_tflops", "value": round(value, 2), "unit": "TFLOP/s",
            "ms_per_step": round(ms, 3), "dtype": "bf16", "pct_bf16_mfma_peak": round(100 * value / PEAK_BF16_TFLOPS, 2),
            "config": {"workload": "inference", "B": B, "H": H, "S": S, "D": D, "virtual_ring": n,
                       "mask": "causal and 1/16 key padding, boolean (1,1,S,S)",
                       "flop_convention": "4*D fwd + 10*D bwd per attended (q,k) pair per head"},
            "roofline": {"bound": "mfma", "kernel": "attn_fwd_ws_kernel + attn_bwd_dkv_ws_kernel + attn_bwd_dq_ws_kernel "
                                                    "(packed boolean mask), whole step",
                         "achieved": round(value, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(value / PEAK_BF16_TFLOPS, 4), "traffic": None},
            "cpu_baseline": None}


def bench_vendor_sdpa(args):
    """The attn32k shape through torch's scaled_dot_product_attention (the fused attention kernels the ROCm build of
    PyTorch ships), timed the same way: a yardstick measured on the same box, not part of the library."""
    import torch
    import torch.nn.functional as F
    from torch.nn.attention import sdpa_kernel, SDPBackend
    dev = "cuda:0"
    B, H, S, D = args.batch or 1, 32, args.seq_len or 32768, 128
    g = torch.Generator(device=dev).manual_seed(0)
    q, k, v = ((torch.randn(B, H, S, D, device=dev, generator=g) / D ** 0.5).to(torch.bfloat16).requires_grad_(True)
               for _ in range(3))
    do = torch.randn(B, H, S, D, device=dev, generator=g).to(torch.bfloat16)
    flops = 14.0 * D * (S * (S + 1) / 2.0) * B * H
    res = {}
    for name, be in (("flash", SDPBackend.FLASH_ATTENTION), ("efficient", SDPBackend.EFFICIENT_ATTENTION)):
        try:
            with sdpa_kernel(be):
                def step():
                    q.grad = k.grad = v.grad = None
                    F.scaled_dot_product_attention(q, k, v, is_causal=True).backward(do)

                def fwd():
                    with torch.no_grad():
                        F.scaled_dot_product_attention(q, k, v, is_causal=True)
                ms = _time_steps(step, args.steps, args.warmup)
                ms_f = _time_steps(fwd, args.steps, args.warmup)
            res[name] = {"ms_per_step": round(ms, 3), "tflops": round(flops / (ms * 1e-3) / 1e12, 1),
                         "fwd_ms": round(ms_f, 3)}
        except Exception as e:                     # a backend this build does not have
            res[name] = {"error": repr(e)[:200]}
    ok = [r for r in res.values() if "ms_per_step" in r]
    if not ok:
        raise RuntimeError("no fused attention backend of torch ran: %r" % res)
    best = min(ok, key=lambda r: r["ms_per_step"])
    return {"metric": "vendor_sdpa_fwd_bwd_tflops", "value": best["tflops"], "unit": "TFLOP/s",
            "ms_per_step": best["ms_per_step"], "dtype": "bf16",
            "config": {"workload": "vendor_sdpa", "B": B, "H": H, "S": S, "D": D, "is_causal": True, "backends": res,
                       "flop_convention": "4*D fwd + 10*D bwd per unmasked (q,k) pair per head"},
            "roofline": None, "cpu_baseline": None}


def bench_mfma_probe(args):
    """What the matrix pipes sustain on bf16 MFMAs alone, by operand activity (ra_mfma_rate_probe): the rate, the
    clock and the board power of a two-second run each.  The value is the rate on random operands: the ceiling a
    bf16 kernel on real data has on this board, next to the published peak."""
    import torch
    from ringattention_amd import _lib as L
    dev = "cuda:0"
    wgs, iters = 256, 8192                      # one workgroup per CU, 64 * iters MFMAs per wavefront
    sink = torch.empty(wgs * 256, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    flop = wgs * 4 * iters * 64 * 32768.0
    rows = {}
    for mode, name in ((0, "one value everywhere"), (1, "a value per lane, constant in time"), (2, "random operands")):
        fn = lambda: L.check(L.load_probe().ra_mfma_rate_probe(sink.data_ptr(), wgs, iters, mode, stream), "ra_mfma_rate_probe")
        fn()
        torch.cuda.synchronize()
        clk = _sclk_under_load(fn, seconds=2.5)
        ms = _event_ms(fn, 10)
        rows[name] = {"tflops": round(flop / (ms * 1e-3) / 1e12, 1), "ms": round(ms, 3),
                      "power_w": clk.pop("power_w", None) if clk else None, "sclk_mhz": clk}
        time.sleep(1.0)
    value = rows["random operands"]["tflops"]
    return {"metric": "mfma_only_tflops", "value": value, "unit": "TFLOP/s", "ms_per_step": rows["random operands"]["ms"],
            "dtype": "bf16", "pct_bf16_mfma_peak": round(100 * value / PEAK_BF16_TFLOPS, 2),
            "config": {"workload": "mfma_probe", "workgroups": wgs, "mfma_per_wavefront": iters * 64,
                       "instruction": "v_mfma_f32_32x32x16_bf16", "by_operands": rows},
            "roofline": {"bound": "mfma", "kernel": "mfma_probe_kernel", "achieved": value, "peak": PEAK_BF16_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(value / PEAK_BF16_TFLOPS, 4), "traffic": None},
            "cpu_baseline": None}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default=None, choices=["attn32k", "ring131k", "ffn", "decode", "inference", "copy", "decode_step", "rmsnorm",
                                                              "dropout32k", "c1", "mfma_probe", "vendor_sdpa"])
    ap.add_argument("--seq-len", type=int, default=0, help="override the sequence / cache / token length")
    ap.add_argument("--batch", type=int, default=0, help="attention workloads: batch rows (the configurations have 1)")
    ap.add_argument("--head-dim", type=int, default=0, choices=[0, 64, 128, 256],
                    help="attention workloads: head size (the number of heads follows, H * D = 4096)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"],
                    help="attention workloads: dtype of q, k, v (fp32 runs on v_mfma_f32_32x32x2_f32; its roofline is the "
                         "fp32 matrix peak)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--ffn-policy", default="nothing_saveable", choices=["nothing_saveable", "save_preactivations"],
                    help="ffn workload: what blockwise_feedforward keeps for the backward pass (default: the "
                         "reference's, nothing: the pre-activations are recomputed)")
    ap.add_argument("--ffn-launch-tokens", type=int, default=0,
                    help="ffn workload: let consecutive chunks share a launch of up to this many tokens (default: one "
                         "chunk per launch, as the reference's scan)")
    ap.add_argument("--ffn-weight-grad-chunks", type=int, default=4,
                    help="ffn workload: chunks whose weight-gradient products share a launch in the backward pass "
                         "(blockwise_feedforward's default is 4; 1 = one launch per chunk)")
    ap.add_argument("--inputs", default="baseline", choices=["baseline", "d-quarter", "unit"],
                    help="attention workloads: scale of q and k (baseline = N(0,1)/sqrt(D), the configuration's)")
    ap.add_argument("--no-extras", action="store_true",
                    help="default workload only: skip the decode leg and the other-inputs timings of the JSON line")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the ring is virtual); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    # no --workload: the whole headline metric in one line - the 32K attention step is the value; the decode leg
    # (B16, 262144 positions, 64 steps) and the same attention step on other input scales ride along as sub-objects
    whole_metric = args.workload is None and not args.no_extras and not args.seq_len and not args.batch
    if args.workload is None:
        args.workload = "attn32k"
    extras = {}
    if args.workload in ("attn32k", "ring131k", "dropout32k", "c1"):
        r = bench_attention(args, ring=(args.workload == "ring131k"), dropout=(args.workload == "dropout32k"),
                            c1=(args.workload == "c1"))
        if whole_metric:
            others = []
            for inputs in ("d-quarter", "unit"):
                a2 = argparse.Namespace(**dict(vars(args), inputs=inputs, no_cpu=True))
                r2 = bench_attention(a2, ring=False)
                others.append({"inputs": r2["config"]["inputs"], "value": r2["value"], "unit": r2["unit"],
                               "ms_per_step": r2["ms_per_step"], "kernel_ms": r2["roofline"]["kernel_ms"]})
            extras["other_inputs"] = others
            # the rate of the matrix pipes on MFMAs alone, same board, same run: what "peak" means for real data here
            pr = bench_mfma_probe(args)
            extras["mfma_probe"] = {"metric": pr["metric"], "value": pr["value"], "unit": pr["unit"],
                                    "by_operands": pr["config"]["by_operands"]}
            if r.get("roofline") and pr["value"]:
                r["roofline"]["frac_of_mfma_only_rate_on_random_operands"] = round(
                    r["roofline"]["achieved"] / pr["value"], 4)
            # the reference's own CPU-runnable configuration (fp32, on the fp32 matrix-core kernels) next to the CPU
            # oracle timed on the whole of it
            c1 = bench_attention(argparse.Namespace(**dict(vars(args), steps=50, warmup=5)), ring=False, c1=True)
            extras["c1"] = {k_: c1[k_] for k_ in ("metric", "value", "unit", "ms_per_step", "dtype", "config",
                                                    "roofline", "cpu_baseline")}
            torch.cuda.empty_cache()
            d = bench_decode(args, steps=64)
            extras["decode"] = {k_: d[k_] for k_ in ("metric", "value", "unit", "steps", "ms_per_step", "dtype",
                                                     "pct_hbm_peak", "config", "roofline", "cpu_baseline")}
            # the other two configurations: the virtual ring of eight over 131072 positions with packed documents and a
            # bias, and the SwiGLU feed-forward over 65536 tokens (one chunk per launch, and 16384 tokens per launch)
            torch.cuda.empty_cache()
            rg = bench_attention(argparse.Namespace(**dict(vars(args), no_extras=True, steps=3, warmup=1)), ring=True)
            extras["ring131k"] = {k_: rg[k_] for k_ in ("metric", "value", "unit", "ms_per_step", "dtype", "config",
                                                        "roofline", "cpu_baseline")}
            torch.cuda.empty_cache()
            ff = bench_ffn(argparse.Namespace(**dict(vars(args), steps=3, warmup=1)))
            extras["ffn"] = {k_: ff[k_] for k_ in ("metric", "value", "unit", "ms_per_step", "dtype", "config",
                                                   "launch_tokens_16384", "roofline", "cpu_baseline")}
    elif args.workload == "decode":
        r = bench_decode(args)
    elif args.workload == "copy":
        r = bench_copy(args)
    elif args.workload == "decode_step":
        r = bench_decode_step(args)
    elif args.workload == "rmsnorm":
        r = bench_rmsnorm(args)
    elif args.workload == "inference":
        r = bench_inference(args)
    elif args.workload == "mfma_probe":
        r = bench_mfma_probe(args)
    elif args.workload == "vendor_sdpa":
        r = bench_vendor_sdpa(args)
    else:
        r = bench_ffn(args)
    line = {"metric": r["metric"], "value": r["value"], "unit": r["unit"], "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": r["dtype"], "data": "synthetic", "config": r["config"],
            "roofline": r["roofline"], "cpu_baseline": r["cpu_baseline"]}
    for extra in ("pct_bf16_mfma_peak", "pct_f32_mfma_peak", "pct_hbm_peak", "launch_tokens_16384"):
        if extra in r:
            line[extra] = r[extra]
    line.update(extras)
    # give the device memory back before the line goes out: whoever reads the line may look at the GPU right away
    import gc
    gc.collect()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
