"""Headline benchmark: TimestepNorm -> complex EMA block (Mega2), B=4, L=4096, D=1024, N=16,
bf16 activations, fp32 parameters and accumulation, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step = one forward of the block over one batch of synthetic input that already sits in
HBM: xn = TimestepNorm(x) ([B, L, D], 16 groups), y = CEMA(xn^T), both results written (the layer
needs xn for its value projection), y as the contiguous [B, D, L] tensor the reference's convolution
returns.  The timed step is one library call (one kernel); the same block as two module calls and
the step with the kernel generation inside the call are timed beside it.  Inputs rotate over several
buffers so that a step never finds its input in the 256 MB last-level cache.  Prints one JSON line
(tokens/s of the whole job), with the HBM roofline of the dominant kernel and the CPU oracle timed
on the host cores beside it.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

B, L, D, N, G = 4, 4096, 1024, 16, 16
HBM_PEAK_GBS = 8000.0
NBUF = 8


def make_params(rng):
    import numpy as np

    alpha = rng.normal(0, 0.2, (D, N, 1))
    delta = rng.normal(0, 0.2, (D, N, 1))
    th = rng.uniform(0.0, np.pi, (D, 1, 1)).clip(1e-3, np.pi - 1e-3)
    frac = th / (2 * np.pi)
    theta = np.log(frac / (1 - frac))
    gamma = np.zeros((D, N, 2))
    gamma[..., 0] = rng.normal(0, 1.0, (D, N))
    omega = rng.normal(0, 1.0, (D, 1))
    return alpha, delta, theta, gamma, omega


def cpu_baseline(params, x_bf16_as_f32, threads):
    """The oracle timed on the host cores: the reference's CPU algorithm for the same block
    (two-stage Welford TimestepNorm loops in C, kernel generation by exp(l log q) in C, the
    zero-padded real-FFT convolution of fused_ops/fftconv.py:45-61 through scipy's pocketfft)."""
    import numpy as np
    import scipy.fft as sfft

    import oracle_c_api as OC
    from oracle import mega_oracle as O

    alpha, delta, theta, gamma, omega = params
    p, q, g = O.ema_coeffs_complex(alpha, delta, theta, gamma, dtype=np.float32)
    x = x_bf16_as_f32
    ones, zeros = np.ones(D, np.float32), np.zeros(D, np.float32)

    def run():
        xn, _, _, _ = OC.timestep_norm(x, np.zeros(B, np.int64), np.zeros((B, G), np.float32),
                                       np.ones((B, G), np.float32), ones, zeros, None, G, 1e-5, np.float32)
        k = OC.ema_kernel(p, q, g, L, np.float32)
        xt = np.ascontiguousarray(xn.transpose(0, 2, 1))
        n2 = 2 * O.pow2ceil(L)
        x_f = sfft.rfft(xt, n=n2, workers=threads)
        k_f = sfft.rfft(k, n=n2, workers=threads) / n2
        y = sfft.irfft(x_f * k_f, n=n2, workers=threads)[..., :L] * n2
        y = y + omega.reshape(1, D, 1).astype(np.float32) * xt
        return y

    run()
    times = []
    t_end = time.time() + 20.0
    while len(times) < 3 or (time.time() < t_end and len(times) < 10):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    return {"value": B * L / t, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"the full B{B}xL{L}xD{D} block, median of {len(times)} runs ({t * 1e3:.0f} ms each)"}


def measured_traffic():
    """HBM bytes per launch from the committed rocprofv3 --pmc summary (FETCH_SIZE / WRITE_SIZE scaled
    by a plain copy of known size): lines `traffic_bytes_per_launch <kernel> = <bytes>`."""
    import re

    out = {}
    path = os.path.join(ROOT, "profiles", "ema_tsn_block_B4_L4096_D1024_bf16.txt")
    if os.path.exists(path):
        for m in re.finditer(r"^traffic_bytes_per_launch\s+(\S+)\s*=\s*(\d+)", open(path).read(), re.M):
            out[m.group(1)] = int(m.group(2))
    return out


def profiled_durations():
    """Average kernel durations (ms) of the committed rocprofv3 --kernel-trace --stats summary of this
    command: lines `avg_duration_us <kernel> = <microseconds>`."""
    import re

    out = {}
    path = os.path.join(ROOT, "profiles", "ema_tsn_block_B4_L4096_D1024_bf16.txt")
    if os.path.exists(path):
        for m in re.finditer(r"^avg_duration_us\s+(\S+)\s*=\s*([0-9.]+)", open(path).read(), re.M):
            out[m.group(1)] = float(m.group(2)) * 1e-3
    return out


def best_region(run, steps, regions=3):
    """(device ms, wall ms, host-enqueue ms) per step of the median of `regions` timed regions of exactly `steps` calls
    run(i), each bracketed by a device synchronisation on both sides (HIP events on the launch stream inside).  Once
    per process, at no fixed step, the runtime stalls one launch on the host for tens of milliseconds; a single
    region would report that stall as step time."""
    import torch

    out = []
    for _ in range(regions):
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        a.record()
        for i in range(steps):
            run(i)
        b.record()
        host = time.perf_counter() - t0
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        out.append((a.elapsed_time(b) / steps, wall * 1e3 / steps, host * 1e3 / steps))
    return sorted(out, key=lambda r: max(r[0], r[1]))[len(out) // 2]


def bench_decode(args):
    """configs[3]: B = 64 streams, D = 2048, N = 16, 16 norm groups: one fused TimestepNorm + EMA decode
    step per token (state-traffic bound: the complex64 state h[B, D, N] is read and written once)."""
    import numpy as np
    import torch

    import fairseq_apollo_amd as M

    Bd, Dd, Nd, Gd = 64, 2048, 16, 16
    dev = torch.device("cuda:0")
    torch.manual_seed(1237)
    ema = M.MultiHeadComplexEMA(Dd, ndim=Nd).to(dev).eval()          # the module's own initialisation
    with torch.no_grad():
        p, q, g = ema.coeffs()
        step = M.ops.DecodeStep(torch.randn(Dd, device=dev) * 0.1, torch.randn(Dd, device=dev) * 0.1, Gd, 1e-5,
                                p.squeeze(-1), q.squeeze(-1), g, ema.omega.reshape(-1), Bd)
    xs = [torch.randn(Bd, Dd, device=dev).to(torch.bfloat16) for _ in range(16)]
    with torch.no_grad():
        for i in range(args.warmup):
            step(xs[i % 16])
        dev_ms, wall_ms, host_ms = best_region(lambda i: step(xs[i % 16]), args.steps)
    ms = max(wall_ms, dev_ms)
    host = host_ms * 1e-3 * args.steps
    alg = 2 * Bd * Dd * Nd * 8 + 3 * Bd * Dd * 2 + 4 * Bd * Gd * 4
    gbs = alg / (dev_ms * 1e-3) / 1e9
    # K tokens of every stream per launch (chunk-wise streaming of given inputs, not autoregressive
    # generation): the state crosses HBM once per launch
    multi = {}
    with torch.no_grad():
        for K in (4, 16, 64):
            chunks = [torch.randn(Bd, K, Dd, device=dev).to(torch.bfloat16) for _ in range(4)]
            n = max(20, args.steps // 4)
            for i in range(5):
                step.steps(chunks[i % 4])
            dev_k, wall_k, _ = best_region(lambda i: step.steps(chunks[i % 4]), n)
            alg_k = 2 * Bd * Dd * Nd * 8 + 3 * Bd * K * Dd * 2 + 4 * Bd * Gd * 4
            multi[f"K={K}"] = {"ms_per_launch": max(wall_k, dev_k), "device_ms_per_launch": dev_k,
                               "tokens_per_s": Bd * K / (max(wall_k, dev_k) * 1e-3),
                               "hbm_gbs": alg_k / (dev_k * 1e-3) / 1e9, "algorithmic_bytes_per_launch": alg_k}
    print(json.dumps({
        "metric": "decode tokens/sec @B64xD2048, fused TimestepNorm + EMA step", "value": Bd / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[3]: 64 streams, D=2048, N=16 complex, 16 norm groups, one token per step"},
        "roofline": {"bound": "hbm", "kernel": "norm_ema_step_kernel", "achieved": gbs, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes_per_launch": alg, "avg_ms": dev_ms, "host_enqueue_ms": host * 1e3 / args.steps},
        "tokens_per_launch": multi,
    }))


def bench_block_bwd(args):
    """Backward of the headline block at configs[2]'s shape: moving-average backward (input
    gradient + parameter-gradient sums) followed by the TimestepNorm backward, per operator with HIP
    events around back-to-back launches."""
    import torch

    import fairseq_apollo_amd as M

    dev = torch.device("cuda:0")
    torch.manual_seed(1237)
    ema = M.MultiHeadComplexEMA(D, ndim=N).to(dev).eval()
    with torch.no_grad():
        p, q, g = ema.coeffs()
        layer = M.ops.PreparedEMA(p.squeeze(-1), q.squeeze(-1), g, ema.omega.reshape(-1))
    gamma = torch.randn(D, device=dev) * 0.1 + 1.0
    beta = torch.randn(D, device=dev) * 0.1
    pc = torch.zeros(B, dtype=torch.int64, device=dev)
    pm = torch.zeros(B, G, device=dev)
    pv = torch.ones(B, G, device=dev)
    nbuf = 4
    xs = [torch.randn(B, L, D, device=dev).to(torch.bfloat16) for _ in range(nbuf)]
    dys = [torch.randn(B, L, D, device=dev).to(torch.bfloat16) for _ in range(nbuf)]
    saved = []
    with torch.no_grad():
        for x in xs:
            xn, cnt, _, _, gm, cm, cr = M.ops.group_timestep_norm_fwd(x, pc, pm, pv, gamma, beta, None, G, 1e-5)
            saved.append((xn, cnt, gm, cm, cr))

    def ema_bwd(i):
        xn = saved[i % nbuf][0]
        return M.ops.ema_backward(dys[i % nbuf].transpose(1, 2), xn.transpose(1, 2), p.squeeze(-1), q.squeeze(-1), g,
                                  ema.omega.reshape(-1), None, layer=layer)

    def tsn_bwd(i, dxn):
        _, cnt, gm, cm, cr = saved[i % nbuf]
        return M.ops.group_timestep_norm_bwd(dxn, None, None, xs[i % nbuf], pm, cnt, gm, cm, cr, gamma, None, G)

    def timed(fn):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for i in range(args.steps):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / args.steps

    with torch.no_grad():
        dxn = None
        for i in range(max(args.warmup, 1)):
            dxn = ema_bwd(i)[0].transpose(1, 2)
            tsn_bwd(i, dxn)
        ms_ema = timed(ema_bwd)
        ms_tsn = timed(lambda i: tsn_bwd(i, dxn))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            tsn_bwd(i, ema_bwd(i)[0].transpose(1, 2))
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
    act = B * L * D * 2
    # algorithmic bytes: EMA backward reads dy twice (input gradient, sums) and x once, writes dx;
    # the norm backward reads dy and x once and writes dx (one launch: a tile keeps both for its dx)
    alg_ema, alg_tsn = 4 * act, 3 * act
    print(json.dumps({
        "metric": "backward tokens/sec @B4xL4096xD1024, CEMA backward + TimestepNorm backward", "value": B * L / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[2] shape, backward of TimestepNorm(16 groups) -> complex EMA (N=16)"},
        "kernels": {
            "ema_backward": {"avg_ms": ms_ema, "algorithmic_bytes": alg_ema, "GBps": alg_ema / (ms_ema * 1e-3) / 1e9},
            "group_timestep_norm_bwd": {"avg_ms": ms_tsn, "algorithmic_bytes": alg_tsn,
                                        "GBps": alg_tsn / (ms_tsn * 1e-3) / 1e9}},
        "roofline": {"bound": "hbm", "kernel": "ema_backward (adjoint + parameter sums)",
                     "achieved": alg_ema / (ms_ema * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": alg_ema / (ms_ema * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None},
    }))


def bench_seqnorm(args):
    """SequenceNorm (16 groups) at configs[2]'s activation shape, both layouts."""
    import torch

    import fairseq_apollo_amd as M

    dev = torch.device("cuda:0")
    torch.manual_seed(1237)
    gamma = torch.randn(D, device=dev) * 0.1 + 1.0
    beta = torch.randn(D, device=dev) * 0.1
    res = {}
    for name, last in (("blh", False), ("bhl", True)):
        xs = [torch.randn((B, D, L) if last else (B, L, D), device=dev).to(torch.bfloat16) for _ in range(NBUF)]
        for i in range(max(args.warmup, 1)):
            M.ops.group_sequence_norm_fwd(xs[i % NBUF], gamma, beta, None, G, 1e-5, last)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for i in range(args.steps):
            M.ops.group_sequence_norm_fwd(xs[i % NBUF], gamma, beta, None, G, 1e-5, last)
        b.record()
        torch.cuda.synchronize()
        res[name] = a.elapsed_time(b) / args.steps
    alg = 2 * B * L * D * 2              # x read once, y written once
    ms = res["bhl"]                      # the layout the reference module uses
    print(json.dumps({
        "metric": "SequenceNorm tokens/sec @B4xL4096xD1024 ([B, H, L], 16 groups)", "value": B * L / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "SequenceNorm(16 groups) at configs[2]'s activation shape"},
        "kernels": {"blh_ms": res["blh"], "bhl_ms": res["bhl"]},
        "roofline": {"bound": "hbm", "kernel": "seqnorm moments + combine + apply", "achieved": alg / (ms * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": None, "algorithmic_bytes_per_step": alg},
    }))


def bench_tsn_feature(args):
    """Per-feature TimestepNorm (every feature its own group) at configs[2]'s activation shape: the three kernels
    parallel over time tiles (rows this long are refused without a workspace)."""
    import torch

    import fairseq_apollo_amd as M

    dev = torch.device("cuda:0")
    torch.manual_seed(1238)
    gamma = torch.randn(D, device=dev) * 0.1 + 1.0
    beta = torch.randn(D, device=dev) * 0.1
    pc = torch.zeros(B, dtype=torch.int64, device=dev)
    pm = torch.zeros(B, D, device=dev)
    pv = torch.ones(B, D, device=dev)
    xs = [torch.randn(B, L, D, device=dev).to(torch.bfloat16) for _ in range(NBUF)]

    def timed(fn, n):
        for i in range(3):
            fn(i)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for i in range(n):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n

    par = timed(lambda i: M.ops.timestep_norm_fwd(xs[i % NBUF], pc, pm, pv, gamma, beta, None, 1e-5, need_stats=False),
                args.steps)
    # a training step of the same norm: the forward that also writes the running statistics, then the backward
    dys = [torch.randn(B, L, D, device=dev).to(torch.bfloat16) for _ in range(2)]
    saved = M.ops.timestep_norm_fwd(xs[0], pc, pm, pv, gamma, beta, None, 1e-5)
    fwd_stats = timed(lambda i: M.ops.timestep_norm_fwd(xs[i % NBUF], pc, pm, pv, gamma, beta, None, 1e-5), args.steps)
    bwd = timed(lambda i: M.ops.timestep_norm_bwd(dys[i % 2], None, None, xs[0], pm, saved[1], saved[4], saved[5], gamma,
                                                  None), args.steps)
    lib = M._lib.load()
    y = torch.empty_like(xs[0])
    cnt = torch.empty(B, dtype=torch.int64, device=dev)
    mean, var = torch.empty(B, D, device=dev), torch.empty(B, D, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    # without a workspace the entry point refuses rows this long (it used to fall back to one thread per feature)
    rc = lib.mega_timestep_norm_fwd(xs[0].data_ptr(), y.data_ptr(), 1, pc.data_ptr(), pm.data_ptr(), pv.data_ptr(),
                                    gamma.data_ptr(), beta.data_ptr(), None, B, L, D, 1e-5, cnt.data_ptr(),
                                    mean.data_ptr(), var.data_ptr(), None, None, None, 0, stream)
    assert rc == -3, rc
    alg = 2 * B * L * D * 2              # x read once, y written once
    print(json.dumps({
        "metric": "per-feature TimestepNorm tokens/sec @B4xL4096xD1024", "value": B * L / (par * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": par,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "TimestepNorm without groups (every feature its own statistics) at configs[2]'s activation shape"},
        "kernels": {"time_tiles_ms": par, "forward_with_saved_statistics_ms": fwd_stats, "backward_ms": bwd,
                    "backward_algorithmic_bytes": 3 * B * L * D * 2 + 2 * B * L * D * 4},
        "roofline": {"bound": "hbm", "kernel": "feature_tile_moments + feature_tile_scan + feature_tile_apply",
                     "achieved": alg / (par * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": alg / (par * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes_per_step": alg},
    }))


def bench_long_conv(args):
    """Explicit-kernel causal convolution (ops.fftconv) at configs[2]'s shape: x [B, D, L], k [D, L]."""
    import torch

    import fairseq_apollo_amd as M

    dev = torch.device("cuda:0")
    torch.manual_seed(1239)
    res = {}
    for name, dt in (("bf16", torch.bfloat16), ("f32", torch.float32)):
        xs = [torch.randn(B, D, L, device=dev).to(dt) for _ in range(4)]
        k = torch.randn(D, L, device=dev) * torch.exp(-torch.arange(L, device=dev) / 300.0)
        for i in range(3):
            M.ops.fftconv(xs[i % 4], k)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for i in range(args.steps):
            M.ops.fftconv(xs[i % 4], k)
        b.record()
        torch.cuda.synchronize()
        res[name] = a.elapsed_time(b) / args.steps
    ms = res["bf16"]
    alg = 2 * B * L * D * 2 + D * L * 4              # x read, y written, the kernel read once
    print(json.dumps({
        "metric": "explicit-kernel causal convolution tokens/sec @B4xD1024xL4096, Lk=4096", "value": B * L / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "fftconv(x, k) with a materialised kernel of L lags at configs[2]'s shape"},
        "kernels": {"bf16_ms": res["bf16"], "f32_ms": res["f32"]},
        "roofline": {"bound": "hbm", "kernel": "long_conv_fft_kernel", "achieved": alg / (ms * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": None, "algorithmic_bytes_per_step": alg,
                     "direct_form_flops": 2 * B * D * L * (L + 1) // 2},
    }))


def bench_ema_real(args):
    """configs[0] and configs[1]: the real MultiHeadEMA forward in fp32 on [B, D, L] rows (one-sided,
    B2 x D512 x L1024; two-sided with a right-padding mask, B1 x D256 x L16384).  The value is
    configs[1]'s; the CPU leg is the oracle's FFT convolution of the same call."""
    import numpy as np
    import torch

    import fairseq_apollo_amd as M
    from conftest import mega_init_real, rel_err
    from oracle import mega_oracle as O

    dev = torch.device("cuda:0")
    out = {}
    for name, (b, d, l, bidir, seed) in (("configs[0]", (2, 512, 1024, False, 1234)),
                                         ("configs[1]", (1, 256, 16384, True, 1235))):
        rng = np.random.default_rng(seed)
        K = 2 * d if bidir else d
        alpha, delta, beta, gamma = mega_init_real(rng, K, N)
        omega = rng.normal(0, 1.0, d)
        m = M.MultiHeadEMA(d, ndim=N, bidirectional=bidir).to(dev).eval()
        with torch.no_grad():
            for prm, v in ((m.alpha, alpha), (m.delta, delta), (m.beta, beta), (m.gamma, gamma), (m.omega, omega)):
                prm.copy_(torch.from_numpy(np.asarray(v, np.float32)).reshape(prm.shape))
        x = rng.normal(size=(b, d, l)).astype(np.float32)
        mask = None
        if bidir:
            mask = np.zeros((b, l), bool)
            for i in range(b):
                mask[i, l - int(rng.integers(0, l // 4 + 1)):] = True
        nbuf = 4
        xs = [torch.from_numpy(x).to(dev) for _ in range(nbuf)]
        tm = None if mask is None else torch.from_numpy(mask).to(dev)
        with torch.no_grad():
            for i in range(max(args.warmup, 1)):
                y = m(xs[i % nbuf], tm)
            regions = []                     # best of three timed regions (a one-off host stall spoils one at most)
            for _ in range(3):
                a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                a.record()
                for i in range(args.steps):
                    y = m(xs[i % nbuf], tm)
                e.record()
                torch.cuda.synchronize()
                regions.append(a.elapsed_time(e) / args.steps)
        ms = min(regions)
        # sixteen of the same call in one HIP graph (no Python and no launch calls on the host between them): tells
        # whether the host or the device bounds a call this small; the replay must reproduce the eager result
        graph_ms = None
        GC = 16
        with torch.no_grad():
            xg = xs[0].clone()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    m(xg, tm)
            torch.cuda.current_stream().wait_stream(side)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for _ in range(GC):
                    yg = m(xg, tm)
            g.replay()
            torch.cuda.synchronize()
            if torch.equal(yg, m(xg, tm)):
                reg = []
                for _ in range(3):
                    a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    torch.cuda.synchronize()
                    a.record()
                    for i in range(max(args.steps // GC, 1)):
                        g.replay()
                    e.record()
                    torch.cuda.synchronize()
                    reg.append(a.elapsed_time(e) / (max(args.steps // GC, 1) * GC))
                graph_ms = min(reg)
        p_, q_, g_ = O.ema_coeffs_real(alpha.astype(np.float32), delta.astype(np.float32), beta.astype(np.float32),
                                       gamma.astype(np.float32))
        cpu = None
        ref = None
        if not args.no_cpu:
            times = []
            for _ in range(3):
                t0 = time.perf_counter()
                ref, _ = O.ema_forward(x, p_, q_, g_, omega.astype(np.float32), padding_mask=mask, bidirectional=bidir)
                times.append(time.perf_counter() - t0)
            cpu = sorted(times)[1]
        alg = 2 * b * d * l * 4
        out[name] = {"ms": ms, "tokens_per_s": b * l / (ms * 1e-3), "algorithmic_bytes": alg,
                     "hbm_gbs": alg / (ms * 1e-3) / 1e9, "cpu_ms": None if cpu is None else cpu * 1e3,
                     "rel_err_vs_oracle": None if ref is None else rel_err(y.float().cpu().numpy(), ref),
                     "timed_regions_ms": regions, "graph_replay_ms": graph_ms,
                     "graph_replay_hbm_gbs": None if graph_ms is None else alg / (graph_ms * 1e-3) / 1e9}
    c1 = out["configs[1]"]
    line = {
        "metric": "real MultiHeadEMA forward tokens/sec @B1xL16384xD256 (bidirectional, fp32)",
        "value": c1["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": c1["ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]: bidirectional real MultiHeadEMA (N=16), B=1 L=16384 D=256, fp32, "
                               "right-padding mask; configs[0] beside it"},
        "roofline": {"bound": "hbm", "kernel": "ema_rows_kernel: block end states, then both directions of every block (matrix cores, fp16 terms)",
                     "achieved": c1["hbm_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": c1["hbm_gbs"] / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes_per_step": c1["algorithmic_bytes"]},
        "cases": out,
    }
    if c1["cpu_ms"] is not None:
        line["cpu_baseline"] = {"value": 16384 / (c1["cpu_ms"] * 1e-3), "unit": "tokens/s",
                                "cores": 1, "kind": "port",
                                "sample": "the whole configs[1] call through the oracle's numpy kernel generation "
                                          "and FFT convolution (fp64, one thread), median of 3"}
    print(json.dumps(line))


def bench_attention(args):
    """configs[4]'s attention: 4 chunks of 2048 tokens, 4 heads, H1 = 128, H2 = 1024, bf16, causal
    (matrix-core bound).  Flops are counted for the causal half only: 2 * C^2/2 * (H1 + H2) per chunk-head."""
    import torch

    import fairseq_apollo_amd as M

    Bc, C, Nh, H1, H2 = 4, 2048, 4, 128, 1024
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(1238)
    mk = lambda *sh: torch.randn(*sh, generator=gen).to(torch.bfloat16).to(dev)
    q, k, v = mk(Bc, C, Nh, H1), mk(Bc, C, Nh, H1), mk(Bc, C, Nh, H2)
    with torch.no_grad():
        for _ in range(args.warmup):
            M.ops.attention_fwd(q, k, v, 1.0 / H1 ** 0.5, 0.0, True)
        dev_ms, wall_ms, _ = best_region(lambda i: M.ops.attention_fwd(q, k, v, 1.0 / H1 ** 0.5, 0.0, True), args.steps)
    ms = max(wall_ms, dev_ms)
    flops_causal = Bc * Nh * (C * (C + 1)) * (H1 + H2)          # 2 flops x C(C+1)/2 pairs x (H1 + H2)
    flops_full = 2 * Bc * Nh * C * C * (H1 + H2)
    tf = flops_causal / (dev_ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": "attention chunk tokens/sec @4x2048, 4 heads, H1=128, H2=1024", "value": Bc * C / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[4] attention: causal softmax(q k^T) v per 2048-token chunk and head"},
        "roofline": {"bound": "mfma", "kernel": "flash_fwd_kernel (scores, causal softmax and the second product in one launch)",
                     "achieved": tf, "peak": 2500.0, "unit": "TFLOP/s", "frac": tf / 2500.0, "traffic": None,
                     "algorithmic_flops_per_call": flops_causal, "full_square_flops": flops_full, "avg_ms": dev_ms},
    }))


def bench_attention_bwd(args):
    """The backward of configs[4]'s attention (q, k, v gradients from y_grad and the forward's weights) through
    mega_attention_bwd: four products on the library's matrix-core kernel, the softmax backward and the transposed
    copies the products need.  Flops for the causal half of the four products: twice the forward's."""
    import torch

    import fairseq_apollo_amd as M

    Bc, C, Nh, H1, H2 = 4, 2048, 4, 128, 1024
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(1239)
    mk = lambda *sh: torch.randn(*sh, generator=gen).to(torch.bfloat16).to(dev)
    q, k, v, dy = mk(Bc, C, Nh, H1), mk(Bc, C, Nh, H1), mk(Bc, C, Nh, H2), mk(Bc, C, Nh, H2)
    scale = 1.0 / H1 ** 0.5
    with torch.no_grad():
        y, w = M.ops.attention_fwd(q, k, v, scale, 0.0, True, need_weights=True)
        run = lambda i: M.ops.attention_bwd(dy, q, k, v, w, scale, True, y=None if args.no_y else y)
        for _ in range(args.warmup):
            run(0)
        dev_ms, wall_ms, _ = best_region(run, args.steps)
    ms = max(wall_ms, dev_ms)
    flops_causal = 2 * Bc * Nh * (C * (C + 1)) * (H1 + H2)
    tf = flops_causal / (dev_ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": "attention backward chunk tokens/sec @4x2048, 4 heads, H1=128, H2=1024", "value": Bc * C / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[4] attention backward: q, k, v gradients per 2048-token chunk and head"},
        "roofline": {"bound": "mfma", "kernel": "gemm_nt_kernel x 4 + softmax_bwd_f32_kernel + transpose_v_kernel x 5",
                     "achieved": tf, "peak": 2500.0, "unit": "TFLOP/s", "frac": tf / 2500.0, "traffic": None,
                     "algorithmic_flops_per_call": flops_causal, "avg_ms": dev_ms},
    }))


def bench_layer(args):
    """configs[4]: one Mega2 layer forward (TimestepNorm -> CEMA -> chunked causal attention with
    rotary -> gates, then TimestepNorm -> SwiGLU), L = 8192, D = 2048, S = 512, E = 4096, chunk 2048,
    4 heads, SwiGLU hidden 5632, bf16.  The projections are library GEMMs; the rest runs in the HIP
    library.  Flops: the dense projections plus the causal half of the attention products."""
    import torch

    import fairseq_apollo_amd as M

    L4, D4, S4, E4, N4, Hf, C4, heads = 8192, 2048, 512, 4096, 16, 5632, 2048, 4
    dev = torch.device("cuda:0")
    torch.manual_seed(1238)
    blk = M.Mega2Layer(D4, S4, E4, N4, Hf, C4, norm_num_groups=16, num_heads=heads, moving_act='silu')
    train = args.workload == "layer_train"
    blk = blk.to(dev).to(torch.bfloat16)
    blk = blk.train() if train else blk.eval()
    xs = [torch.randn(1, L4, D4, device=dev).to(torch.bfloat16) for _ in range(4)]
    ws = torch.randn(1, L4, D4, device=dev).to(torch.bfloat16)

    def step(i):
        if train:                      # forward + backward of sum(y * w), from cleared gradients as a trainer's
            blk.zero_grad(set_to_none=True)    # zero_grad leaves them (fairseq/trainer.py:438)
            (blk(xs[i % 4]) * ws).sum().backward()
        else:
            blk(xs[i % 4])

    with torch.set_grad_enabled(train):
        for i in range(args.warmup):
            step(i)
        dev_ms, wall_ms, _ = best_region(step, args.steps)
    ms = max(wall_ms, dev_ms)
    gemm = 2 * L4 * D4 * (E4 + (S4 + E4 + 2 * D4)) + 2 * L4 * E4 * D4 + 3 * 2 * L4 * D4 * Hf
    nchunk = L4 // C4
    attn = nchunk * heads * C4 * (C4 + 1) * (S4 // heads + E4 // heads)
    if train:                          # two more products per forward product; the backward attention is dense
        gemm, attn = 3 * gemm, attn + 2 * nchunk * heads * 2 * C4 * C4 * (S4 // heads + E4 // heads)
    tf = (gemm + attn) / (ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": ("Mega2 layer training tokens/sec (forward + backward) @B1xL8192xD2048" if train else
                   "Mega2 layer tokens/sec @B1xL8192xD2048"), "value": L4 / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[4]: one Mega2 layer, L=8192 D=2048 z=512 h=4096 chunk=2048 4 heads, "
                               "SwiGLU 5632"},
        "roofline": {"bound": "mfma", "kernel": "whole layer (library GEMMs + HIP kernels)", "achieved": tf,
                     "peak": 2500.0, "unit": "TFLOP/s", "frac": tf / 2500.0, "traffic": None,
                     "gemm_flops": gemm, "attention_flops_causal": attn},
    }))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--settle", type=float, default=0.3, metavar="SECONDS",
                    help="block workload: seconds of untimed load before the warm-up steps (device clocks settle)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="N",
                    help="also run N plain device copies of one [B, L, D] bf16 buffer (32 MiB read + 32 MiB "
                         "written each): the known-size kernel that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                         "readings are scaled by")
    ap.add_argument("--no-y", action="store_true",
                    help="attention_bwd: call the backward as the reference does, without the forward's output")
    ap.add_argument("--workload", choices=["block", "decode", "attention", "attention_bwd", "layer", "block_bwd", "layer_train", "seqnorm", "ema_real", "tsn_feature", "long_conv"],
                    default="block",
                    help="block: the headline TimestepNorm -> EMA block (default); decode / attention / layer: "
                         "the decode step of configs[3] / the chunk attention / the whole layer of configs[4]; "
                         "ema_real: the fp32 real-EMA calls of configs[0] and configs[1]; one JSON line each")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU; --gpus N with N > 1 is not supported", file=sys.stderr)
        sys.exit(2)

    if args.workload == "decode":
        return bench_decode(args)
    if args.workload == "ema_real":
        return bench_ema_real(args)
    if args.workload == "seqnorm":
        return bench_seqnorm(args)
    if args.workload == "tsn_feature":
        return bench_tsn_feature(args)
    if args.workload == "long_conv":
        return bench_long_conv(args)
    if args.workload == "block_bwd":
        return bench_block_bwd(args)
    if args.workload == "attention_bwd":
        return bench_attention_bwd(args)
    if args.workload == "attention":
        return bench_attention(args)
    if args.workload in ("layer", "layer_train"):
        return bench_layer(args)

    import numpy as np
    import torch

    import fairseq_apollo_amd as M

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    rng = np.random.default_rng(1236)
    params = make_params(rng)
    alpha, delta, theta, gamma, omega = params

    norm = M.TimestepNorm(D, G).to(dev).eval()
    ema = M.MultiHeadComplexEMA(D, ndim=N).to(dev).eval()
    with torch.no_grad():
        for name, val in (("alpha", alpha), ("delta", delta), ("theta", theta), ("gamma", gamma), ("omega", omega)):
            getattr(ema, name).copy_(torch.from_numpy(val.astype(np.float32)))
    ema._coeffs = None
    ema._prepared = None

    gen = torch.Generator().manual_seed(1236)
    xs = [torch.randn(B, L, D, generator=gen, dtype=torch.float32).to(torch.bfloat16).to(dev) for _ in range(NBUF)]

    def step(i):
        # the head of the layer as one library call: x read once, xn and y written once
        return M.norm_then_move(norm, ema, xs[i % NBUF])

    def step_two_modules(i):
        # the same block across the module boundary: two kernels, xn travels through HBM in between
        xn = norm(xs[i % NBUF])
        return xn, ema(xn.transpose(1, 2))

    regions_log = {}

    def timed(fn, steps, warmup, name=None, regions=3):
        """(device ms per step from events on the launch stream, wall ms per step, host enqueue ms per step) of
        the median of `regions` timed regions of exactly `steps` steps each, every one bracketed by a device
        synchronisation on both sides.  The runtime now and then stalls one launch of a process for tens of
        milliseconds on the host (seen once per process, at no fixed step); a single region would then report
        that stall, not the step, and the median of three leaves it out as surely as the minimum does.  All
        regions are listed in the output line, the best one beside the median."""
        for i in range(warmup):
            fn(i)
        runs = []
        for _ in range(regions):
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            e0.record()
            for i in range(steps):
                fn(i)
            e1.record()
            host = time.perf_counter() - t0
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
            runs.append((e0.elapsed_time(e1) / steps, wall * 1e3 / steps, host * 1e3 / steps))
        if name:
            regions_log[name] = [max(r[0], r[1]) for r in runs]
        return sorted(runs, key=lambda r: max(r[0], r[1]))[len(runs) // 2]

    def settle(fn, seconds):
        """Set-up, not measurement: the device enters the run from idle and its clocks need some tens of
        milliseconds of load to settle (the first of three timed regions read 10 % slower than the third without
        this).  Runs the step for `seconds` of wall time before the W warm-up steps; neither is timed."""
        t0, i = time.perf_counter(), 0
        while time.perf_counter() - t0 < seconds:
            for _ in range(50):
                fn(i)
                i += 1
            torch.cuda.synchronize()

    with torch.no_grad():
        settle(step, args.settle)
        gpu_ms, wall_ms, host_step = timed(step, args.steps, args.warmup, name="one_call")
        ms_per_step = max(wall_ms, gpu_ms)
        reps = max(20, min(args.steps, 200))
        two_ms, _, two_host = timed(step_two_modules, reps, 8, name="two_modules")

        # per-kernel device time of the two-module variant: an event between the two calls (the EMA finds
        # its input where the norm has just left it)
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(reps)]
        for i in range(reps):
            a, b, c = evs[i]
            a.record()
            xn = norm(xs[i % NBUF])
            b.record()
            ema(xn.transpose(1, 2))
            c.record()
        torch.cuda.synchronize()
        norm_ev = float(np.median([a.elapsed_time(b) for a, b, _ in evs]))
        ema_ev = float(np.median([b.elapsed_time(c) for _, b, c in evs]))
        # the event packets between the kernels cost about a microsecond each: a kernel's time is its
        # share of the two-module step, split in the proportion of the event intervals
        norm_avg = two_ms * norm_ev / (norm_ev + ema_ev)
        ema_avg = two_ms * ema_ev / (norm_ev + ema_ev)

        # kernel generation inside the call (what a training forward does, where the coefficients change every
        # step: complex_exponential_moving_average.py:98-109): the prepared operand images are withheld, the
        # call builds them from (p, q, gamma) into its workspace first
        layer = ema._prepared_layer()
        saved_image = layer.image
        layer.image = None
        gen_ms, _, gen_host = timed(step, reps, 8, name="kernel_generation_in_call")
        layer.image = saved_image

        if args.copy_calibration:
            dst = torch.empty_like(xs[0])
            for i in range(args.copy_calibration):
                dst.copy_(xs[i % NBUF])
            torch.cuda.synchronize()
    status = M.ops.timestep_norm_status()

    traffic = measured_traffic()
    prof = profiled_durations()
    tokens = B * L
    alg_bytes_block = 4 * B * L * D * 2          # module boundary kept: norm reads x, writes xn; EMA reads xn, writes y
    alg_bytes_fused = 3 * B * L * D * 2          # what one kernel has to move: x in, xn and y out
    alg_bytes_ema = 2 * B * L * D * 2
    alg_bytes_norm = 2 * B * L * D * 2
    ema_gbs = alg_bytes_ema / (ema_avg * 1e-3) / 1e9
    norm_gbs = alg_bytes_norm / (norm_avg * 1e-3) / 1e9
    fused_gbs = alg_bytes_fused / (gpu_ms * 1e-3) / 1e9

    def kern(name, what, gbs, alg, avg):
        return {"bound": "hbm", "kernel": what, "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": gbs / HBM_PEAK_GBS, "traffic": traffic.get(name), "algorithmic_bytes_per_launch": alg,
                "avg_ms": avg, "avg_ms_source": "HIP events on the launch stream around the timed steps / steps",
                "rocprof_avg_ms": prof.get(name)}

    out = {
        "metric": "EMA+norm block tokens/sec @B4xL4096xD1024; achieved HBM GB/s vs peak",
        "value": tokens / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup, "settle_s": args.settle,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "configs[2]: TimestepNorm(16 groups) -> complex EMA (N=16), B=4 L=4096 D=1024, "
                               "bf16 activations, fp32 parameters/accumulation, forward, one library call "
                               "(xn and y both written)",
                   "input_buffers_rotated": NBUF},
        # the dominant (only) kernel of the step, priced at the bytes it has to move: x in, xn and y out
        "roofline": kern("norm_ema_fused_kernel", "norm_ema_fused_kernel (TimestepNorm and EMA in one launch)",
                         fused_gbs, alg_bytes_fused, gpu_ms),
        # the same step priced at the bytes of the two-module boundary (x, xn written and read again, y): what two
        # kernels would have to move for the same result; not what this kernel moves
        "two_module_equivalent": {"bytes_per_step": alg_bytes_block,
                                  "gbs": alg_bytes_block / (ms_per_step * 1e-3) / 1e9,
                                  "frac_of_hbm_peak": alg_bytes_block / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "best_region_ms_per_step": min(regions_log["one_call"]),
        "device_ms_per_step": gpu_ms,
        "host_enqueue_ms_per_step": host_step,
        "two_module_variant": {
            "ms_per_step": two_ms, "host_enqueue_ms_per_step": two_host,
            "hbm_frac": alg_bytes_block / (two_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "kernels": {
                "ema_mfma_kernel": kern("ema_mfma_kernel", "ema_mfma_kernel (the EMA call)", ema_gbs, alg_bytes_ema,
                                        ema_avg),
                "group_tsn_kernel": kern("group_tsn_kernel", "group_tsn_kernel (the TimestepNorm call)", norm_gbs,
                                         alg_bytes_norm, norm_avg)},
            "event_intervals_ms": {"group_tsn_kernel": norm_ev, "ema_mfma_kernel": ema_ev}},
        "kernel_generation_in_call": {
            "ms_per_step": gen_ms, "host_enqueue_ms_per_step": gen_host, "tokens_per_s": tokens / (gen_ms * 1e-3),
            "what": "the same step with the prepared operand images withheld (image = NULL): the call generates "
                    "them from (p, q, gamma) before the block kernel"},
        "timestep_norm_status": status,
        # every workload is timed in three regions of exactly `steps` steps; the line reports the median region
        "timed_regions_ms_per_step": regions_log,
    }
    if not args.no_cpu:
        threads = min(os.cpu_count() or 1, 16)
        x_host = xs[0].float().cpu().numpy()
        out["cpu_baseline"] = cpu_baseline(params, x_host, threads)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
