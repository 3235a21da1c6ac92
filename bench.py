"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one forward + backward of flash_attention_fn on the headline workload of BASELINE.json:
bf16, B=2, H=16, M=N=4096, D=128, non-causal, trainable bf16 bias (B, H, M, N); inputs are synthetic
N(0, 1) tensors already resident in HBM.  Prints ONE JSON line on stdout (everything else goes to
stderr).  Besides the whole-step throughput the line carries

  roofline      the dominant kernel (the backward kernel that produces dK, dV and dBias), timed
                with events on the launch stream around the stage that runs only that kernel,
                against the HBM peak;
  cpu_baseline  the eager fp32 oracle timed on this machine's host cores on a bounded sample;
  stages / other_configs   fwd, bwd and fwd+bwd of every BASELINE.json config.
"""
import argparse
import json
import os
import sys
import time

import torch

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, GB/s
MFMA_PEAK_TFLOPS = 2516.6    # MI355X dense bf16/fp16 MFMA, TFLOP/s
# HBM bytes per launch of the roofline kernel on the headline workload come from a committed counter
# summary (rocprofv3 FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for a plain
# 1 GiB copy); its line "traffic_bytes_per_launch: <number>" is what `roofline.traffic` reports
TRAFFIC_SUMMARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "fa_kernels_c3_hbm_traffic.txt")


def measured_traffic_bytes():
    """The figure of the counter summary, or None when the file or the line is missing."""
    try:
        with open(TRAFFIC_SUMMARY) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1].split()[0])
    except OSError:
        pass
    return None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def flops(B, H, M, N, D, causal):
    f_fwd = 4.0 * B * H * M * N * D * (0.5 if causal else 1.0)
    return f_fwd, 2.5 * f_fwd


def algorithmic_bytes(B, H, M, N, D, causal, bias_es, trainable):
    """Every input read once per pass, every output written once (workspace traffic not counted)."""
    c = 0.5 if causal else 1.0
    q = B * M * H * D * 2
    kv = B * N * H * D * 2
    bias = c * B * H * M * N * bias_es
    lse = 4 * B * H * M
    y_fwd = q + 2 * kv + q + bias + lse
    y_bwd = (q + 2 * kv + q + q) + (q + 2 * kv) + lse + bias + (bias if trainable else 0)
    # the dK/dV/dBias kernel alone: reads q, k, v, do, lse, delta, bias; writes dk, dv, dbias
    y_main = (2 * q + 2 * kv) + 2 * kv + 2 * lse + bias + (bias if trainable else 0)
    return y_fwd, y_bwd, y_main, bias * (2 + (1 if trainable else 0))


def make_config(name, dev):
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s, dt=torch.bfloat16: torch.randn(*s, device=dev, generator=g).to(dt)
    if name == "C2":
        B, M, N, H, D, causal, dt = 4, 2048, 2048, 16, 64, True, torch.float16
        return dict(q=rn(B, M, H, D, dt=dt), k=rn(B, N, H, D, dt=dt), v=rn(B, N, H, D, dt=dt), do=rn(B, M, H, D, dt=dt),
                    bias=None, causal=causal, dims=(B, H, M, N, D), bias_es=0, trainable=False)
    if name == "C3":
        B, M, N, H, D = 2, 4096, 4096, 16, 128
        return dict(q=rn(B, M, H, D), k=rn(B, N, H, D), v=rn(B, N, H, D), do=rn(B, M, H, D),
                    bias=rn(B, H, M, N).requires_grad_(True), causal=False, dims=(B, H, M, N, D), bias_es=2,
                    trainable=True)
    if name in ("C4", "C4_expanded_mask"):
        B, S, H, D = 8, 1024, 12, 64
        qkv = rn(B, S, 3, H, D)
        lens = torch.randint(512, 1025, (B,), device=dev, generator=g)
        keep = (torch.arange(S, device=dev)[None, :] < lens[:, None])[:, None, None, :].expand(B, H, S, S)
        if name == "C4":
            keep = keep.contiguous()  # the number of record; the other one reads the (B,1,1,S) mask in place
        return dict(q=qkv[:, :, 0], k=qkv[:, :, 1], v=qkv[:, :, 2], do=rn(B, S, H, D), bias=keep, causal=True,
                    dims=(B, H, S, S, D), bias_es=1, trainable=False)
    if name == "C5":
        B, H, M, N, D = 1, 32, 1024, 8192, 128
        slopes = 2.0 ** (-8.0 * (torch.arange(H, device=dev) + 1) / H)
        i = torch.arange(M, device=dev, dtype=torch.float32)[:, None]
        j = torch.arange(N, device=dev, dtype=torch.float32)[None, :]
        bias = (-slopes[:, None, None] * (i * N / M - j).abs())[None].bfloat16().requires_grad_(True)
        return dict(q=rn(B, M, H, D), k=rn(B, N, H, D), v=rn(B, N, H, D), do=rn(B, M, H, D), bias=bias, causal=False,
                    dims=(B, H, M, N, D), bias_es=2, trainable=True)
    if name == "C5_alibi_in_kernel":
        # the same attention with the bias formed from indices inside the kernels (no bias tensor,
        # the gradient is that of the 32 slopes)
        from triton_flashattn_amd import AlibiBias
        B, H, M, N, D = 1, 32, 1024, 8192, 128
        slopes = (2.0 ** (-8.0 * (torch.arange(H, device=dev) + 1) / H)).float().requires_grad_(True)
        return dict(q=rn(B, M, H, D), k=rn(B, N, H, D), v=rn(B, N, H, D), do=rn(B, M, H, D), bias=AlibiBias(slopes),
                    causal=False, dims=(B, H, M, N, D), bias_es=0, trainable=True)
    if name == "C3_row_broadcast_bias":
        # trainable bias (1, H, 1, N): gradient reduced inside the dK/dV kernel
        B, M, N, H, D = 2, 4096, 4096, 16, 128
        return dict(q=rn(B, M, H, D), k=rn(B, N, H, D), v=rn(B, N, H, D), do=rn(B, M, H, D),
                    bias=rn(1, H, 1, N).requires_grad_(True), causal=False, dims=(B, H, M, N, D), bias_es=0,
                    trainable=True)
    raise ValueError(name)


def event_time_ms(fn, iters, warmup=2):
    """Average duration of fn() over `iters` calls, from events on torch's current stream (the
    stream the kernels are launched on)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    for i in range(iters):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    return sum(s.elapsed_time(e) for s, e in zip(starts, ends)) / iters


def time_stages(cfg, iters):
    """fwd, bwd (three stages), dK/dV/dBias kernel alone, dQ kernel alone: milliseconds each."""
    import triton_flashattn_amd.flash_attention as fa
    from triton_flashattn_amd import _native
    q, k, v, do, bias, causal = cfg["q"], cfg["k"], cfg["v"], cfg["do"], cfg["bias"], cfg["causal"]
    B, M, H, D = q.shape
    N = k.shape[1]
    scale = D ** -0.5
    alibi = isinstance(bias, fa.AlibiBias)
    fwd_bias = bias if alibi or bias is None else bias.detach()
    t_fwd = event_time_ms(lambda: fa._flash_attn_fwd(q, k, v, fwd_bias, causal, scale), iters)
    o, lse = fa._flash_attn_fwd(q, k, v, fwd_bias, causal, scale)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    if alibi:
        b = bias.slopes.detach()
        dbias = torch.empty_like(b)
    else:
        b = None if bias is None else bias.detach().expand(B, H, M, N)
        dbias = torch.empty_like(bias.detach()).expand(B, H, M, N) if cfg["trainable"] else None
    be = fa._backend
    ws = be.bwd_workspace(q, k, b, causal, scale, alibi)
    run = lambda stages: be.bwd(do, q, k, v, o, b, causal, scale, lse, dq, dk, dv, dbias, stages=stages, workspace=ws,
                                alibi=alibi)
    t_bwd = event_time_ms(lambda: run(_native.FA_STAGE_ALL), iters)
    run(_native.FA_STAGE_PREP)
    t_main = event_time_ms(lambda: run(_native.FA_STAGE_MAIN), iters)
    t_dq = event_time_ms(lambda: run(_native.FA_STAGE_DQ | _native.FA_STAGE_DQ_FROM_DBIAS), iters)
    return t_fwd, t_bwd, t_main, t_dq


def step(cfg):
    from triton_flashattn_amd import flash_attention_fn
    q = cfg["q"].detach().requires_grad_(True)
    k = cfg["k"].detach().requires_grad_(True)
    v = cfg["v"].detach().requires_grad_(True)
    bias = cfg["bias"]
    if isinstance(bias, torch.Tensor) and bias.grad is not None:
        bias.grad = None
    out = flash_attention_fn(q, k, v, bias, cfg["causal"])
    out.backward(cfg["do"])


def cpu_baseline(log_fn):
    """The eager fp32 oracle on the host cores: one (batch, head) pair of the headline workload
    (1/32 of a step), forward + backward, plus the small CPU reference case of BASELINE.json."""
    from oracle.attention_oracle import reference_grads
    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)
    B, H, M, N, D = 1, 1, 4096, 4096, 128
    q, k, v, do = (torch.randn(B, M, H, D, generator=g) for _ in range(4))
    bias = torch.randn(B, H, M, N, generator=g)
    reference_grads(q, k, v, bias, do, False)
    times = []
    t_begin = time.time()
    while len(times) < 5 and time.time() - t_begin < 20.0:
        t0 = time.time()
        reference_grads(q, k, v, bias, do, False)
        times.append(time.time() - t0)
    t = sorted(times)[len(times) // 2]
    f_fwd, f_bwd = flops(B, H, M, N, D, False)
    # BASELINE.json configs[0]
    B1, M1, H1, D1 = 2, 128, 4, 64
    q1, k1, v1, do1 = (torch.randn(B1, M1, H1, D1, generator=g) for _ in range(4))
    b1 = torch.randn(B1, H1, M1, M1, generator=g)
    for _ in range(3):
        reference_grads(q1, k1, v1, b1, do1, False)
    t1 = []
    for _ in range(10):
        t0 = time.time()
        reference_grads(q1, k1, v1, b1, do1, False)
        t1.append(time.time() - t0)
    c1_ms = sorted(t1)[5] * 1e3
    log_fn("cpu oracle: slice %.1f ms (%d runs), C1 %.3f ms, %d threads" % (t * 1e3, len(times), c1_ms, threads))
    return {
        "value": (f_fwd + f_bwd) / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": "eager fp32 oracle fwd+bwd on 1 of the 32 (batch, head) pairs of the workload "
                  "(M=N=4096, D=128, fp32 bias), median of %d runs; host has %d logical CPUs" % (len(times), os.cpu_count()),
        "ms_per_sample": t * 1e3,
        "c1_reference_case_ms": c1_ms,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run one plain 1 GiB device-to-device copy and exit (reference point for "
                         "the FETCH_SIZE / WRITE_SIZE counters of a profiler)")
    ap.add_argument("--profile", metavar="CONFIG", default=None,
                    help="run only forward + backward of one config (C2, C3, C4, C5, C5_alibi_in_kernel ...) "
                         "--steps times and exit: the command to put under a profiler")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU (every (batch, head) pair is independent, so more GPUs "
            "would only shard B or H with no exchange); --gpus %d is not supported" % args.gpus)
        sys.exit(2)
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)   # 1 GiB
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        log("copied %d bytes" % (src.numel() * 4))
        return
    from triton_flashattn_amd import _native
    _native.load()  # fail loudly before timing anything

    if args.profile:
        cfg = make_config(args.profile, dev)
        for _ in range(args.warmup + args.steps):
            step(cfg)
        torch.cuda.synchronize()
        log("ran %d forward + backward steps of %s" % (args.warmup + args.steps, args.profile))
        return

    cfg = make_config("C3", dev)
    B, H, M, N, D = cfg["dims"]
    # Order of the measurements.  The first autograd step of a process spends 0.13 s on the host
    # (engine thread, allocator, library load) with the GPU idle, and an idle GPU drops its clock and
    # takes some 20 steps (25 ms) to come back: measured per step 1.9, 1.9, 1.8, 1.65, 1.6 ... 1.38 ms.
    # W = 5 warm-up steps right in front of the timed ones would put that ramp into the timed region.
    # So: one priming step first (the host-side one-off), then the per-stage timings (events around
    # each stage, repeated; the first pass is discarded), which leave the clock settled, then the W
    # warm-up steps and the K timed steps back to back.
    step(cfg)
    torch.cuda.synchronize()
    iters = max(5, min(args.steps, 30))
    time_stages(cfg, iters)
    t_fwd, t_bwd, t_main, t_dq = time_stages(cfg, iters)
    for _ in range(args.warmup):
        step(cfg)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(cfg)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    f_fwd, f_bwd = flops(B, H, M, N, D, False)
    y_fwd, y_bwd, y_main, y_bias = algorithmic_bytes(B, H, M, N, D, False, 2, True)
    value = (f_fwd + f_bwd) / (ms_per_step * 1e-3) / 1e12
    log("C3: step %.3f ms | fwd %.3f ms, bwd %.3f ms (dK/dV/dBias kernel %.3f ms, dQ kernel %.3f ms)"
        % (ms_per_step, t_fwd, t_bwd, t_main, t_dq))
    achieved = y_main / (t_main * 1e-3) / 1e9
    result = {
        "metric": "fwd+bwd TFLOP/s & bias HBM GB/s, bf16 B=2 H=16 M=N=4096 D=128",
        "value": value, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "order": "one priming step (host-side one-off), per-stage timings (they settle the clock), W warm-up steps, K timed steps",
        "config": {"workload": "BASELINE.json configs[2]: trainable bf16 bias (B,H,M,N), non-causal, "
                               "B=2 H=16 M=N=4096 D=128, flash_attention_fn forward + backward",
                   "B": B, "H": H, "M": M, "N": N, "D": D, "causal": False, "bias": "bf16, requires_grad"},
        "bias_hbm_gbs": y_bias / (ms_per_step * 1e-3) / 1e9,
        "hbm_roofline_frac_step": (y_fwd + y_bwd) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "mfma_peak_frac_step": value / MFMA_PEAK_TFLOPS,
        "stages": {
            "fwd_ms": t_fwd, "bwd_ms": t_bwd, "bwd_dkdv_kernel_ms": t_main, "bwd_dq_kernel_ms": t_dq,
            "fwd_tflops": f_fwd / (t_fwd * 1e-3) / 1e12, "bwd_tflops": f_bwd / (t_bwd * 1e-3) / 1e12,
            "fwd_gbs": y_fwd / (t_fwd * 1e-3) / 1e9, "bwd_gbs": y_bwd / (t_bwd * 1e-3) / 1e9,
        },
        "roofline": {
            "kernel": "fa_bwd_kernel<bf16, D=128, bias=bf16, non-causal, dbias>",
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic_bytes(),
            "traffic_source": "profiles/fa_kernels_c3_hbm_traffic.txt",
            "algorithmic_bytes_per_launch": y_main, "avg_launch_ms": t_main,
            # the kernel's own share of the algorithmic backward FLOPs: 4 of the 5 matrix products
            "mfma_frac_same_kernel": 0.8 * f_bwd / (t_main * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS,
        },
        "peaks": {"hbm_gbs": HBM_PEAK_GBS, "mfma_bf16_tflops": MFMA_PEAK_TFLOPS},
    }

    if not args.no_other_configs:
        others = {}
        for name in ("C2", "C4", "C4_expanded_mask", "C5", "C5_alibi_in_kernel", "C3_row_broadcast_bias"):
            del cfg
            torch.cuda.empty_cache()
            cfg = make_config(name, dev)
            Bc, Hc, Mc, Nc, Dc = cfg["dims"]
            ff, fb = flops(Bc, Hc, Mc, Nc, Dc, cfg["causal"])
            yf, yb, _, _ = algorithmic_bytes(Bc, Hc, Mc, Nc, Dc, cfg["causal"], cfg["bias_es"], cfg["trainable"])
            tf, tb, tm, tq = time_stages(cfg, 10)
            others[name] = {
                "fwd_ms": tf, "bwd_ms": tb, "fwd_bwd_ms": tf + tb,
                "fwd_tflops": ff / (tf * 1e-3) / 1e12, "bwd_tflops": fb / (tb * 1e-3) / 1e12,
                "fwd_bwd_tflops": (ff + fb) / ((tf + tb) * 1e-3) / 1e12,
                "fwd_bwd_gbs": (yf + yb) / ((tf + tb) * 1e-3) / 1e9,
                "mfma_peak_frac": (ff + fb) / ((tf + tb) * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS,
                "hbm_roofline_frac": (yf + yb) / ((tf + tb) * 1e-3) / 1e9 / HBM_PEAK_GBS,
            }
            log("%s: fwd %.3f ms, bwd %.3f ms, %.1f TFLOP/s" % (name, tf, tb, others[name]["fwd_bwd_tflops"]))
        result["other_configs"] = others

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(log)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
