#!/usr/bin/env python3
"""Benchmark of the fused chunk-list Adam step on one MI355X.

A "step" is one optimizer.step() over the whole chunk list: one launch of the fused Adam kernel that
reads every element's fp16 gradient and fp32 param/m/v once and writes fp32 param/m/v and the fp16 param
once (28 algorithmic bytes per element).  Inputs are resident in HBM before the timed region.

Workload (default): the 1.5 B-parameter configuration -- 24 chunks of 64 Mi elements (1.61 G parameters incl. padding),
g16 = (N(0,1e-3) * 2^12).half(), p ~ N(0,.02), m ~ N(0,1e-4), v = |N(0,1e-6)|, AdamW lr 1e-4
betas (.9,.999) eps 1e-8 wd .01, static loss scale 2^12, first timed step t=100.

Prints ONE JSON line (see the keys below).  `cpu_baseline` times the CPU oracle (a port of the reference's
AVX/OpenMP Adam) on this host as a reported baseline only.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

N_CHUNK = 64 * 1024 * 1024
HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak
BYTES_PER_ELEMENT = 28  # read 2+4+4+4, write 4+4+4+2


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--chunks", type=int, default=24, help="chunk-list length (24 = the 1.5 B-parameter configuration)")
    ap.add_argument("--chunk-size", type=int, default=N_CHUNK)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-unfused-baseline", action="store_true",
                    help="skip timing the reference's un-fused GPU branch (a sequence of torch element-wise kernels)")
    ap.add_argument("--cpu-reps", type=int, default=20, help="CPU baseline: at least this many timed steps")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU baseline: keep stepping for about this long")
    ap.add_argument("--host-chunks", type=int, default=0,
                    help="with --mode hybrid: how many of --chunks live in pinned host memory (the LAST ones)")
    ap.add_argument("--slots", type=int, default=2, help="with --mode hybrid: HBM staging slots")
    ap.add_argument("--host-fp16", choices=["host", "hbm"], default="host",
                    help="with --mode hybrid: where a host-resident position keeps its fp16 payload (host: the whole "
                    "position is streamed, 14 B/element each way; hbm: only fp32 param / m / v are, 12 B/element)")
    ap.add_argument("--mode", choices=["static", "dynamic", "hybrid"], default="static",
                    help="static: the 1.5 B-parameter configuration as specified (static loss scale, one fused kernel per step). "
                    "dynamic: same data with a DynamicLossScaler: inf/nan scan (2 B/element) + device-gated kernel + "
                    "scaler update per step, no host sync")
    ap.add_argument("--arithmetic", choices=["operator", "torch"], default="operator",
                    help="operator: the native operator's order of operations (default, the headline line); "
                    "torch: the formula of the reference's GPU branch")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also launch one plain device-to-device copy of 1 Gi floats (4 GiB read, 4 GiB written) "
                    "so that a rocprofv3 --pmc run holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    return ap.parse_args()


PROFILE_OF = {
    ("static", "operator"): "adam_chunks_config4_pmc.txt",
    ("dynamic", "operator"): "adam_chunks_gated_config4_dynamic.txt",
}


def traffic_from_profile(mode="static", arithmetic="operator"):
    """HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (calibrated against a copy
    kernel), as recorded in the committed profile summary; None when no such summary exists."""
    if (mode, arithmetic) not in PROFILE_OF:
        return None
    path = os.path.join(ROOT, "profiles", PROFILE_OF[(mode, arithmetic)])
    try:
        m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", open(path).read(), flags=re.M)
        return float(m.group(1)) if m else None
    except OSError:
        return None


def cpu_baseline(reps, seconds):
    """The CPU oracle on one 64 Mi-element chunk with the one-chunk reference-CPU-path inputs (p~N(0,.02), m=v=0, g16=(N(0,1e-3)*8).half(), static scale 8), all host cores of this process."""
    import numpy as np

    import oracle

    n = N_CHUNK
    rng = np.random.default_rng(0)
    p = rng.standard_normal(n, dtype=np.float32) * np.float32(0.02)
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    g = (rng.standard_normal(n, dtype=np.float32) * np.float32(8e-3)).astype(np.float16)
    o = oracle.AdamOracle(1e-3, 0.9, 0.999, 1e-6, 0.0, False)
    isa = o.update(1, 1e-3, 0.9, 0.999, 1e-6, 0.0, True, p, g, m, v, 8.0)
    o.update(2, 1e-3, 0.9, 0.999, 1e-6, 0.0, True, p, g, m, v, 8.0)
    times = []
    started = time.perf_counter()
    while len(times) < reps or (time.perf_counter() - started < seconds and len(times) < 100000):
        t0 = time.perf_counter()
        o.update(3 + len(times), 1e-3, 0.9, 0.999, 1e-6, 0.0, True, p, g, m, v, 8.0)
        times.append(time.perf_counter() - t0)
    best = min(times)
    median = sorted(times)[len(times) // 2]
    reps = len(times)
    # the un-vectorised code path as well (what the reference's own builder selects on a non-Intel host)
    t0 = time.perf_counter()
    o.update(3 + reps, 1e-3, 0.9, 0.999, 1e-6, 0.0, True, p, g, m, v, 8.0, oracle.ISA_SCALAR)
    scalar_s = time.perf_counter() - t0
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count()
    cpu_model = "unknown CPU"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                cpu_model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    omp = os.environ.get("OMP_NUM_THREADS")
    if omp and omp.isdigit():
        cores = min(cores, int(omp))
    return {
        "value": n / best,
        "unit": "params/s",
        "cores": cores,
        "kind": "port",
        "sample": f"1 chunk of {n} elements (one-chunk CPU-path inputs, static scale 8), best of {reps} steps over "
        f"{sum(times):.1f} s after 2 warm-up (median step {n / median / 1e9:.2f} G params/s); "
        f"oracle code path {['', 'scalar', 'AVX2', 'AVX-512'][isa]}; 26 B/element -> {26 * n / best / 1e9:.0f} GB/s; "
        f"scalar code path of the same oracle, 1 step: {n / scalar_s / 1e9:.2f} G params/s; host CPU: {cpu_model}",
    }


def run_hybrid(args):
    """The hybrid-placement configuration: C chunks, the last H of them in pinned host memory, streamed through HBM staging.
    Reports effective params/s over the whole list and the overlap efficiency
    max(kernel total, H2D total, D2H total) / wall."""
    import torch

    import patrickstar_amd as ps
    from patrickstar_amd import _lib

    dev = torch.device("cuda:0")
    C, H, N = args.chunks, args.host_chunks, args.chunk_size
    first_host = C - H
    fp16_on_host = args.host_fp16 == "host"
    link_per_element = 14 if fp16_on_host else 12
    client = ps.PatrickStarClient(
        0, N, config={"host_chunk_policy": lambda pos: pos >= first_host, "host_keeps_fp16": fp16_on_host}
    )
    params = client.append_flat_chunks(C)
    opt = ps.FP16Adam(client, params, loss_scaler=ps.LossScaler(2**12), lr=1e-4, betas=(0.9, 0.999), eps=1e-8,
                      weight_decay=0.01, use_adamw=True)
    opt.staging_slots = args.slots
    gen = torch.Generator(device=dev)
    gen.manual_seed(0)
    cl = client.chunk_list
    tmp = torch.empty(N, device=dev)
    for pos in client.positions():
        cl[pos.fp32].payload.copy_(tmp.normal_(0, 0.02, generator=gen))
        cl[pos.exp_avg].payload.copy_(tmp.normal_(0, 1e-4, generator=gen))
        cl[pos.exp_avg_sq].payload.copy_(tmp.normal_(0, 1e-6, generator=gen).abs_())
        cl[pos.fp16].payload.copy_(tmp.normal_(0, 1e-3, generator=gen).mul_(2.0**12).half())
    del tmp
    torch.cuda.synchronize()
    for p in params:
        dict.__setitem__(opt.state[p], "step", 99 - args.warmup)
    for _ in range(args.warmup):
        opt.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    enqueue = 0.0
    for _ in range(args.steps):
        t1 = time.perf_counter()
        opt.step()
        enqueue += time.perf_counter() - t1  # host time inside step(): everything is only enqueued
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / args.steps
    enqueue /= args.steps

    # the three legs on their own
    host_pos = [q for q in client.positions() if q.on_host]
    slot = [torch.empty(N, dtype=torch.float, device=dev) for _ in range(3)] + [torch.empty(N, dtype=torch.half, device=dev)]
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def timed(fn):
        torch.cuda.synchronize()
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3

    n_streamed = 4 if fp16_on_host else 3  # payloads of a host position that cross the link

    def h2d():
        for q in host_pos:
            for dst, cid in list(zip(slot, (q.fp32, q.exp_avg, q.exp_avg_sq, q.fp16)))[:n_streamed]:
                dst.copy_(cl[cid].payload, non_blocking=True)

    def d2h():
        for q in host_pos:
            for src, cid in list(zip(slot, (q.fp32, q.exp_avg, q.exp_avg_sq, q.fp16)))[:n_streamed]:
                cl[cid].payload.copy_(src, non_blocking=True)

    lib = _lib.load()
    lib.ps_adam_create(991, 1e-4, 0.9, 0.999, 1e-8, 0.01, 1, 0)
    one = _lib.chunk_array([[t.data_ptr() for t in slot]])
    res_rows = [[cl[c].payload.data_ptr() for c in (q.fp32, q.exp_avg, q.exp_avg_sq, q.fp16)] for q in client.positions() if not q.on_host]
    res = _lib.chunk_array(res_rows) if res_rows else None

    def kernels():
        s = _lib.current_stream_handle()
        if res_rows:
            lib.ps_adam_step_chunks(991, 1, 1e-4, 0.9, 0.999, 1e-8, 0.01, 1, res, len(res_rows), N, None, 4096.0, s)
        for _ in host_pos:
            lib.ps_adam_step_chunks(991, 1, 1e-4, 0.9, 0.999, 1e-8, 0.01, 1, one, 1, N, None, 4096.0, s)

    t_h2d, t_d2h = timed(h2d), timed(d2h)
    h2d()  # leave finite data in the slot for the kernel leg
    t_kernel = timed(kernels)
    lib.ps_adam_destroy(991)
    bound = max(t_h2d, t_d2h, t_kernel)
    elements = C * N
    link_bytes = link_per_element * H * N
    out = {
        "metric": "Adam params/sec, chunk-list optimizer step with host-resident chunks streamed through HBM, 1 GPU",
        "value": elements / wall,
        "unit": "params/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"hybrid placement: {C} chunks x {N} elements, {C - H} resident in HBM, {H} in pinned host memory "
            f"streamed through {args.slots} HBM staging slots ({link_per_element} B/element each way over the host link; "
            f"fp16 payloads of host positions in {'pinned host memory' if fp16_on_host else 'HBM'})",
            "chunks": C, "host_chunks": H, "chunk_numel": N, "slots": args.slots, "host_fp16": args.host_fp16,
        },
        "hybrid": {
            "overlap_efficiency": bound / wall,
            "wall_s": wall, "host_enqueue_s": enqueue, "kernel_total_s": t_kernel, "h2d_total_s": t_h2d, "d2h_total_s": t_d2h,
            "h2d_GBps": link_bytes / t_h2d / 1e9 if H else None,
            "d2h_GBps": link_bytes / t_d2h / 1e9 if H else None,
        },
    }
    print(json.dumps(out))


def unfused_gpu_branch(C, N, steps=3):
    """The reference's GPU branch of one step, restated op for op with torch kernels on fresh buffers of the same
    shape (patrickstar/ops/fp16_cpu_adam.py:245-277,430 per tensor -- here per chunk -- followed by the whole-chunk
    fp32->fp16 copy_ of patrickstar/ops/chunk_io_buff.py:116-126).  A same-GPU baseline for the fused kernel, reported
    beside it; not part of `value`."""
    import math

    import torch

    dev = torch.device("cuda:0")
    lr, b1, b2, eps, wd, scale, t = 1e-4, 0.9, 0.999, 1e-8, 0.01, 4096.0, 100
    p = [torch.randn(N, device=dev) * 0.02 for _ in range(C)]
    m = [torch.randn(N, device=dev) * 1e-4 for _ in range(C)]
    v = [(torch.randn(N, device=dev) * 1e-6).abs_() for _ in range(C)]
    h = [(torch.randn(N, device=dev) * 4).half() for _ in range(C)]

    def one_step(step):
        bc1, bc2 = 1 - b1**step, 1 - b2**step
        for c in range(C):
            g = h[c].float()
            g.div_(scale)
            p[c].mul_(1 - lr * wd)
            m[c].mul_(b1).add_(g, alpha=1 - b1)
            v[c].mul_(b2).addcmul_(g, g, value=1 - b2)
            denom = (v[c].sqrt() / math.sqrt(bc2)).add_(eps)
            p[c].addcdiv_(m[c], denom, value=-(lr / bc1))
            h[c].copy_(p[c])

    one_step(t)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        one_step(t + 1 + k)
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / steps
    return {
        "value": C * N / sec,
        "unit": "params/s",
        "ms_per_step": sec * 1e3,
        "kind": "port of the reference's un-fused GPU branch (12 torch kernels per chunk), same GPU, same shapes",
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (every GPU box here has one GPU)")
    import torch

    import patrickstar_amd as ps

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    if args.mode == "hybrid":
        torch.cuda.set_device(0)
        return run_hybrid(args)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    C, N = args.chunks, args.chunk_size

    client = ps.PatrickStarClient(0, N)
    params = client.append_flat_chunks(C)
    if args.mode == "static":
        scaler = ps.LossScaler(2**12)
    else:
        scaler = ps.DynamicLossScaler(init_scale=2**12, scale_factor=2, scale_window=1000, min_scale=1)
    opt = ps.FP16Adam(client, params, loss_scaler=scaler, lr=1e-4, betas=(0.9, 0.999), eps=1e-8,
                      weight_decay=0.01, use_adamw=True, arithmetic=args.arithmetic)
    gen = torch.Generator(device=dev)
    gen.manual_seed(0)
    cl = client.chunk_list
    grads = []
    for pos in client.positions():
        cl[pos.fp32].payload.normal_(0, 0.02, generator=gen)
        cl[pos.exp_avg].payload.normal_(0, 1e-4, generator=gen)
        cl[pos.exp_avg_sq].payload.normal_(0, 1e-6, generator=gen).abs_()
        tmp = torch.empty(N, device=dev).normal_(0, 1e-3, generator=gen).mul_(2.0**12)
        cl[pos.fp16].payload.copy_(tmp)
        del tmp
    # the step overwrites the fp16 gradients with fp16 parameters; later steps then read those as "gradients" of the
    # same magnitude class (|p| ~ 0.02 vs |g*scale| ~ 4), which changes values, not the work done per element
    if args.mode == "static":
        for p in params:
            dict.__setitem__(opt.state[p], "step", 99 - args.warmup)
    else:
        scaler._seed_step(99 - args.warmup)

    if args.calibration_copy:
        src = torch.empty(1 << 30, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        opt.step()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        starts[i].record()  # on torch's current stream, the stream the kernel is launched on
        opt.step()
        ends[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kernel_ms = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    avg_kernel_ms = sum(kernel_ms) / len(kernel_ms)
    ms_per_step = wall * 1e3 / args.steps
    elements = C * N
    # the dynamic mode adds the 2 B/element probe pass to the step
    algorithmic = (BYTES_PER_ELEMENT + (2 if args.mode == "dynamic" else 0)) * elements
    achieved = algorithmic / (avg_kernel_ms * 1e-3) / 1e9

    out = {
        "metric": "Adam params/sec, fused chunk-list optimizer step, 1 GPU",
        "value": elements / (ms_per_step * 1e-3),
        "unit": "params/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"1.5B-parameter chunk list: {C} chunks x {N} elements ({elements} parameters incl. padding) resident in HBM, "
            "AdamW lr 1e-4 betas (0.9,0.999) eps 1e-8 wd 0.01, static loss scale 2^12, fp16 grads -> fp32 p/m/v + fp16 params",
            "chunks": C,
            "chunk_numel": N,
            "kernel": f"adam_chunks_kernel<{args.arithmetic}, decoupled, reciprocal unscale>" if args.mode == "static"
            else "scan_chunks_kernel + adam_chunks_gated_kernel<decoupled> + scaler_update_kernel",
            "mode": args.mode,
            "arithmetic": args.arithmetic,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic_from_profile(args.mode, args.arithmetic) if (C, N) == (24, N_CHUNK) else None,
            "algorithmic_bytes_per_launch": algorithmic,
            "avg_kernel_ms": avg_kernel_ms,
            "median_kernel_ms": sorted(kernel_ms)[len(kernel_ms) // 2],
            "min_kernel_ms": min(kernel_ms),
        },
    }
    del opt, client, params, grads
    torch.cuda.empty_cache()
    if not args.no_unfused_baseline and args.mode == "static":
        out["unfused_gpu_baseline"] = unfused_gpu_branch(C, N)
        torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.cpu_reps, args.cpu_seconds)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
