#!/usr/bin/env python3
"""Benchmark of the fused optimizer step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the hot path over one resident parameter set: for the default workload one
`raf.op.lans` step over a BERT-large-shaped list (391 tensors, 335,141,888 elements; fp32 weights and
state, fp16 gradients scaled by 1024 and unscaled in the kernel), called through the C ABI.  Inputs
are synthetic (seeded, generated on the GPU) and resident in HBM before the timed region.  Prints
ONE JSON line; `value` is algorithmic bytes per step divided by the wall time per step.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak

# Algorithmic bytes per element of a three-pass LANS step, the figure the bandwidth is quoted on:
#   norms of g and w (read g,w); norms of the update directions (read g,w,m,v); the update itself
#   (read g,w,m,v, write w,m,v): 28 compulsory + 24 re-read = 52 B with fp32 gradients, 46 B with fp16.
# The kernels move less than that (||w|| rides along with the second pass, saving its 4 B), which
# is reported separately as `kernel_bytes_per_element`.
def lans_bytes_per_elt(g_bytes: int):
    a = g_bytes + 4
    b = g_bytes + 12
    c = g_bytes + 12 + 12
    return a, b, c


def lans_kernel_bytes_per_elt(g_bytes: int):
    return g_bytes, g_bytes + 12, g_bytes + 12 + 12


SGD_BYTES_PER_ELT = 20  # read x, dx, v; write v1, x1

# Memory traffic per launch of the dominant kernel (bytes), from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# runs scaled by a plain 1 GiB copy (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0); figures and commands are in
# profiles/.  Workloads not listed were not measured (null).
MEASURED_TRAFFIC = {
    ("lans_bert_large_fp16grad", "lans_pipelined"): 14_088_700_000,
    ("lans_bert_large_fp16grad", "lans_apply"): 8_716_600_000,
    ("sgd_4m_fp32", "sgd_vec4_kernel"): 83_925_600,
    ("lans_bert_large_mixed_fp16", "lans_pipelined"): 14_759_300_000,
    ("sgd_multi_bert_large_fp32", "sgd_multi_kernel"): 6_708_200_000,
    ("l2norm_bert_large_flat_fp32", "l2norm_partials"): 1_340_800_000,
    ("fuse_bert_large_fp32", "fuse_copy"): 2_683_900_000,
    ("defuse_bert_large_fp32", "fuse_copy"): 2_683_900_000,
}


def workloads():
    from raf_amd import shapes

    return {
        "lans_bert_large_fp16grad": dict(kind="lans", sizes=shapes.numels(shapes.bert_large_shapes()), g16=True,
                                         zero_state=True, step0=1),
        # half-precision model with fp32 master weights: fp16 gradients in, fp16 weight copies out
        "lans_bert_large_mixed_fp16": dict(kind="lans", sizes=shapes.numels(shapes.bert_large_shapes()), g16=True,
                                           zero_state=True, step0=1, copy16=True),
        "lans_bert_large_fp32grad": dict(kind="lans", sizes=shapes.numels(shapes.bert_large_shapes()), g16=False,
                                         zero_state=True, step0=1),
        "lans_bert_base_fp32": dict(kind="lans", sizes=shapes.numels(shapes.bert_base_shapes()), g16=False,
                                    zero_state=True, step0=1),
        "lans_2000_small_tensors": dict(kind="lans", sizes=shapes.log_uniform_numels(), g16=False,
                                        zero_state=False, step0=2),
        "lans_gpt2_1p5b_fp32": dict(kind="lans", sizes=shapes.numels(shapes.gpt2_shapes()), g16=False,
                                    zero_state=True, step0=1),
        "sgd_4m_fp32": dict(kind="sgd", n=4_194_304),
        "sgd_multi_bert_large_fp32": dict(kind="sgd_multi", sizes=shapes.numels(shapes.bert_large_shapes())),
        # the traced optimizer's per-parameter op sequence after dialect fusion: one fused call per parameter
        "traced_sgd_fused_bert_large_fp32": dict(kind="traced_sgd", sizes=shapes.numels(shapes.bert_large_shapes())),
        # neighbours of the optimizer step that reuse its machinery
        "l2norm_bert_large_flat_fp32": dict(kind="l2norm", n=sum(shapes.numels(shapes.bert_large_shapes()))),
        "fuse_bert_large_fp32": dict(kind="fuse", sizes=shapes.numels(shapes.bert_large_shapes()), gather=True),
        "defuse_bert_large_fp32": dict(kind="fuse", sizes=shapes.numels(shapes.bert_large_shapes()), gather=False),
        # a plain device-to-device copy of known size: the yardstick that rocprofv3's FETCH_SIZE /
        # WRITE_SIZE counters are scaled by when HBM traffic is measured
        "copy_1gib": dict(kind="copy", nbytes=1 << 30),
    }


def gen_lans(sizes, g16, zero_state, dev, seed=2024):
    import torch

    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    g, w, m, v = [], [], [], []
    for n in sizes:
        gt = torch.randn(n, device=dev, generator=gen) * 1e-3
        g.append((gt * 1024.0).half() if g16 else gt)
        w.append(torch.randn(n, device=dev, generator=gen) * 0.02)
        if zero_state:
            m.append(torch.zeros(n, device=dev))
            v.append(torch.zeros(n, device=dev))
        else:
            m.append(torch.randn(n, device=dev, generator=gen) * 1e-4)
            v.append((torch.randn(n, device=dev, generator=gen) * 1e-6).abs())
    return g, w, m, v


def cpu_baseline_lans(sizes, g16, budget_s=12.0):
    """The oracle's C restatement (a port: the reference has no CPU LANS) timed on the host cores
    over a prefix of the same tensor list, large enough to be memory-bound."""
    from oracle import c_oracle
    from oracle.lans_f64 import LansHParams

    threads = min(16, os.cpu_count() or 1, c_oracle.max_threads())
    sample, total = [], 0
    for n in sizes:
        sample.append(n)
        total += n
        if total >= 64_000_000:
            break
    rng = np.random.default_rng(2024)
    g = [(rng.standard_normal(n, dtype=np.float32) * (1.024 if g16 else 1e-3)).astype(np.float16 if g16 else np.float32)
         for n in sample]
    w = [rng.standard_normal(n, dtype=np.float32) * np.float32(0.02) for n in sample]
    m = [np.zeros(n, np.float32) for n in sample]
    v = [np.zeros(n, np.float32) for n in sample]
    hp = LansHParams(grad_unscale=(1.0 / 1024 if g16 else 1.0))
    best, reps, t_all = None, 0, time.perf_counter()
    while reps < 1000 and time.perf_counter() - t_all < budget_s:  # about 12 s on all host cores
        t0 = time.perf_counter()
        c_oracle.lans_step_inplace(g, w, m, v, reps + 1, hp, threads=threads)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
        reps += 1
    bpe = sum(lans_bytes_per_elt(2 if g16 else 4))
    return {"value": round(total * bpe / best / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"first {len(sample)} tensors of the list ({total} elements), best of {reps} steps, "
                      f"float64 C restatement of the rule, OpenMP {threads} threads",
            "ms_per_step_extrapolated": round(best * 1e3 * sum(sizes) / total, 1)}


def cpu_baseline_sgd(n, budget_s=10.0):
    from oracle import c_oracle

    threads = min(16, os.cpu_count() or 1, c_oracle.max_threads())
    rng = np.random.default_rng(2024)
    x, dx, v = (rng.standard_normal(n, dtype=np.float32) for _ in range(3))
    best, reps, t_all = None, 0, time.perf_counter()
    while reps < 50 and time.perf_counter() - t_all < budget_s:
        t0 = time.perf_counter()
        c_oracle.sgd_step(x, dx, v, 0.01, 0.9, threads=threads)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
        reps += 1
    return {"value": round(n * SGD_BYTES_PER_ELT / best / 1e9, 2), "unit": "GB/s", "cores": threads,
            "kind": "port", "sample": f"the full tensor ({n} elements), best of {reps} steps, fp32 C restatement "
                                      f"(-ffp-contract=off), OpenMP {threads} threads"}


def bench_lans(name, wl, args):
    import torch

    from raf_amd import kernels

    dev = torch.device("cuda:0")
    sizes, g16 = wl["sizes"], wl["g16"]
    total = sum(sizes)
    g, w, m, v = gen_lans(sizes, g16, wl["zero_state"], dev)
    plan = kernels.LansPlan(sizes, torch.float16 if g16 else torch.float32, dev)
    if args.schedule != "auto":
        plan.set_schedule(args.schedule)
    schedule = plan.schedule
    hp = kernels.make_hparams(grad_unscale=(1.0 / 1024 if g16 else 1.0))
    copy16 = bool(wl.get("copy16"))
    p16 = [torch.empty(n, dtype=torch.float16, device=dev) for n in sizes] if copy16 else None
    plan.bind(g, w, m, v, hp, p=p16)
    step_t = torch.full((), float(wl["step0"]), dtype=torch.float32, device=dev)

    def one_step():
        plan.step_bound(step_t)
        step_t.add_(1.0)  # the step counter lives on the device, as in the reference's traced optimizer

    for _ in range(args.warmup):
        one_step()
    graph = None
    if args.hip_graph:
        # The launches of one step (and the counter's increment) recorded once and replayed: what a
        # training loop captured in a HIP graph pays per step.  Per-kernel events stay outside.
        args.no_kernel_events = True
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            one_step()
        for _ in range(3):
            graph.replay()
    if not args.no_kernel_events:
        plan.timing_enable(args.steps)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        if graph is not None:
            graph.replay()
        else:
            one_step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps

    a, b, c = lans_bytes_per_elt(2 if g16 else 4)
    ka, kb, kc = lans_kernel_bytes_per_elt(2 if g16 else 4)
    # phased: five launches, or three when the list fits the cache and no tensor has more than 32 chunks
    # (every workgroup then adds its tensor's few partial sums itself)
    lib = _libs()
    short = all(-(-n // lib.rafhip_lans_chunk_elements(n)) <= 32 for n in sizes if n)
    cached = total * (14 if g16 else 16) <= (192 << 20)
    launches = 2 if schedule == "pipelined" else (3 if short and cached else 5)
    if copy16:  # the third pass also writes the 2-byte copy of the new weight
        c, kc = c + 2, kc + 2
    bytes_step = total * (a + b + c)
    out = {
        "metric": "LANS optimizer-step achieved HBM bandwidth (algorithmic bytes / step time); "
                  "ms_per_step is the step time",
        "value": round(bytes_step / (ms_per_step * 1e-3) / 1e9, 1),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64", "data": "synthetic",
        "config": {"workload": name, "tensors": len(sizes), "elements": total,
                   "storage": "fp32 w/m/v, " + ("fp16 g (x1024, unscaled in kernel)" if g16 else "fp32 g") +
                              (", fp16 copy of the new weights written" if copy16 else ""),
                   "bytes_per_element": a + b + c, "bytes_per_step": bytes_step,
                   "kernel_bytes_per_element": ka + kb + kc,
                   "pct_of_hbm_peak": round(100 * bytes_step / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
                   "schedule": schedule, "launches_per_step": launches, "hip_graph": bool(args.hip_graph)},
    }
    if not args.no_kernel_events:
        ts = np.array([plan.timing_read(i) for i in range(args.steps)], dtype=np.float64)
        avg = ts.mean(axis=0)
        if schedule == "phased":
            # dominant kernel: lans_apply (reads g,w,m,v, writes w,m,v)
            apply_ms = float(avg[4])
            achieved = total * c / (apply_ms * 1e-3) / 1e9
            out["roofline"] = {"bound": "hbm", "kernel": "lans_apply", "achieved": round(achieved, 1),
                               "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                               "traffic": MEASURED_TRAFFIC.get((name, "lans_apply")),
                               "bytes_per_launch": total * c, "avg_launch_ms": round(apply_ms, 4)}
            out["kernels_ms"] = {"lans_norm_g": round(float(avg[0]), 4), "lans_finish(a)": round(float(avg[1]), 4),
                                 "lans_norm_u": round(float(avg[2]), 4), "lans_finish(b)": round(float(avg[3]), 4),
                                 "lans_apply": round(apply_ms, 4)}
            out["kernels_GBps"] = {"lans_norm_g": round(total * ka / avg[0] / 1e6, 1),
                                   "lans_norm_u": round(total * kb / avg[2] / 1e6, 1),
                                   "lans_apply": round(total * kc / avg[4] / 1e6, 1)}
        else:
            # one persistent kernel does all three passes
            k_ms = float(avg[1])
            achieved = bytes_step / (k_ms * 1e-3) / 1e9
            out["roofline"] = {"bound": "hbm", "kernel": "lans_pipelined", "achieved": round(achieved, 1),
                               "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                               "traffic": MEASURED_TRAFFIC.get((name, "lans_pipelined")),
                               "bytes_per_launch": bytes_step, "avg_launch_ms": round(k_ms, 4),
                               # the same launch priced by the bytes the kernel requests (the norm of w
                               # rides on pass B) and by the compulsory read-once/write-once bytes
                               "achieved_by_requested_bytes": round(total * (ka + kb + kc) / (k_ms * 1e-3) / 1e9, 1),
                               "achieved_by_compulsory_bytes": round(total * c / (k_ms * 1e-3) / 1e9, 1)}
            out["kernels_ms"] = {"lans_prepare": round(float(avg[0]), 4), "lans_pipelined": round(k_ms, 4)}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_lans(sizes, g16)
    return out


def bench_sgd(name, wl, args):
    import torch

    from raf_amd import kernels

    dev = torch.device("cuda:0")
    n = wl["n"]
    # 84 MB per buffer set would sit in the 256 MB Infinity Cache: rotate over enough disjoint sets
    # that every step streams from HBM.
    sets = 8
    gen = torch.Generator(device=dev)
    gen.manual_seed(2024)
    bufs = []
    for _ in range(sets):
        x = torch.randn(n, device=dev, generator=gen) * 0.02
        dx = torch.randn(n, device=dev, generator=gen) * 1e-3
        v = torch.zeros(n, device=dev)
        bufs.append((x, dx, v, torch.empty_like(x), torch.empty_like(x)))
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(args.warmup):
        x, dx, v, v1, x1 = bufs[i % sets]
        kernels.sgd_f32(x, dx, v, 0.01, 0.9, v_out=v1, x_out=x1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for i in range(args.steps):
        x, dx, v, v1, x1 = bufs[i % sets]
        kernels.sgd_f32(x, dx, v, 0.01, 0.9, v_out=v1, x_out=x1)
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    dev_ms = start.elapsed_time(stop) / args.steps  # kernels run on torch's current stream
    bytes_step = n * SGD_BYTES_PER_ELT
    achieved = bytes_step / (dev_ms * 1e-3) / 1e9
    out = {
        "metric": "SGD momentum step achieved HBM bandwidth (algorithmic bytes / step time)",
        "value": round(bytes_step / (ms_per_step * 1e-3) / 1e9, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": name, "elements": n, "bytes_per_element": SGD_BYTES_PER_ELT,
                   "buffer_sets_rotated": sets},
        "roofline": {"bound": "hbm", "kernel": "sgd_vec4_kernel", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC.get((name, "sgd_vec4_kernel")), "bytes_per_launch": bytes_step,
                     "avg_launch_ms": round(dev_ms, 5)},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_sgd(n)
    return out


def _timed(fn, args):
    """Warm-up, then `steps` calls of fn between events on torch's current stream (the one the
    kernels are launched on); returns (wall ms per step, device ms per step)."""
    import torch

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(args.warmup):
        fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for i in range(args.steps):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    return wall_ms, start.elapsed_time(stop) / args.steps


def _line(metric, name, dtype, bytes_step, wall_ms, dev_ms, kernel, args, config):
    achieved = bytes_step / (dev_ms * 1e-3) / 1e9
    return {
        "metric": metric, "value": round(bytes_step / (wall_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": dict(workload=name, **config),
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC.get((name, kernel)), "bytes_per_launch": bytes_step,
                     "avg_launch_ms": round(dev_ms, 5)},
    }


def bench_sgd_multi(name, wl, args):
    import torch

    from oracle import c_oracle
    from raf_amd import kernels

    dev = torch.device("cuda:0")
    sizes = wl["sizes"]
    total = sum(sizes)
    gen = torch.Generator(dev).manual_seed(2024)
    x = [torch.randn(n, device=dev, generator=gen) * 0.02 for n in sizes]
    dx = [torch.randn(n, device=dev, generator=gen) * 1e-3 for n in sizes]
    v = [torch.zeros(n, device=dev) for n in sizes]
    plan = kernels.SgdPlan(sizes, torch.float32, dev)
    m = plan.marshal(x, dx, v)
    wall_ms, dev_ms = _timed(lambda i: plan.step(x, dx, v, 0.01, 0.9, marshalled=m), args)
    res = _line("multi-tensor SGD momentum step achieved HBM bandwidth (algorithmic bytes / step time)", name, "f32",
                total * SGD_BYTES_PER_ELT, wall_ms, dev_ms, "sgd_multi_kernel", args,
                {"tensors": len(sizes), "elements": total, "bytes_per_element": SGD_BYTES_PER_ELT,
                 "launches_per_step": 1})
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline_sgd(1 << 24)
    return res


def bench_l2norm(name, wl, args):
    import torch

    from oracle import tensor_ops
    from raf_amd import kernels

    dev = torch.device("cuda:0")
    n = wl["n"]
    x = torch.randn(n, device=dev, generator=torch.Generator(dev).manual_seed(2024)) * 0.02
    out = torch.empty((), device=dev)
    ws = torch.empty(max(_libs().rafhip_l2norm_workspace_bytes(n), 8), dtype=torch.uint8, device=dev)
    wall_ms, dev_ms = _timed(lambda i: kernels.l2norm(x, out=out, workspace=ws), args)
    res = _line("L2 norm achieved HBM bandwidth (algorithmic bytes / time)", name, "f64", 4 * n, wall_ms, dev_ms,
                "l2norm_partials", args, {"elements": n, "bytes_per_element": 4, "storage": "fp32"})
    if not args.no_cpu_baseline:
        sample = x[:1 << 26].cpu().numpy()
        best = None
        for _ in range(5):
            t0 = time.perf_counter()
            tensor_ops.l2norm(sample)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        res["cpu_baseline"] = {"value": round(sample.size * 4 / best / 1e9, 2), "unit": "GB/s", "cores": 1,
                               "kind": "port", "sample": f"first {sample.size} elements, best of 5, NumPy float64 oracle"}
    return res


def bench_fuse(name, wl, args):
    import torch

    from oracle import tensor_ops
    from raf_amd import kernels

    dev = torch.device("cuda:0")
    sizes = wl["sizes"]
    gen = torch.Generator(dev).manual_seed(2024)
    parts = [torch.randn(n, device=dev, generator=gen) for n in sizes]
    flat = torch.randn(sum(sizes), device=dev, generator=gen)
    plan = kernels.FusePlan([4 * n for n in sizes], dev)
    if wl["gather"]:
        step, kernel, what = (lambda i: plan.fuse(parts, flat)), "fuse_copy", "fuse_tensor"
    else:
        step, kernel, what = (lambda i: plan.defuse(flat, parts)), "fuse_copy", "defuse_tensor"
    wall_ms, dev_ms = _timed(step, args)
    moved = 2 * plan.total_bytes
    res = _line(f"{what} achieved HBM bandwidth (bytes read + written / time)", name, "u8", moved, wall_ms, dev_ms,
                kernel, args, {"tensors": len(sizes), "bytes_read_per_step": plan.total_bytes,
                               "bytes_written_per_step": plan.total_bytes, "launches_per_step": 1})
    if not args.no_cpu_baseline:
        host = [p.cpu().numpy() for p in parts[:48]]
        best = None
        for _ in range(5):
            t0 = time.perf_counter()
            tensor_ops.fuse_tensor(host)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        nb = sum(a.nbytes for a in host)
        res["cpu_baseline"] = {"value": round(2 * nb / best / 1e9, 2), "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"first {len(host)} tensors ({nb} bytes), best of 5, NumPy oracle (fuse direction)"}
    return res


def _libs():
    from raf_amd import _lib

    return _lib.optim()


def bench_copy(name, wl, args):
    import torch

    dev = torch.device("cuda:0")
    n = wl["nbytes"] // 4
    src = torch.randn(n, device=dev)
    dst = torch.empty_like(src)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(args.warmup):
        dst.copy_(src)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        dst.copy_(src)
    stop.record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    dev_ms = start.elapsed_time(stop) / args.steps
    moved = 2 * wl["nbytes"]
    return {"metric": "device-to-device copy bandwidth (read + write bytes / time)",
            "value": round(moved / (ms_per_step * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": name, "bytes_read_per_step": wl["nbytes"], "bytes_written_per_step": wl["nbytes"]},
            "roofline": {"bound": "hbm", "kernel": "torch copy", "achieved": round(moved / (dev_ms * 1e-3) / 1e9, 1),
                         "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(moved / (dev_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                         "traffic": None, "bytes_per_launch": moved, "avg_launch_ms": round(dev_ms, 4)}}


def bench_traced_sgd(name, wl, args):
    """One step = the traced SGD update of every parameter, each parameter's add/multiply/subtract
    sequence fused by the dialect pass into one primitive function and run as one launch."""
    import torch

    from raf_amd import op

    dev = torch.device("cuda:0")
    sizes = wl["sizes"]
    total = sum(sizes)
    gen = torch.Generator(dev).manual_seed(2024)
    x = [torch.randn(n, device=dev, generator=gen) * 0.02 for n in sizes]
    dx = [torch.randn(n, device=dev, generator=gen) * 1e-3 for n in sizes]
    v = [torch.zeros(n, device=dev) for n in sizes]

    updates = [op.TracedSgdUpdate(w_, d_, v_, 0.01, 0.9) for w_, d_, v_ in zip(x, dx, v)]

    def step(_):
        for upd in updates:
            upd()

    wall_ms, dev_ms = _timed(step, args)
    res = _line("traced SGD update after dialect fusion, achieved HBM bandwidth (algorithmic bytes / step time)",
                name, "f32", total * SGD_BYTES_PER_ELT, wall_ms, dev_ms, "sgd_vec4_kernel", args,
                {"tensors": len(sizes), "elements": total, "bytes_per_element": SGD_BYTES_PER_ELT,
                 "launches_per_step": len(sizes), "unfused_kernels_per_step": 4 * len(sizes)})
    # the roofline object is about one launch of the dominant kernel; here a step is many launches of
    # different sizes, so the step as a whole stands in for it
    res["roofline"]["note"] = "whole step (one launch per parameter), not a single launch"
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline_sgd(1 << 24)
    return res


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="lans_bert_large_fp16grad")
    ap.add_argument("--schedule", default="auto", choices=["auto", "phased", "pipelined"],
                    help="LANS launch schedule (bit-identical results); auto = the library's choice")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-side baseline leg")
    ap.add_argument("--no-kernel-events", action="store_true", help="do not record per-kernel HIP events")
    ap.add_argument("--hip-graph", action="store_true",
                    help="LANS workloads: capture one step in a HIP graph and time its replays")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this path is built and measured on ONE GPU (no collectives, no sharding); "
                 "run with --gpus 1")
    if args.steps < 1 or args.warmup < 0:
        sys.exit("bench.py: --steps must be >= 1 and --warmup >= 0")
    table = workloads()
    if args.workload not in table:
        sys.exit(f"bench.py: unknown workload {args.workload!r}; choose from {sorted(table)}")
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    from raf_amd import _lib

    _lib.optim()  # fails loudly if the HIP library is not built
    wl = table[args.workload]
    fn = {"lans": bench_lans, "sgd": bench_sgd, "copy": bench_copy, "l2norm": bench_l2norm,
          "fuse": bench_fuse, "sgd_multi": bench_sgd_multi, "traced_sgd": bench_traced_sgd}[wl["kind"]]
    out = fn(args.workload, wl, args)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
