#!/usr/bin/env python3
"""Benchmark of the fused optimizer step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME|all]

A step is one pass of the hot path over one resident parameter set.  The headline workload is one
`raf.op.lans` step over a BERT-large-shaped list (391 tensors, 335,141,888 elements; fp32 weights
and state, fp16 gradients scaled by 1024 and unscaled in the kernel), called through the C ABI.
Inputs are synthetic (seeded, generated on the GPU) and resident in HBM before the timed region.

Prints ONE JSON line.  Its top-level fields are the headline workload's; `value` is algorithmic
bytes per step (the three-pass model: 46 B per element with fp16 gradients, 52 B with fp32) divided
by the wall time per step.  With the default `--workload all` the line also carries
  "configs"    every benchmark configuration (SGD on one tensor; LANS on the BERT-base, BERT-large,
               2000-small-tensor and GPT-2-1.5B lists): step time, the dominant kernel and its time
               from HIP events, its fraction of the 8 TB/s peak by the algorithmic (`frac`) and by
               the compulsory bytes (`frac_c`), the bytes per launch rocprofv3 measured (`traffic`);
  "entries"    for BERT-large and the small-tensor list, ms per step through each way into the
               step: the C ABI, the operator front end (`raf_amd.op.lans`: dialect dispatch ->
               OpEnv -> Execute) with a list handle, a plain list, new gradient objects every step,
               and the VM's calling pattern (a new tuple every step, gradients at alternating
               addresses), each with its difference to the C ABI in per cent;
  "neighbours" multi-tensor SGD, the traced optimizers after the dialect's graph rewrites, the
               mixed-precision step, l2norm, fuse and defuse: ms per step and fraction of the peak;
  "yardsticks" GB/s of plain torch streaming kernels on the same GPU in the same process (write,
               read+write, copy beyond the Infinity Cache; read+write and write inside it, with
               zeros and with other values), beside which the fractions above can be read;
  "parity"     a check of the very buffers that were timed, after the timed region, against the
               CPU oracle: SGD bit for bit, LANS w, m, v of whole tensors of the timed list by the
               strict per-element relative error (`max_rel`), the count of elements over the
               tolerance (`over_tol`) and of elements not bit-equal (`ne`).
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import re
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
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


_COMMENTS = re.compile(r"//[^\n]*|/\*.*?\*/", re.S)


def kernel_sources_digest() -> str:
    """Digest of the HIP sources the kernel library is built from, comments and white space aside: a
    traffic figure measured with rocprofv3 belongs to the kernels it was measured on."""
    from raf_amd import build

    h = hashlib.sha256()
    files = sorted([build.CSRC / s for s in build.OPTIM_SOURCES] + list(build.CSRC.glob("*.h")))
    for f in files:
        h.update(f.name.encode())
        h.update(" ".join(_COMMENTS.sub(" ", f.read_text()).split()).encode())
    return h.hexdigest()[:16]


_TRAFFIC_LINE = re.compile(r"^traffic: workload=(\S+) kernel=(\S+) bytes_per_launch=(\d+) kernel_sources=(\w+)\s*$")
_NO_TRAFFIC_LINE = re.compile(r"^no traffic figure: workload=(\S+) reason=(.+)$")


def measured_traffic(workload: str, kernel: str):
    """(bytes per launch or None, where that comes from).  The figures live in the rocprofv3
    summaries under profiles/ as lines `traffic: workload=... kernel=... bytes_per_launch=...
    kernel_sources=<digest>`; one measured on other kernel sources than the ones in the tree is not
    quoted."""
    try:
        now = kernel_sources_digest()
    except Exception as e:  # sources not shipped with the library
        return None, f"kernel sources not readable ({e})"
    stale = None
    for md in sorted((ROOT / "profiles").glob("*.md")):
        for line in md.read_text().splitlines():
            m = _TRAFFIC_LINE.match(line.strip())
            if m and m.group(1) == workload and m.group(2) == kernel:
                if m.group(4) == now:
                    return int(m.group(3)), f"profiles/{md.name} (rocprofv3 FETCH_SIZE + WRITE_SIZE, kernel sources {now})"
                stale = f"profiles/{md.name} holds a figure for other kernel sources ({m.group(4)}, tree is {now}): not quoted"
            m = _NO_TRAFFIC_LINE.match(line.strip())
            if m and m.group(1) == workload and stale is None:
                stale = f"not measured: {m.group(2)} (profiles/{md.name})"
    return None, stale or "not measured"


def roofline_obj(workload, kernel, bytes_per_launch, launch_ms, **extra):
    achieved = bytes_per_launch / (launch_ms * 1e-3) / 1e9
    traffic, source = measured_traffic(workload, kernel)
    obj = {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
           "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
           "traffic_source": source, "bytes_per_launch": bytes_per_launch,
           "avg_launch_ms": round(launch_ms, 5)}
    if traffic:
        obj["frac_by_measured_traffic"] = round(traffic / (launch_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)
    obj.update(extra)
    return obj


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
        # the traced optimizer's per-parameter op sequence after dialect fusion: one multi-tensor call
        "traced_sgd_fused_bert_large_fp32": dict(kind="traced_sgd", sizes=shapes.numels(shapes.bert_large_shapes())),
        # the traced LANS optimizer of a half-precision model after the graph rewrite: one lans_mixed call
        "traced_lans_mixed_bert_large_fp16": dict(kind="traced_lans", sizes=shapes.numels(shapes.bert_large_shapes())),
        # neighbours of the optimizer step that reuse its machinery
        "l2norm_bert_large_flat_fp32": dict(kind="l2norm", n=sum(shapes.numels(shapes.bert_large_shapes()))),
        "fuse_bert_large_fp32": dict(kind="fuse", sizes=shapes.numels(shapes.bert_large_shapes()), gather=True),
        "defuse_bert_large_fp32": dict(kind="fuse", sizes=shapes.numels(shapes.bert_large_shapes()), gather=False),
        # a plain device-to-device copy of known size: the yardstick that rocprofv3's FETCH_SIZE /
        # WRITE_SIZE counters are scaled by when HBM traffic is measured
        "copy_1gib": dict(kind="copy", nbytes=1 << 30),
        "stream_yardsticks": dict(kind="yardsticks"),
    }


def gen_lans(sizes, g16, zero_state, dev, seed=2024, flat=False):
    """Seeded synthetic tensors generated on the GPU.  `flat`: four flat buffers cut into views
    that start on 512-byte boundaries (where torch's allocator would put separate tensors): a
    handful of generator launches instead of two per tensor, for runs under a profiler."""
    import torch

    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    if flat:
        starts, total = [], 0
        for n in sizes:
            starts.append(total)
            total += -(-n // 128) * 128
        cut = lambda buf: [buf[s:s + n] for s, n in zip(starts, sizes)]
        gt = torch.randn(total, device=dev, generator=gen) * 1e-3
        g = cut((gt * 1024.0).half() if g16 else gt)
        w = cut(torch.randn(total, device=dev, generator=gen) * 0.02)
        if zero_state:
            return g, w, cut(torch.zeros(total, device=dev)), cut(torch.zeros(total, device=dev))
        return (g, w, cut(torch.randn(total, device=dev, generator=gen) * 1e-4),
                cut((torch.randn(total, device=dev, generator=gen) * 1e-6).abs()))
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


# ------------------------------------------------------------------ parity after the timed region
TOL_ONE_STEP = 1e-5     # max relative error per element after one step
TOL_100_STEPS = 1e-4    # ... and after up to 100 consecutive steps
PARITY_ELEMENT_BUDGET = 48_000_000  # elements followed on the CPU per LANS workload


def pick_parity_tensors(sizes):
    """Whole tensors of the timed list to follow on the CPU: the first, the last, the smallest, the
    median and the largest that fit the budget, then more from the front while the budget lasts
    (lists of small tensors are checked completely)."""
    order = sorted(range(len(sizes)), key=lambda t: sizes[t])
    wanted = [0, len(sizes) - 1, order[0], order[len(order) // 2]]
    big = [t for t in order if sizes[t] <= PARITY_ELEMENT_BUDGET // 2]
    if big:
        wanted.append(big[-1])
    picks, used = [], 0
    for t in wanted + list(range(len(sizes))):
        if t in picks or sizes[t] == 0 or used + sizes[t] > PARITY_ELEMENT_BUDGET:
            continue
        picks.append(t)
        used += sizes[t]
    return sorted(picks)


def error_metrics(got, ref, old_w=None, tol=TOL_ONE_STEP):
    """Strict max relative error, count of elements over the tolerance, and (for weights) the error
    relative to max(|reference|, |old weight|), which does not blow up where a weight lands next to
    zero."""
    got = got.astype(np.float64).ravel()
    ref = ref.astype(np.float64).ravel()
    d = np.abs(got - ref)
    with np.errstate(divide="ignore", invalid="ignore"):
        rel = np.where(d == 0.0, 0.0, d / np.abs(ref))
    out = {"max_rel": float(rel.max()) if rel.size else 0.0, "over_tol": int((rel > tol).sum()),
           "not_bit_equal": int((d != 0.0).sum())}
    if old_w is not None:
        floor = np.maximum(np.abs(ref), np.abs(old_w.astype(np.float64).ravel()))
        with np.errstate(divide="ignore", invalid="ignore"):
            out["max_floored"] = float(np.where(d == 0.0, 0.0, d / floor).max()) if d.size else 0.0
    return out


class LansParity:
    """Follows picked tensors of a LANS workload on the CPU.  Up to 100 steps the whole trajectory
    is recomputed from the initial state (the GPU's state after warm-up + timed steps is a
    deterministic function of it); beyond that, ONE more step is run on the GPU from the state the
    timed region left and compared with one oracle step from that same state."""

    def __init__(self, sizes, g, w, m, v, g16, step0, hp):
        self.picks = pick_parity_tensors(sizes)
        self.g16, self.step0, self.hp = g16, step0, hp
        self.host = lambda ts: [ts[t].cpu().numpy() for t in self.picks]
        self.g0, self.w0, self.m0, self.v0 = (self.host(x) for x in (g, w, m, v))
        self.elements = sum(sizes[t] for t in self.picks)

    def check(self, steps_done, g, w, m, v, one_more_step):
        import torch

        from oracle import c_oracle
        from oracle.lans_f64 import LansHParams

        threads = min(16, os.cpu_count() or 1, c_oracle.max_threads())
        ohp = LansHParams(learning_rate=self.hp.learning_rate, beta1=self.hp.beta1, beta2=self.hp.beta2,
                          eps=self.hp.eps, bias_correction=self.hp.bias_correction,
                          weight_decay=self.hp.weight_decay, grad_averaging=self.hp.grad_averaging,
                          mode=self.hp.mode, normalize_grad=bool(self.hp.normalize_grad),
                          grad_unscale=self.hp.grad_unscale)
        t0 = time.perf_counter()
        if steps_done <= 100:
            mode, tol = f"trajectory of {steps_done} steps from the initial state", (
                TOL_ONE_STEP if steps_done == 1 else TOL_100_STEPS)
            rw, rm, rv = [a.copy() for a in self.w0], [a.copy() for a in self.m0], [a.copy() for a in self.v0]
            old_w = [a.copy() for a in self.w0]
            for s in range(steps_done):
                if s == steps_done - 1:
                    old_w = [a.copy() for a in rw]
                c_oracle.lans_step_inplace(self.g0, rw, rm, rv, self.step0 + s, ohp, threads=threads)
        else:
            mode, tol = f"one more step from the state after {steps_done} steps", TOL_ONE_STEP
            torch.cuda.synchronize()
            rw, rm, rv = self.host(w), self.host(m), self.host(v)
            old_w = [a.copy() for a in rw]
            one_more_step()
            torch.cuda.synchronize()
            c_oracle.lans_step_inplace(self.g0, rw, rm, rv, self.step0 + steps_done, ohp, threads=threads)
        worst = {}
        for name, dev, ref, old in (("w", w, rw, old_w), ("m", m, rm, None), ("v", v, rv, None)):
            agg = {"max_rel": 0.0, "over_tol": 0, "not_bit_equal": 0}
            for i, t in enumerate(self.picks):
                e = error_metrics(dev[t].cpu().numpy(), ref[i], old[i] if old else None, tol)
                agg["max_rel"] = max(agg["max_rel"], e["max_rel"])
                agg["over_tol"] += e["over_tol"]
                agg["not_bit_equal"] += e["not_bit_equal"]
                if "max_floored" in e:
                    agg["max_floored"] = max(agg.get("max_floored", 0.0), e["max_floored"])
            worst[name] = {k: (float(f"{x:.3e}") if isinstance(x, float) else x) for k, x in agg.items()}
        g_intact = all(np.array_equal(g[t].cpu().numpy(), self.g0[i]) for i, t in enumerate(self.picks))
        ok = g_intact and all(worst[q]["over_tol"] == 0 and np.isfinite(worst[q]["max_rel"]) for q in "wmv")
        return {"ok": bool(ok), "against": "float64 C restatement of the rule (oracle/optim_oracle.c)",
                "mode": mode, "tolerance": tol, "tensors_checked": len(self.picks),
                "elements_checked": self.elements, "w": worst["w"], "m": worst["m"], "v": worst["v"],
                "gradient_untouched": bool(g_intact), "cpu_seconds": round(time.perf_counter() - t0, 2)}


def bench_lans(name, wl, args, entry="c_abi", parity=True, cpu_baseline=True):
    import torch

    from raf_amd import kernels, op

    dev = torch.device("cuda:0")
    sizes, g16 = wl["sizes"], wl["g16"]
    total = sum(sizes)
    g, w, m, v = gen_lans(sizes, g16, wl["zero_state"], dev, flat=getattr(args, "flat_inputs", False))
    hp = kernels.make_hparams(grad_unscale=(1.0 / 1024 if g16 else 1.0))
    copy16 = bool(wl.get("copy16"))
    p16 = [torch.empty(n, dtype=torch.float16, device=dev) for n in sizes] if copy16 else None
    step_t = torch.full((), float(wl["step0"]), dtype=torch.float32, device=dev)
    checker = LansParity(sizes, g, w, m, v, g16, wl["step0"], hp) if parity and not args.hip_graph else None

    plan = None
    if entry == "c_abi":
        # rafhip_lans_plan_bind once, then one rafhip_lans_step_bound per step
        plan = kernels.LansPlan(sizes, torch.float16 if g16 else torch.float32, dev)
        if args.schedule != "auto":
            plan.set_schedule(args.schedule)
        schedule = plan.schedule
        plan.bind(g, w, m, v, hp, p=p16)

        def one_step():
            plan.step_bound(step_t)
            step_t.add_(1.0)  # the step counter lives on the device, as in the reference's traced optimizer
    else:
        # raf.op.lans(tensor_list, step, ...) as the reference's LANS.step calls it
        # (python/raf/optim/lans.py:74-103): schema -> declare -> dialect dispatch -> OpEnv -> Execute.
        #   dialect              the list as a TensorList handle (the tuple value RAF's callers hold)
        #   dialect_list         a plain Python list of the same tensor objects every step
        #   dialect_fresh_grads  a plain list whose gradient objects are new at every step (same storage)
        #   vm_fresh_tuple       Execute receives a NEW TupleValue over the same tensor values at every
        #                        step, as the VM allocates one per iteration (src/impl/vm/vm.cc:764-769)
        #   vm_moving_grads      that, and the gradients alternate between two allocations every step,
        #                        as per-iteration allocation gives them (vm.cc:1099-1105)
        if args.schedule != "auto":
            os.environ["RAFHIP_LANS_SCHEDULE"] = args.schedule
        op.clear_op_env_cache()
        op.set_lans_grad_unscale(hp.grad_unscale)
        op.set_executor("vm" if entry.startswith("vm_") else "interpreter")
        rest = w + m + v + (p16 or [])
        call = op.lans_mixed if copy16 else op.lans
        schedule = args.schedule
        if entry == "dialect_list":
            lists = [g + rest]
        elif entry == "dialect_fresh_grads":
            # new tensor objects over the same gradient storage for every step, made before the clock starts
            lists = [[t.detach() for t in g] + rest for _ in range(args.warmup + args.steps + 4)]
        elif entry == "vm_moving_grads":
            first = op.TensorList(g + rest)
            lists = [first, first.replaced(0, [t.clone() for t in g])]  # same values at another address
        else:
            lists = [op.TensorList(g + rest)]
        calls_made = [0]

        def one_step():
            tensor_list = lists[calls_made[0] % len(lists)]
            calls_made[0] += 1
            call(tensor_list, step_t, hp.learning_rate, hp.beta1, hp.beta2, hp.eps, True, hp.weight_decay,
                 True, True, True)
            step_t.add_(1.0)

    steps_done = 0
    for _ in range(args.warmup):
        one_step()
    steps_done += args.warmup
    graph = None
    kernel_events = entry == "c_abi" and not args.no_kernel_events and not args.hip_graph
    if args.hip_graph:
        # The launches of one step (and the counter's increment) recorded once and replayed: what a
        # training loop captured in a HIP graph pays per step.  Per-kernel events stay outside.
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            one_step()
        for _ in range(3):
            graph.replay()
    if kernel_events:
        plan.timing_enable(args.steps)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        if graph is not None:
            graph.replay()
        else:
            one_step()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    steps_done += args.steps
    ms_per_step = wall * 1e3 / args.steps
    dev_ms_per_step = start.elapsed_time(stop) / args.steps  # events on the stream the steps run on

    a, b, c = lans_bytes_per_elt(2 if g16 else 4)
    ka, kb, kc = lans_kernel_bytes_per_elt(2 if g16 else 4)
    # phased: five launches, or three when the list fits the cache and no tensor has more than 32 chunks
    # (every workgroup then adds its tensor's few partial sums itself)
    lib = _libs()
    short = all(-(-n // lib.rafhip_lans_chunk_elements(n)) <= 32 for n in sizes if n)
    cached = total * (14 if g16 else 16) <= (192 << 20)
    if schedule == "auto":
        schedule = "pipelined" if total >= (64 << 20) else "phased"
    launches = 2 if schedule == "pipelined" else (3 if short and cached else 5)
    if copy16:  # the third pass also writes the 2-byte copy of the new weight
        c, kc = c + 2, kc + 2
    bytes_step = total * (a + b + c)
    out = {
        "metric": "LANS optimizer step: algorithmic bandwidth = three-pass model bytes "
                  f"({a + b + c} B per element) / step time, not bytes moved; ms_per_step is the step time",
        "value": round(bytes_step / (ms_per_step * 1e-3) / 1e9, 1),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64", "data": "synthetic",
        "config": {"workload": name, "entry": entry, "tensors": len(sizes), "elements": total,
                   "storage": "fp32 w/m/v, " + ("fp16 g (x1024, unscaled in kernel)" if g16 else "fp32 g") +
                              (", fp16 copy of the new weights written" if copy16 else ""),
                   "bytes_per_element": a + b + c, "bytes_per_step": bytes_step,
                   "kernel_bytes_per_element": ka + kb + kc, "compulsory_bytes_per_element": c,
                   "pct_of_peak_by_algorithmic_bytes": round(100 * bytes_step / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
                   "pct_of_peak_by_requested_bytes": round(100 * total * (ka + kb + kc) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
                   "pct_of_peak_by_compulsory_bytes": round(100 * total * c / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
                   "device_ms_per_step": round(dev_ms_per_step, 4),
                   "schedule": schedule, "launches_per_step": launches, "hip_graph": bool(args.hip_graph)},
    }
    if kernel_events:
        ts = np.array([plan.timing_read(i) for i in range(args.steps)], dtype=np.float64)
        avg = ts.mean(axis=0)
        if schedule == "phased":
            # dominant kernel: lans_apply (reads g,w,m,v, writes w,m,v)
            apply_ms = float(avg[4])
            out["roofline"] = roofline_obj(name, "lans_apply", total * c, apply_ms)
            out["kernels_ms"] = {"lans_norm_g": round(float(avg[0]), 4), "lans_finish(a)": round(float(avg[1]), 4),
                                 "lans_norm_u": round(float(avg[2]), 4), "lans_finish(b)": round(float(avg[3]), 4),
                                 "lans_apply": round(apply_ms, 4)}
            out["kernels_GBps"] = {"lans_norm_g": round(total * ka / avg[0] / 1e6, 1),
                                   "lans_norm_u": round(total * kb / avg[2] / 1e6, 1),
                                   "lans_apply": round(total * kc / avg[4] / 1e6, 1)}
        else:
            # one persistent kernel does all three passes; the same launch is also priced by the bytes
            # the kernel requests (the norm of w rides on pass B) and by the compulsory
            # read-once/write-once bytes
            k_ms = float(avg[1])
            out["roofline"] = roofline_obj(
                name, "lans_pipelined", bytes_step, k_ms,
                achieved_by_requested_bytes=round(total * (ka + kb + kc) / (k_ms * 1e-3) / 1e9, 1),
                achieved_by_compulsory_bytes=round(total * c / (k_ms * 1e-3) / 1e9, 1),
                frac_by_requested_bytes=round(total * (ka + kb + kc) / (k_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                frac_by_compulsory_bytes=round(total * c / (k_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4))
            out["kernels_ms"] = {"lans_prepare": round(float(avg[0]), 4), "lans_pipelined": round(k_ms, 4)}
    else:
        # no per-kernel events through this entry: the whole step on the device stands in for the launch
        out["roofline"] = roofline_obj(name, "lans step (all launches)", bytes_step, dev_ms_per_step,
                                       note="device time of the whole step between events on the step's stream")
    if checker is not None:
        out["parity"] = checker.check(steps_done, g, w, m, v, one_step)
    if entry != "c_abi":
        op.set_lans_grad_unscale(1.0)
        op.set_executor("interpreter")
        op.clear_op_env_cache()
        os.environ.pop("RAFHIP_LANS_SCHEDULE", None)
    if plan is not None:
        plan.close()
    if cpu_baseline and not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_lans(sizes, g16)
    return out


def bench_sgd(name, wl, args, parity=True, cpu_baseline=True):
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
    out = {
        "metric": "SGD momentum step: algorithmic bandwidth (20 B per element / step time)",
        "value": round(bytes_step / (ms_per_step * 1e-3) / 1e9, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": name, "entry": "c_abi", "elements": n, "bytes_per_element": SGD_BYTES_PER_ELT,
                   "compulsory_bytes_per_element": SGD_BYTES_PER_ELT, "buffer_sets_rotated": sets},
        "roofline": roofline_obj(name, "sgd_vec4_kernel", bytes_step, dev_ms),
    }
    if parity:
        # every element of the outputs of the timed calls, bit for bit: the op is out of place, so
        # each buffer set still holds the inputs its outputs were computed from
        from oracle import c_oracle

        bad, checked = 0, 0
        for x, dx, v, v1, x1 in bufs[:min(sets, args.warmup + args.steps)]:
            ov, ox = c_oracle.sgd_step(x.cpu().numpy(), dx.cpu().numpy(), v.cpu().numpy(), 0.01, 0.9, threads=8)
            bad += int((v1.cpu().numpy().view(np.uint32) != ov.view(np.uint32)).sum())
            bad += int((x1.cpu().numpy().view(np.uint32) != ox.view(np.uint32)).sum())
            checked += 2 * n
        out["parity"] = {"ok": bad == 0, "against": "fp32 C restatement, four roundings, no contraction (oracle/optim_oracle.c)",
                         "mode": "bit-exact comparison of v1 and x1 of every buffer set used", "elements_checked": checked,
                         "not_bit_equal": bad}
    if cpu_baseline and not args.no_cpu_baseline:
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
    return {
        "metric": metric, "value": round(bytes_step / (wall_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": dict(workload=name, **config),
        "roofline": roofline_obj(name, kernel, bytes_step, dev_ms),
    }


def bench_sgd_multi(name, wl, args):
    import torch

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
        from oracle import tensor_ops

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
                kernel, args, {"tensors": len(sizes), "elements": sum(sizes), "bytes_per_element": 8,
                               "bytes_read_per_step": plan.total_bytes,
                               "bytes_written_per_step": plan.total_bytes, "launches_per_step": 1})
    if not args.no_cpu_baseline:
        from oracle import tensor_ops

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
            "roofline": roofline_obj(name, "torch copy", moved, dev_ms)}


def stream_yardsticks(steps=30, warmup=5):
    """What plain streaming kernels of the framework underneath (torch's element-wise kernels and
    its device-to-device copy, not this library's code) reach on the same GPU in the same process:
    GB/s by the bytes each one reads plus writes.  They are the rates the memory system gives a
    read-only, a write-only and a read-and-write stream, beyond the Infinity Cache (1 GiB per
    array) and inside it (180 MiB in all, the footprint of the 2000-tensor list), and they show
    that a cache-resident stream of zeros is written faster than one of other values."""
    import torch

    dev = torch.device("cuda:0")

    def rate(fn, nbytes):
        for _ in range(warmup):
            fn()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(steps):
            fn()
        stop.record()
        torch.cuda.synchronize()
        return round(nbytes * steps / (start.elapsed_time(stop) * 1e-3) / 1e9)

    out = {}
    n = (1 << 30) // 4
    src, dst = torch.randn(n, device=dev), torch.empty(n, device=dev)
    out["torch_sum_1gib"] = rate(lambda: torch.sum(src), 4 * n)         # torch's own reduction: reads only
    out["write_1gib"] = rate(lambda: dst.fill_(1.2345), 4 * n)
    out["read_write_1gib"] = rate(lambda: torch.mul(src, 1.5, out=dst), 8 * n)
    out["copy_1gib"] = rate(lambda: dst.copy_(src), 8 * n)
    del src, dst
    n = (90 << 20) // 4                                                   # 90 MiB + 90 MiB: cache-resident
    src, dst = torch.randn(n, device=dev), torch.empty(n, device=dev)
    zeros = torch.zeros(n, device=dev)
    out["cached_read_write"] = rate(lambda: torch.mul(src, 1.5, out=dst), 8 * n)
    out["cached_read_write_zeros"] = rate(lambda: torch.mul(zeros, 1.5, out=dst), 8 * n)
    out["cached_write"] = rate(lambda: dst.fill_(1.2345), 4 * n)
    out["cached_write_zeros"] = rate(lambda: dst.fill_(0.0), 4 * n)
    out["unit"] = "GB/s"
    return out


def bench_traced_sgd(name, wl, args):
    """One step = the optimizer part of the reference's traced SGD optimizer over the whole model
    (per parameter: add(multiply(momentum, v), dx, out=v), subtract(w, multiply(lr, new_v), out=w)),
    taken through the FuseDialect pass: the hip dialect gathers every parameter's update into one
    raf.op.hip.sgd_multi call, i.e. one launch for the model."""
    import torch

    from raf_amd import op

    dev = torch.device("cuda:0")
    sizes = wl["sizes"]
    total = sum(sizes)
    gen = torch.Generator(dev).manual_seed(2024)
    x = [torch.randn(n, device=dev, generator=gen) * 0.02 for n in sizes]
    dx = [torch.randn(n, device=dev, generator=gen) * 1e-3 for n in sizes]
    v = [torch.zeros(n, device=dev) for n in sizes]
    opt = op.TracedSgdOptimizer(x, dx, v, 0.01, 0.9)
    calls = opt.ops
    wall_ms, dev_ms = _timed(lambda i: opt(), args)
    res = _line("traced SGD optimizer after dialect fusion: algorithmic bandwidth (20 B per element / step time)",
                name, "f32", total * SGD_BYTES_PER_ELT, wall_ms, dev_ms, "sgd_multi_kernel", args,
                {"tensors": len(sizes), "elements": total, "bytes_per_element": SGD_BYTES_PER_ELT,
                 "calls_in_fused_graph": calls, "launches_per_step": len(calls),
                 "unfused_kernels_per_step": 4 * len(sizes)})
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline_sgd(1 << 24)
    return res


def bench_traced_lans(name, wl, args):
    """One step = the optimizer part of the reference's traced LANS optimizer for a half-precision
    model (group_cast, raf.op.lans, and per parameter cast + add(out=p)), taken through the
    FuseDialect pass: the hip dialect's graph rewrite folds all of it into one raf.op.hip.lans_mixed
    call, executed through the C window; the step counter is advanced on the device."""
    import torch

    from raf_amd import op

    dev = torch.device("cuda:0")
    sizes = wl["sizes"]
    total = sum(sizes)
    g, w, m, v = gen_lans(sizes, True, True, dev)
    p16 = [torch.empty(n, dtype=torch.float16, device=dev) for n in sizes]
    step_t = torch.full((), 1.0, dtype=torch.float32, device=dev)
    op.set_lans_grad_unscale(1.0 / 1024)
    opt = op.TracedLansOptimizer(g, w, m, v, p16, step_t)
    calls = opt.ops

    def one_step(i):
        opt()
        step_t.add_(1.0)

    wall_ms, dev_ms = _timed(one_step, args)
    op.set_lans_grad_unscale(1.0)
    a, b, c = lans_bytes_per_elt(2)
    bytes_step = total * (a + b + c + 2)
    res = _line("traced mixed-precision LANS optimizer after the dialect's graph rewrite: algorithmic bandwidth "
                "(48 B per element / step time)", name, "f64", bytes_step, wall_ms, dev_ms,
                "lans step (all launches)", args,
                {"tensors": len(sizes), "elements": total, "bytes_per_element": a + b + c + 2,
                 "calls_in_fused_graph": calls,
                 "unfused_ops_per_step": 2 + 2 * len(sizes)})
    return res


def _short_traffic_source(source: str) -> str:
    """One token instead of the sentence, to keep the JSON line short: the summary's path, "stale"
    (measured on other kernel sources) or "unmeasured"."""
    if "other kernel sources" in source:
        return "stale"
    if source.startswith("profiles/"):
        return source.split(" ")[0]
    return "unmeasured"


def _config_entry(line):
    """What the "configs" block keeps of a workload's full line: step time, the dominant kernel and
    its time from HIP events, and its fraction of the 8 TB/s peak by algorithmic bytes (`frac`), by
    compulsory bytes (`frac_c`: every operand read once, every result written once) and by the
    traffic rocprofv3 measured (`traffic`, bytes per launch, or null)."""
    cfg, roof = line["config"], line["roofline"]
    comp = cfg.get("compulsory_bytes_per_element")
    launch_s = roof["avg_launch_ms"] * 1e-3
    entry = {"ms": line["ms_per_step"], "kernel": roof["kernel"], "kernel_ms": roof["avg_launch_ms"],
             "frac": roof["frac"], "frac_c": roof.get("frac_by_compulsory_bytes"), "traffic": roof["traffic"]}
    if entry["frac_c"] is None and comp and roof["kernel"] not in ("lans_apply",):
        entry["frac_c"] = round(cfg["elements"] * comp / launch_s / 1e9 / HBM_PEAK_GBPS, 4)
    if "kernels_ms" in line and cfg.get("schedule") == "phased":
        entry["kernels_ms"] = line["kernels_ms"]
    return entry


def _parity_entry(p):
    if p is None:
        return None
    if "w" not in p:  # SGD: bit-exact
        return {"ok": p["ok"], "n": p["elements_checked"], "ne": p["not_bit_equal"]}
    return {"ok": p["ok"], "n": p["elements_checked"], "tol": p["tolerance"],
            "max_rel": max(p[q]["max_rel"] for q in "wmv"), "over_tol": sum(p[q]["over_tol"] for q in "wmv"),
            "ne": sum(p[q]["not_bit_equal"] for q in "wmv")}


def run_suite(table, args):
    """Every benchmark configuration in one process, one after the other, each with its parity
    check; the headline workload first, and its line is the one whose fields go to the top level.
    The line stays well under 8 KB so that a log tail of that size holds all of it; per-workload
    detail is printed by `--workload NAME`."""
    import copy
    import gc

    import torch

    def release():
        gc.collect()
        torch.cuda.empty_cache()

    headline = "lans_bert_large_fp16grad"
    out = bench_lans(headline, table[headline], args, entry="c_abi", parity=True, cpu_baseline=True)
    configs = {headline: _config_entry(out)}
    parity = {headline: _parity_entry(out.pop("parity", None))}
    out["roofline"]["traffic_source"] = _short_traffic_source(out["roofline"]["traffic_source"])
    out["config"] = {k: out["config"][k] for k in ("workload", "entry", "tensors", "elements", "bytes_per_element",
                                                   "kernel_bytes_per_element", "compulsory_bytes_per_element",
                                                   "schedule", "launches_per_step")}
    out["metric"] = "LANS optimizer step, algorithmic bandwidth (46 B per element by the three-pass model / step time)"
    if "cpu_baseline" in out:
        out["cpu_baseline"]["sample"] = out["cpu_baseline"]["sample"].split(", float64")[0]
    release()

    def more_steps(k):
        a = copy.copy(args)
        a.steps, a.warmup = max(1, int(args.steps * k)), args.warmup
        return a

    def add(name, line):
        configs[name] = _config_entry(line)
        if "parity" in line:
            parity[name] = _parity_entry(line["parity"])
        release()

    add("sgd_4m_fp32", bench_sgd("sgd_4m_fp32", table["sgd_4m_fp32"], more_steps(4), parity=True, cpu_baseline=False))
    add("lans_bert_base_fp32", bench_lans("lans_bert_base_fp32", table["lans_bert_base_fp32"], args, cpu_baseline=False))
    small = "lans_2000_small_tensors"
    add(small, bench_lans(small, table[small], more_steps(4), cpu_baseline=False))
    big = copy.copy(args)
    big.steps, big.warmup = min(args.steps, 20), min(args.warmup, 5)  # 10 ms per step, 25 GB resident
    add("lans_gpt2_1p5b_fp32", bench_lans("lans_gpt2_1p5b_fp32", table["lans_gpt2_1p5b_fp32"], big, cpu_baseline=False))
    out["configs"] = configs

    # The ways into the same step, ms per step each and percent over the C ABI (no per-kernel events
    # in either, they cost a fifth of the 0.1 ms step): the operator front end with a TensorList
    # handle, with a plain list, with new gradient objects every step, and the VM's calling pattern.
    quiet = copy.copy(args)
    quiet.no_kernel_events = True
    entries = {}
    for base, steps_factor, variants in (
            (headline, 1, ("dialect", "vm_fresh_tuple", "vm_moving_grads")),
            (small, 4, ("dialect", "dialect_list", "dialect_fresh_grads", "vm_fresh_tuple", "vm_moving_grads"))):
        quiet.steps = max(1, int(args.steps * steps_factor))
        direct = bench_lans(base, table[base], quiet, parity=False, cpu_baseline=False)["ms_per_step"]
        release()
        block = {"c_abi": direct}
        for entry in variants:
            line = bench_lans(base, table[base], quiet, entry=entry, parity=entry != "dialect_list", cpu_baseline=False)
            block[entry] = line["ms_per_step"]
            block[entry + "_pct"] = round(100 * (line["ms_per_step"] / direct - 1), 1)
            if "parity" in line:
                parity[f"{base}@{entry}"] = _parity_entry(line["parity"])
            release()
        entries[base] = block
    out["entries"] = entries

    # The callers and neighbours either side of the path, timed in the same run (no parity here:
    # the GPU tests pin their bits): the traced optimizers after the dialect's graph rewrites beside
    # the C-ABI calls they end in, and the list operators.
    neighbours = {}
    quick = copy.copy(args)
    quick.no_cpu_baseline = True
    for name in ("sgd_multi_bert_large_fp32", "traced_sgd_fused_bert_large_fp32", "lans_bert_large_mixed_fp16",
                 "traced_lans_mixed_bert_large_fp16", "l2norm_bert_large_flat_fp32", "fuse_bert_large_fp32",
                 "defuse_bert_large_fp32"):
        wl = table[name]
        if wl["kind"] == "lans":
            line = bench_lans(name, wl, quick, parity=False, cpu_baseline=False)
        else:
            fn = {"l2norm": bench_l2norm, "fuse": bench_fuse, "sgd_multi": bench_sgd_multi,
                  "traced_sgd": bench_traced_sgd, "traced_lans": bench_traced_lans}[wl["kind"]]
            line = fn(name, wl, quick)
        neighbours[name] = {"ms": line["ms_per_step"], "frac": line["roofline"]["frac"]}
        release()
    out["neighbours"] = neighbours
    out["yardsticks"] = stream_yardsticks()
    release()
    parity["ok"] = all(p is None or p.get("ok", False) for p in parity.values())
    out["parity"] = parity
    return out


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all",
                    help="a workload name, or 'all' (default): the headline line plus every configuration and parity")
    ap.add_argument("--entry", default="c_abi",
                    choices=["c_abi", "dialect", "dialect_list", "dialect_fresh_grads", "vm_fresh_tuple",
                             "vm_moving_grads"],
                    help="LANS workloads: call the C ABI (bound plan), or the operator front end raf_amd.op.lans "
                         "with a TensorList handle (dialect), a plain list, a list with new gradient objects "
                         "every step, or the way RAF's VM calls an OpEnv (a new tuple value every step; "
                         "gradients alternating between two allocations)")
    ap.add_argument("--schedule", default="auto", choices=["auto", "phased", "pipelined"],
                    help="LANS launch schedule (bit-identical results); auto = the library's choice")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-side baseline leg")
    ap.add_argument("--no-parity", action="store_true", help="skip the parity check after the timed region")
    ap.add_argument("--no-kernel-events", action="store_true", help="do not record per-kernel HIP events")
    ap.add_argument("--flat-inputs", action="store_true",
                    help="LANS workloads: generate the list as four flat buffers cut into views (a few "
                         "generator launches instead of thousands; for runs under rocprofv3 --pmc)")
    ap.add_argument("--hip-graph", action="store_true",
                    help="LANS workloads: capture one step in a HIP graph and time its replays")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this path is built and measured on ONE GPU (no collectives, no sharding); "
                 "run with --gpus 1")
    if args.steps < 1 or args.warmup < 0:
        sys.exit("bench.py: --steps must be >= 1 and --warmup >= 0")
    table = workloads()
    if args.workload != "all" and args.workload not in table:
        sys.exit(f"bench.py: unknown workload {args.workload!r}; choose from {sorted(table)} or 'all'")
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    from raf_amd import _lib

    _lib.optim()  # fails loudly if the HIP library is not built
    if args.workload == "all":
        out = run_suite(table, args)
    else:
        wl = table[args.workload]
        if wl["kind"] == "lans":
            out = bench_lans(args.workload, wl, args, entry=args.entry, parity=not args.no_parity)
        elif wl["kind"] == "sgd":
            out = bench_sgd(args.workload, wl, args, parity=not args.no_parity)
        elif wl["kind"] == "yardsticks":
            out = {"workload": args.workload, **stream_yardsticks(args.steps, args.warmup)}
        else:
            fn = {"copy": bench_copy, "l2norm": bench_l2norm, "fuse": bench_fuse, "sgd_multi": bench_sgd_multi,
                  "traced_sgd": bench_traced_sgd, "traced_lans": bench_traced_lans}[wl["kind"]]
            out = fn(args.workload, wl, args)
    print(json.dumps(out), flush=True)
    parity = out.get("parity")
    if parity is not None and not parity.get("ok", True):
        sys.exit("bench.py: the parity check after the timed region FAILED; the figures above are invalid")


if __name__ == "__main__":
    main()
