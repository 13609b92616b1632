#!/usr/bin/env python3
"""Benchmark of the Hogwild! fused decode-attention step on one MI355X.

A "step" is one call of the fused operator (per-fragment q-RoPE + fragmented-KV GQA attention + LSE
merge) for one decoder layer of the QwQ-32B-shape, 4-worker workload.  Inputs are synthetic, generated
on the CPU from a fixed seed and resident in HBM before the timed region starts.

Cold-cache protocol: the K/V fragments exist in a ring of distinct copies totalling > 640 MB, and
consecutive steps walk the ring, so neither the L2 nor the 256 MiB Infinity Cache can serve a repeat.

Timing: the K steps (--steps) are captured as one HIP graph (launch overhead of a Python loop would
otherwise dominate a ~15 us step; the K steps are repeated until the graph holds at least 200) that is
replayed back to back at least 30 times and at least 2000 steps in total; every replay is bracketed by a
pair of HIP events on the stream the kernels run on.
`ms_per_step` is the median over the replays, p10 / p90 are reported next to it, so the figure does not
depend on --steps.  Before anything is timed the output of the first ring set is checked against the
CPU reference (the parity gate); the script exits non-zero if it fails.

Prints ONE JSON line.  `value` = algorithmic KV bytes per step / median time per step.  Under "extra":
the other workload configurations and the paged decode workload measured the same way, the hot-cache
figure, an eager Python loop, and a plain streaming-read calibration.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0   # MI355X published HBM3E bandwidth
METRIC = "KV-read HBM GB/s (% of peak) + µs/decode step, QwQ-32B shape, 4 workers"
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "hbm_traffic.json")   # rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summaries
MIN_REPLAYS = 30
MIN_TOTAL_STEPS = 2000


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--case", type=int, default=3, help="workload configuration 1..5 (3 = headline); 6 = the headline's fragments at head dimension 256")
    ap.add_argument("--splits", type=int, default=0, help="workgroups per kv head (0 = library default)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg (and with it the parity gate)")
    ap.add_argument("--no-rq", action="store_true", help="do not write the rotated-query side output")
    ap.add_argument("--no-extra", action="store_true", help="headline workload only: skip the other configurations under extra")
    ap.add_argument("--variant", choices=["mfma", "valu_qk"], default="mfma",
                    help="valu_qk = logits by VALU dot products instead of MFMA (configurations with at most 16 rows per kv head)")
    ap.add_argument("--profile-steps", type=int, default=0,
                    help="profiling mode for rocprofv3: run this many eager steps of the chosen workload over the cold ring plus the "
                         "calibration kernels, time nothing, print a short JSON line (graphs and the other legs are skipped)")
    ap.add_argument("--ring-mb", type=int, default=640)
    ap.add_argument("--workload", choices=["fragments", "paged", "varlen", "stack"], default="fragments",
                    help="fragments = the headline fused operator; paged = hogwild_paged_sdpa decode step at the same model shape; "
                         "varlen = hogwild_varlen_paged_sdpa on the same cache with 1 / 8 / 32 / 64 query tokens per sequence; "
                         "stack = the attention part of a 64-layer decode step through HogwildCache (append + attention + merge per "
                         "layer), eagerly and as one HIP graph")
    ap.add_argument("--layers", type=int, default=64, help="stack workload: decoder layers")
    ap.add_argument("--seq-len", type=int, default=12528, help="paged workload: tokens per sequence")
    ap.add_argument("--block-size", type=int, default=16, help="paged workload: tokens per cache block")
    ap.add_argument("--q-lens", default="1,8,32,64", help="varlen workload: query tokens of the four sequences")
    ap.add_argument("--row-blocks", type=int, default=0, help="paged workloads: 16-row blocks per workgroup (0 = the planner's choice; 8 = the 128-row kernel)")
    return ap.parse_args()


# ------------------------------------------------------------------------------------------------------------
# timing
# ------------------------------------------------------------------------------------------------------------
def pct(sorted_vals, p):
    return sorted_vals[min(len(sorted_vals) - 1, max(0, int(round(p * (len(sorted_vals) - 1)))))]


MIN_GRAPH_STEPS = 200   # a replay costs a few microseconds of its own: spread over at least this many steps


def time_graph(stream, step_fn, K, warmup=20, min_replays=MIN_REPLAYS, min_total=MIN_TOTAL_STEPS):
    """Capture step_fn(0..K-1) as one HIP graph on `stream` (the K steps repeated until the graph holds at least
    MIN_GRAPH_STEPS, so that what a replay itself costs does not depend on K), replay it back to back and time every
    replay with a pair of HIP events recorded on that stream.  Returns microseconds per step: dict(median, p10, p90,
    replays, graph_steps)."""
    import torch
    inner = max(1, math.ceil(MIN_GRAPH_STEPS / K))
    n = inner * K
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for i in range(n):
            step_fn(i)
    replays = max(min_replays, math.ceil(min_total / n))
    with torch.cuda.stream(stream):
        for _ in range(max(1, math.ceil(warmup / n))):
            graph.replay()
        torch.cuda.synchronize()
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(replays + 1)]
        evs[0].record(stream)
        for r in range(replays):
            graph.replay()
            evs[r + 1].record(stream)
        torch.cuda.synchronize()
    per = sorted(evs[r].elapsed_time(evs[r + 1]) * 1e3 / n for r in range(replays))
    del graph
    return {"median": per[len(per) // 2], "p10": pct(per, 0.10), "p90": pct(per, 0.90), "replays": replays, "graph_steps": n}


def load_traffic(key, with_commit=False):
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE and WRITE_SIZE in separate runs, each scaled by
    what the same counter reads for the copy kernel of known size this script launches); None when the workload was
    not measured.  The numbers live next to the rocprof summaries they come from, each with the commit of the kernel
    sources it was taken at."""
    try:
        with open(TRAFFIC_JSON) as fh:
            entry = json.load(fh).get(key)
        if entry is None:
            return (None, None) if with_commit else None
        return (int(entry["traffic_bytes"]), entry.get("commit")) if with_commit else int(entry["traffic_bytes"])
    except (OSError, ValueError, KeyError):
        return (None, None) if with_commit else None


def torch_op_leg(run, stream, K, warmup):
    """The operator a caller of the reference invokes, torch.ops.libhogatt.hogwild_fused (it sizes and allocates its
    split-K workspace from torch's caching allocator on every call): per-call time in a Python loop on one stream,
    synchronised at both ends, and of the same calls captured in a HIP graph.  Cold ring like everything else."""
    import torch
    from inference_lib_amd import attention
    if not attention.HAVE_TORCH_OPS:
        return None
    cd, case = run.cd, run.case
    frag = torch.tensor(case.lens, dtype=torch.int32, device=cd.q.device)

    def op(i):
        keys, vals = run.ring[i % run.n]
        torch.ops.libhogatt.hogwild_fused(run.out, run.rq, case.scale, cd.locations, cd.q, frag, keys, vals, cd.cos, cd.sin)

    with torch.cuda.stream(stream):
        for i in range(warmup):
            op(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(K):
            op(i)
        torch.cuda.synchronize()
        loop_us = (time.perf_counter() - t0) / K * 1e6
    graph = time_graph(stream, op, K, warmup=warmup, min_replays=10, min_total=1000)
    return {"python_loop": round(loop_us, 3), "hip_graph": round(graph["median"], 3),
            "what": "torch.ops.libhogatt.hogwild_fused (writes the rotated queries, allocates its workspace per call); "
                    "python_loop = K calls on one stream between two synchronisations, host-bound; hip_graph = the same calls "
                    "captured once and replayed"}


def bench_lib():
    """The calibration kernels (libhogwild_bench.so, include/hogwild_bench.h); not part of the product library."""
    path = os.path.join(ROOT, "inference_lib_amd", "libhogwild_bench.so")
    if not os.path.exists(path):
        raise SystemExit(f"{path} is missing: build it with `python -m inference_lib_amd.build`")
    lib = C.CDLL(path)
    lib.hw_stream_read.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p]
    lib.hw_stream_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
    lib.hw_stream_read_shaped.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_void_p]
    return lib


def make_ring(case, dev, ring_mb):
    """Distinct device copies of the KV fragments; q / locations / cos / sin are shared (tiny)."""
    import torch
    kvb = case.kv_bytes()
    n = max(2, math.ceil(ring_mb * 1e6 / kvb))
    ring = []
    for i in range(n):
        if i == 0:
            keys = [k.to(dev) for k in case.keys]
            vals = [v.to(dev) for v in case.values]
        else:
            # same distribution, different bytes: roll along the token axis (cheap, keeps N(0,1) statistics)
            keys = [torch.roll(k, shifts=i, dims=1).to(dev).contiguous() for k in case.keys]
            vals = [torch.roll(v, shifts=i, dims=1).to(dev).contiguous() for v in case.values]
        ring.append((keys, vals))
    return ring


class FragmentRun:
    """One workload configuration set up on the GPU: the ring of KV sets, one prepared hw_problem per set."""

    def __init__(self, case_id, dev, args, with_rq=True, variant=None):
        import torch
        from inference_lib_amd import _lib, cases
        self.case = case = cases.baseline_case(case_id)
        self.kv_bytes = case.kv_bytes()
        self.cd = cd = case.to(dev)
        self.ring = make_ring(case, dev, args.ring_mb)
        W, Hq, S, E = cd.q.shape
        tdt = cd.q.dtype
        self.out = torch.full((W, Hq, S, E), float("nan"), dtype=tdt, device=dev)
        self.lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=dev)
        self.rq = torch.empty((case.F, W, Hq, S, E), dtype=tdt, device=dev) if with_rq else None
        self.problems = []
        self.ws = None
        for keys, vals in self.ring:
            pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=keys, values=vals, scale=case.scale, out=self.out,
                              cosines=cd.cos, sines=cd.sin, rq=self.rq, lse=self.lse, splits=args.splits,
                              variant={"mfma": 0, "valu_qk": 1}[variant or args.variant])
            if self.ws is None:
                self.ws = torch.empty(pr.workspace_bytes(), dtype=torch.uint8, device=dev)
            pr.set_workspace(self.ws)
            self.problems.append(pr)
        self.n = len(self.problems)
        self.plan = _lib.plan(case.lens, W=case.W, S=case.S, Hq=case.Hq, Hkv=case.Hkv, Ev=case.E,
                              num_cus=_lib.lib.hw_device_cus(), splits=args.splits,
                              dtype={"f32": _lib.HW_F32, "f16": _lib.HW_F16, "bf16": _lib.HW_BF16}[case.dtype])

    def step(self, i):
        self.problems[i % self.n].run()

    def kernel(self, i):
        self.problems[i % self.n].run(stages=1)

    def hot(self, i):
        self.problems[0].run()

    def name(self):
        c = self.case
        return f"W={c.W} S={c.S} Hq={c.Hq} Hkv={c.Hkv} D={c.E} {c.dtype}, fragments={c.lens}"


# ------------------------------------------------------------------------------------------------------------
# parity gate + CPU baseline (the only leg that touches oracle/)
# ------------------------------------------------------------------------------------------------------------
def cpu_leg(run, stream):
    """The reference's eager PyTorch path (python/hogwild/attention.py:38-67 + :84-90) restated in oracle/: first as
    the checker of the GPU output of ring set 0 (parity gate, exits non-zero on failure), then timed on the host cores
    of this box as the reported baseline."""
    import torch
    from oracle import hogwild_oracle as O
    case = run.case
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    args = (case.q, case.locations, case.keys, case.values, case.scale, case.cos, case.sin)
    o_ref, l_ref = O.torch_reference_step(*args)          # fp32 reference on the same (already quantised) inputs

    with torch.cuda.stream(stream):
        run.out.fill_(float("nan"))
        run.lse.fill_(float("nan"))
        run.problems[0].run()
        torch.cuda.synchronize()
    got_o, got_l = run.out.float().cpu(), run.lse.cpu()
    err_o = float((got_o - o_ref).abs().max())
    err_l = float((got_l - l_ref).abs().max())
    scale_o = float(o_ref.abs().max())
    half = case.dtype != "f32"
    tol_ns = 2e-2 if half else 1e-4                        # the tolerance the task states: max-abs against an fp32 reference
    tol_o = (2.0 ** -7) * scale_o + 1e-3 if half else 1e-4  # relative to the signal (outputs of a long softmax are small)
    tol_l = 2e-3 if half else 1e-4
    ok = bool(torch.isfinite(got_o).all() and torch.isfinite(got_l).all()) and err_o <= min(tol_ns, tol_o) and err_l <= min(tol_ns, tol_l)
    parity = {"checked": f"out and lse of ring set 0 vs the fp32 CPU reference, {case.dtype}", "max_abs_err_out": err_o,
              "max_abs_err_lse": err_l, "max_abs_out_ref": scale_o, "tol_out": min(tol_ns, tol_o), "tol_lse": min(tol_ns, tol_l), "ok": ok}
    if not ok:
        print(json.dumps({"parity": parity}), file=sys.stderr)
        print("bench.py: parity gate failed, nothing timed", file=sys.stderr)
        sys.exit(4)

    for _ in range(2):
        O.torch_reference_step(*args)
    ts = []
    t_all = time.perf_counter()
    while (len(ts) < 10 or (time.perf_counter() - t_all) < 12.0) and (time.perf_counter() - t_all) < 30.0:   # about 12 s of CPU work
        t0 = time.perf_counter()
        O.torch_reference_step(*args)
        ts.append(time.perf_counter() - t0)
    ts.sort()
    med = ts[len(ts) // 2]
    baseline = {
        "value": round(run.kv_bytes / med / 1e9, 3),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "us_per_step": round(med * 1e6, 1),
        "sample": f"{len(ts)} full steps of the same workload (median), torch fp32 eager restatement of the reference path",
    }
    return parity, baseline


# ------------------------------------------------------------------------------------------------------------
# workloads
# ------------------------------------------------------------------------------------------------------------
def side_config(case_id, dev, args, stream):
    """Kernel / step time of another workload configuration, measured like the headline (fewer replays)."""
    import torch
    run = FragmentRun(case_id, dev, args)
    K = args.steps
    kw = dict(warmup=args.warmup, min_replays=10, min_total=1000)
    with torch.cuda.stream(stream):
        for i in range(5):
            run.step(i)
        torch.cuda.synchronize()
    step = time_graph(stream, run.step, K, **kw)
    kern = time_graph(stream, run.kernel, K, **kw)
    res = {"workload": f"config {case_id} ({run.case.name}): {run.name()}", "kv_bytes_per_step": run.kv_bytes,
           "workgroups": run.plan.workgroups, "kernel_us": round(kern["median"], 3), "step_us": round(step["median"], 3),
           "step_us_p10_p90": [round(step["p10"], 3), round(step["p90"], 3)],
           "kernel_frac_of_peak": round(run.kv_bytes / kern["median"] / 1e3 / PEAK_HBM_GBS, 4),
           "step_GBps": round(run.kv_bytes / step["median"] / 1e3, 1)}
    if run.plan.rows <= 16 and args.variant == "mfma" and run.case.E <= 128:
        # the matrix-core choice measured against VALU logits on the same workload (same ring, same plan)
        del run
        torch.cuda.empty_cache()
        run = FragmentRun(case_id, dev, args, variant="valu_qk")
        with torch.cuda.stream(stream):
            for i in range(5):
                run.step(i)
            torch.cuda.synchronize()
        res["valu_logits_kernel_us"] = round(time_graph(stream, run.kernel, K, **kw)["median"], 3)
        res["valu_logits_step_us"] = round(time_graph(stream, run.step, K, **kw)["median"], 3)
    del run
    torch.cuda.empty_cache()
    return res


def profile_mode(args, dev, stream, step_fn, kv_bytes, name):
    """What a rocprofv3 run of this script executes: eager launches only (a profiler serialises dispatches, so the
    replay timing above would take minutes and mean nothing), the workload walking its cold ring, then the streaming
    read and the 256 MiB copy whose known sizes scale the FETCH_SIZE / WRITE_SIZE counters."""
    import torch
    from inference_lib_amd import _lib
    blib = bench_lib()
    with torch.cuda.stream(stream):
        for i in range(5):
            step_fn(i)
        torch.cuda.synchronize()
        for i in range(args.profile_steps):
            step_fn(5 + i)
        torch.cuda.synchronize()
        big = torch.empty(2 * 256 * 1024 * 1024, dtype=torch.uint8, device=dev)
        big.random_(0, 255)
        sink = torch.zeros(256, dtype=torch.int32, device=dev)
        s_handle = C.c_void_p(stream.cuda_stream)
        half = 256 * 1024 * 1024
        for _ in range(3):
            _lib.check(blib.hw_stream_read(big.data_ptr(), big.numel(), sink.data_ptr(), s_handle), "hw_stream_read")
            _lib.check(blib.hw_stream_copy(big.data_ptr() + half, big.data_ptr(), half, s_handle), "hw_stream_copy")
        torch.cuda.synchronize()
        # the control of the counter passes: a bare read of the workload's own byte count in the attention kernel's launch
        # shape (one 256-thread workgroup per compute unit), walking the 512 MiB buffer
        kvb16 = kv_bytes // 16 * 16
        nbare = max(1, big.numel() // kvb16)
        cus = _lib.lib.hw_device_cus()
        for i in range(args.profile_steps):
            _lib.check(blib.hw_stream_read_shaped(big.data_ptr() + (i % nbare) * kvb16, kvb16, sink.data_ptr(), cus, s_handle),
                       "hw_stream_read_shaped")
        torch.cuda.synchronize()
    print(json.dumps({"profile_mode": True, "workload": name, "steps": args.profile_steps, "kv_bytes_per_step": kv_bytes,
                      "calibration": {"stream_read_bytes": 2 * half, "stream_copy_bytes_each_way": half}}))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no multi-GPU part); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from inference_lib_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.workload in ("paged", "varlen"):
        print(json.dumps(bench_paged(args, dev), ensure_ascii=False))
        return
    if args.workload == "stack":
        bench_stack(args, dev)
        return

    stream = torch.cuda.Stream()
    run = FragmentRun(args.case, dev, args, with_rq=not args.no_rq)
    case, cd, kv_bytes, problems, nring = run.case, run.cd, run.kv_bytes, run.problems, run.n
    W, Hq, S, E = cd.q.shape
    tdt = cd.q.dtype
    K, Wm = args.steps, args.warmup

    if args.profile_steps > 0:
        profile_mode(args, dev, stream, run.step, kv_bytes, f"config {args.case} ({case.name})")
        return

    parity, baseline = (None, None) if args.no_cpu else cpu_leg(run, stream)

    with torch.cuda.stream(stream):
        # ---------------- eager loop (launch-bound from Python; reported under extra) ----------------
        for i in range(Wm):
            run.step(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(K):
            run.step(i)
        torch.cuda.synchronize()
        eager_us = (time.perf_counter() - t0) / K * 1e6

    step = time_graph(stream, run.step, K, warmup=Wm)            # the headline: attention + merge, cold ring
    kern = time_graph(stream, run.kernel, K, warmup=Wm)          # the attention kernel alone (merge stage off)
    hot = time_graph(stream, run.hot, K, warmup=Wm, min_replays=10, min_total=1000)
    torch_op = torch_op_leg(run, stream, K, Wm) if run.rq is not None else None

    # ---------------- the same steps with the fragment lengths read from device memory ----------------
    len_dev = torch.tensor(case.lens, dtype=torch.int32, device=dev)
    problems_dl = []
    for keys, vals in run.ring:
        pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=keys, values=vals, scale=case.scale, out=run.out,
                          cosines=cd.cos, sines=cd.sin, rq=run.rq, lse=run.lse, splits=args.splits, len_dev=len_dev)
        pr.set_workspace(run.ws)
        problems_dl.append(pr)
    devlen = time_graph(stream, lambda i: problems_dl[i % nring].run(), K, warmup=Wm, min_replays=10, min_total=1000)

    # ---------------- the caller-side steps of a decode step at this shape (latency-bound, tiny) ----------------
    Hkv = cd.keys[0].size(0)
    seg_k = [torch.zeros((Hkv, 256, E), dtype=tdt, device=dev) for _ in range(W)]
    seg_v = [torch.zeros((Hkv, 256, E), dtype=tdt, device=dev) for _ in range(W)]
    k_new = torch.randn((W, S, Hkv, E), device=dev).to(tdt).transpose(1, 2)
    ck = torch.ones((W, S, E), dtype=tdt, device=dev)
    inv = torch.ones(E // 2, dtype=torch.float32, device=dev)
    pos_end = [[1000 + 7 * f + w for w in range(W)] for f in range(case.F)]
    small = dict(warmup=Wm, min_replays=10, min_total=1000)
    append = time_graph(stream, lambda i: _lib.rope_append(k_new, k_new, seg_k, seg_v, [i % 200] * W, cosines=ck, sines=ck), K, **small)
    build = time_graph(stream, lambda i: _lib.build_inputs(pos_end, S, inv, table_dtype=tdt if tdt != torch.float32 else None), K, **small)

    def layer(i):   # what one layer of a decode step launches: key rotation + append, then attention and merge (cold ring)
        _lib.rope_append(k_new, k_new, seg_k, seg_v, [i % 200] * W, cosines=ck, sines=ck)
        run.step(i)
    layer_t = time_graph(stream, layer, K, **small)

    # ---------------- plain streaming read of the whole ring (achievable HBM rate) ----------------
    blib = bench_lib()
    with torch.cuda.stream(stream):
        big = torch.empty(int(args.ring_mb * 1e6) // 16 * 16, dtype=torch.uint8, device=dev)
        big.random_(0, 255)
        sink = torch.zeros(256, dtype=torch.int32, device=dev)
        s_handle = C.c_void_p(stream.cuda_stream)
        for _ in range(2):
            _lib.check(blib.hw_stream_read(big.data_ptr(), big.numel(), sink.data_ptr(), s_handle), "hw_stream_read")
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(5):
            _lib.check(blib.hw_stream_read(big.data_ptr(), big.numel(), sink.data_ptr(), s_handle), "hw_stream_read")
        e1.record(stream)
        torch.cuda.synchronize()
        stream_gbs = big.numel() * 5 / (e0.elapsed_time(e1) * 1e-3) / 1e9
        # a plain copy of known size (256 MiB read + 256 MiB written): the reference point that scales the
        # FETCH_SIZE / WRITE_SIZE hardware counters when this command runs under rocprofv3 --pmc
        half = 256 * 1024 * 1024
        for _ in range(2):
            _lib.check(blib.hw_stream_copy(big.data_ptr() + half, big.data_ptr(), half, s_handle), "hw_stream_copy")
        torch.cuda.synchronize()
    # launches of the kernel's own byte count walking the same amount of cold memory: what a bare read of these bytes costs
    kvb16 = kv_bytes // 16 * 16
    nbare = max(2, big.numel() // kvb16)
    bare = time_graph(stream, lambda i: _lib.check(blib.hw_stream_read(big.data_ptr() + (i % nbare) * kvb16, kvb16, sink.data_ptr(),
                                                                       C.c_void_p(stream.cuda_stream)), "hw_stream_read"), K, **small)
    cus = _lib.lib.hw_device_cus()
    bare_shape = time_graph(stream, lambda i: _lib.check(blib.hw_stream_read_shaped(big.data_ptr() + (i % nbare) * kvb16, kvb16, sink.data_ptr(), cus,
                                                                                    C.c_void_p(stream.cuda_stream)), "hw_stream_read_shaped"), K, **small)
    del big

    graph_us = step["median"]
    value = kv_bytes / (graph_us * 1e-6) / 1e9
    achieved = kv_bytes / (kern["median"] * 1e-6) / 1e9
    result = {
        "metric": METRIC,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": Wm,
        "ms_per_step": round(graph_us * 1e-3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": case.dtype,
        "data": "synthetic",
        "config": {
            "workload": f"config {args.case} ({case.name}): {run.name()}",
            "kv_bytes_per_step": kv_bytes,
            "visible_tokens": case.visible_tokens(),
            "cold_cache_ring_sets": nring,
            "workgroups": run.plan.workgroups,
            "wgs_per_head": run.plan.wgs_per_head,
            "writes_rotated_q": run.rq is not None,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": PEAK_HBM_GBS,
            "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM_GBS, 4),
            "traffic": load_traffic(f"attention_kernel/{case.name}"),
            "traffic_commit": load_traffic(f"attention_kernel/{case.name}", with_commit=True)[1],
            "kernel": "hw::attention_wide_kernel" if run.plan.row_blocks == 8 else "hw::attention_kernel",
            "kernel_us_avg": round(kern["median"], 3),
            "kernel_us_p10_p90": [round(kern["p10"], 3), round(kern["p90"], 3)],
            "timing": f"HIP event pairs around each of {kern['replays']} back-to-back replays of a graph of K attention-kernel launches "
                      "(merge stage off) on the kernels' stream; median per launch",
        },
        "extra": {
            "us_per_step": round(graph_us, 3),
            "us_per_step_p10_p90": [round(step["p10"], 3), round(step["p90"], 3)],
            "graph_replays_timed": step["replays"],
            "steps_per_graph": step["graph_steps"],
            "pct_of_peak": round(100.0 * value / PEAK_HBM_GBS, 2),
            "eager_loop_us_per_step": round(eager_us, 3),
            "torch_op_us_per_step": torch_op,
            "hot_cache_us_per_step": round(hot["median"], 3),
            "device_lengths_us_per_step": round(devlen["median"], 3),
            "hot_cache_GBps": round(kv_bytes / (hot["median"] * 1e-6) / 1e9, 1),
            "stream_read_GBps": round(stream_gbs, 1),
            "bare_read_us_per_launch": {"bytes": kvb16, "us": round(bare["median"], 3)},
            "bare_read_in_launch_shape_us": {"bytes": kvb16, "workgroups": cus, "us": round(bare_shape["median"], 3),
                                             "what": "the same bytes read by one 256-thread workgroup per compute unit, the attention kernel's launch shape"},
            "rope_append_us_per_call": round(append["median"], 3),
            "build_inputs_us_per_call": round(build["median"], 3),
            "append_plus_attention_us_per_layer": round(layer_t["median"], 3),
            "timing": f"K steps captured as one HIP graph, replayed {step['replays']} times back to back, each replay between two HIP "
                      "events on the kernels' stream; median / p10 / p90 over the replays",
        },
    }
    if parity is not None:
        result["extra"]["parity_gate"] = parity
    else:
        result["extra"]["parity_gate"] = "skipped (--no-cpu)"

    if not args.no_extra:
        del run, problems, problems_dl
        torch.cuda.empty_cache()
        cfgs = []
        for cid in (1, 2, 4, 5, 6):
            if cid != args.case:
                cfgs.append(side_config(cid, dev, args, stream))
        for wl in ("paged", "varlen"):
            pargs = argparse.Namespace(**vars(args))
            pargs.workload, pargs.no_cpu = wl, True
            pg = bench_paged(pargs, dev, quick=True)
            cfgs.append({"workload": pg["config"]["workload"], "kv_bytes_per_step": pg["config"]["kv_bytes_per_step"],
                         "workgroups": pg["config"]["workgroups"], "kernel": pg["roofline"]["kernel"],
                         "kernel_us": pg["roofline"]["kernel_us_avg"],
                         "step_us": pg["extra"]["us_per_step"], "step_us_p10_p90": pg["extra"]["us_per_step_p10_p90"],
                         "kernel_frac_of_peak": pg["roofline"]["frac"], "step_GBps": pg["value"]})
            del pg
            torch.cuda.empty_cache()
        result["extra"]["configs"] = cfgs

    if baseline is not None:
        result["cpu_baseline"] = baseline
    print(json.dumps(result, ensure_ascii=False))


def bench_paged(args, dev, quick=False):
    """One decode step of hogwild_paged_sdpa: 4 sequences of --seq-len tokens each in a paged bf16 cache (blocks of
    --block-size tokens, shuffled), QwQ-32B head shape, one query token per sequence.  Every sequence has its own KV,
    so a step reads W * seq_len * Hkv * (E + Ev) * 2 bytes.  Cold cache: consecutive steps use block tables that point
    at disjoint parts of the cache."""
    import torch
    from inference_lib_amd import _lib
    W, Hq, Hkv, D, S, F = 4, 40, 8, 128, 1, 1
    L, bs = args.seq_len, args.block_size
    nblk = (L + bs - 1) // bs
    kv_bytes = W * L * Hkv * 2 * D * 2
    nring = max(2, math.ceil(args.ring_mb * 1e6 / kv_bytes))
    NB = nring * W * nblk
    g = torch.Generator(device=dev).manual_seed(7)
    kc = torch.randn((NB, Hkv, bs, D), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    vc = torch.randn((NB, Hkv, bs, D), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    perm = torch.randperm(NB, generator=torch.Generator().manual_seed(8)).to(torch.int32)
    varlen = args.workload == "varlen"
    cu = None
    if varlen:   # packed queries: the last 1 / 8 / 32 / 64 positions of the four sequences (causal)
        q_lens = [int(x) for x in args.q_lens.split(",")]
        assert len(q_lens) == W and all(0 <= n <= L for n in q_lens), "--q-lens takes four lengths"
        T = sum(q_lens)
        cu = torch.tensor([0] + [sum(q_lens[:i + 1]) for i in range(W)], dtype=torch.int32, device=dev)
        q = torch.randn((F, T, Hq, D), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        loc = torch.cat([torch.arange(L - n, L, dtype=torch.int32) for n in q_lens]).reshape(F, T).to(dev)
        fl = torch.full((F, W), L, dtype=torch.int32, device=dev)
        out = torch.empty((T, Hq, D), dtype=torch.bfloat16, device=dev)
        lse = torch.empty((T, Hq), dtype=torch.float32, device=dev)
    else:
        q = torch.randn((F, W, Hq, S, D), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        loc = torch.full((F, W, S), L - 1, dtype=torch.int32, device=dev)
        fl = torch.full((F,), L, dtype=torch.int32, device=dev)
        out = torch.empty((W, Hq, S, D), dtype=torch.bfloat16, device=dev)
        lse = torch.empty((W, Hq, S), dtype=torch.float32, device=dev)
    scale = 1.0 / math.sqrt(D)
    problems, tables = [], []
    ws = None
    for i in range(nring):
        bt = perm[i * W * nblk:(i + 1) * W * nblk].reshape(W, nblk).contiguous().to(dev)
        tables.append(bt)
        pr = _lib.PagedProblem(q=q, locations=loc, fragment_lengths=fl, key_cache=kc, value_cache=vc, block_table=bt,
                               scale=scale, out=out, lse=lse, splits=args.splits, cu_seqlens_q=cu, row_blocks=args.row_blocks)
        if ws is None:
            ws = torch.empty(pr.workspace_bytes(), dtype=torch.uint8, device=dev)
        pr.set_workspace(ws)
        problems.append(pr)
    plan = _lib.paged_plan(W=W, Hq=Hq, Hkv=Hkv, Ev=D, block_size=bs, max_blocks=nblk, num_cus=_lib.lib.hw_device_cus(), S=S,
                           splits=args.splits, total_q=(q.size(1) if varlen else None), row_blocks=args.row_blocks)
    K, Wm = args.steps, args.warmup
    if getattr(args, "profile_steps", 0) > 0 and not quick:
        profile_mode(args, dev, torch.cuda.Stream(), lambda i: problems[i % nring].run(), kv_bytes, "paged " + args.workload)
        sys.exit(0)
    kw = dict(warmup=Wm, min_replays=10, min_total=1000) if quick else dict(warmup=Wm)
    small = dict(warmup=Wm, min_replays=10, min_total=1000)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(Wm):
            problems[i % nring].run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(K):
            problems[i % nring].run()
        torch.cuda.synchronize()
        eager_us = (time.perf_counter() - t0) / K * 1e6
    step = time_graph(stream, lambda i: problems[i % nring].run(), K, **kw)
    kern = time_graph(stream, lambda i: problems[i % nring].run(stages=1), K, **kw)
    hot_us = copy_us = None
    if not quick:
        hot_us = time_graph(stream, lambda i: problems[0].run(), K, **small)["median"]
        # the append that precedes every decode step: one new token per sequence into the paged cache
        ks = torch.randn((W, 1, Hkv, D), device=dev).to(torch.bfloat16).transpose(1, 2)
        seq = torch.full((W,), L - 1, dtype=torch.int32, device=dev)
        copy_us = time_graph(stream, lambda i: _lib.copy_to_blocks(ks, ks, kc, vc, tables[i % nring], seq), K, **small)["median"]

    graph_us, kern_us = step["median"], kern["median"]
    value = kv_bytes / (graph_us * 1e-6) / 1e9
    achieved = kv_bytes / (kern_us * 1e-6) / 1e9
    result = {
        "metric": "KV-read HBM GB/s (% of peak) + µs/decode step, QwQ-32B shape, 4 sequences, paged KV cache"
                  + (", packed variable-length queries" if varlen else ""),
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": Wm,
        "ms_per_step": round(graph_us * 1e-3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": (f"varlen paged: W={W} sequences x {L} tokens, query tokens per sequence {args.q_lens.replace(',', '/')}, " if varlen else
                                f"paged decode: W={W} sequences x {L} tokens, S={S}, ") + f"Hq={Hq} Hkv={Hkv} D={D} bf16, block_size={bs}, F={F}", "kv_bytes_per_step": kv_bytes, "cold_cache_ring_sets": nring,
                   "workgroups": plan.workgroups, "splits": plan.splits},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4),
                     "traffic": load_traffic((("paged_wide_kernel" if plan.row_blocks == 8 else "paged_attention_kernel") +
                                              ("/varlen" if varlen else "/decode")) + f"_{L}_{bs}"),
                     "kernel": "hw::paged_wide_kernel" if plan.row_blocks == 8 else "hw::paged_attention_kernel",
                     "kernel_us_avg": round(kern_us, 3),
                     "kernel_us_p10_p90": [round(kern["p10"], 3), round(kern["p90"], 3)],
                     "timing": f"HIP event pairs around each of {kern['replays']} back-to-back replays of a graph of K attention-kernel launches "
                               "(merge stage off); median per launch"},
        "extra": {"us_per_step": round(graph_us, 3), "us_per_step_p10_p90": [round(step["p10"], 3), round(step["p90"], 3)],
                  "pct_of_peak": round(100.0 * value / PEAK_HBM_GBS, 2), "eager_loop_us_per_step": round(eager_us, 3),
                  "hot_cache_us_per_step": None if hot_us is None else round(hot_us, 3),
                  "copy_to_blocks_us": None if copy_us is None else round(copy_us, 3)},
    }
    if not args.no_cpu:
        from oracle import paged_oracle as po
        qn, kn, vn = q.float().cpu().numpy(), kc.float().cpu().numpy(), vc.float().cpu().numpy()
        ts = []
        t_all = time.perf_counter()
        while (len(ts) < 5 or (time.perf_counter() - t_all) < 12.0) and (time.perf_counter() - t_all) < 30.0:   # about 12 s of CPU work
            t0 = time.perf_counter()
            if varlen:
                po.varlen_paged_sdpa(qn, loc.cpu().numpy(), fl.cpu().numpy(), kn, vn, tables[0].cpu().numpy(), cu.cpu().numpy(), scale,
                                     dtype=np_f32())
            else:
                po.paged_sdpa(qn, loc.cpu().numpy(), fl.cpu().numpy(), kn, vn, tables[0].cpu().numpy(), scale, dtype=np_f32())
            ts.append(time.perf_counter() - t0)
        med = sorted(ts)[len(ts) // 2]
        cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
        cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
        result["cpu_baseline"] = {"value": round(kv_bytes / med / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
                                  "us_per_step": round(med * 1e6, 1),
                                  "sample": f"{len(ts)} full steps of the same workload (median), numpy fp32 restatement of the paged kernel"}
    del problems, kc, vc
    torch.cuda.empty_cache()
    return result


def bench_stack(args, dev):
    """The attention part of one decode step of a whole model at the headline shape: per layer the new keys are rotated
    and appended to every worker's segment (hw_rope_append), then attention + merge (hogwild_fused); at layer 0 the
    step's locations and rotary tables are built.  Every layer has its own KV buffers (prompt of 4096 tokens, four
    worker segments of 2048), so a step streams layers x 51 MB.  Three ways of driving it: eagerly from Python with
    host-side lengths, eagerly with the lengths in device memory, and the latter captured once as a HIP graph and
    replayed.  `value` is the graph replay."""
    import torch
    from inference_lib_amd import attention, cache
    L, W, Hq, Hkv, D, S = args.layers, 4, 40, 8, 128, 1
    tdt = torch.bfloat16
    seg_lens = [4096, 2048, 2048, 2048, 2048]
    inv = (1e6 ** (-torch.arange(0, D, 2, dtype=torch.float32) / D)).to(dev)
    orders = [[0] + [1 + o for o in range(W) if o != w] + [1 + w] for w in range(W)]

    def make():
        segs = [cache.SegmentCache(L, Hkv, D, n + 160, dtype=tdt, device=dev) for n in seg_lens]
        for sg, n in zip(segs, seg_lens):
            sg.lengths = [n] * L
            for layer in range(L):
                sg.k[layer].normal_()
                sg.v[layer].normal_()
        return cache.HogwildCache([[segs[i] for i in o] for o in orders], inv_freq=inv)

    q = torch.randn((W, Hq, S, D), device=dev).to(tdt)
    kn = torch.randn((W, S, Hkv, D), device=dev).to(tdt).transpose(1, 2)
    vn = torch.randn((W, S, Hkv, D), device=dev).to(tdt).transpose(1, 2)
    ids = torch.zeros((W, S), dtype=torch.int64, device=dev)

    def step(hc):
        pos = hc.get_input_kwargs(ids)["position_ids"]
        ang = pos.to(torch.float32)[..., None] * inv
        emb = torch.cat([ang, ang], dim=-1)
        ck, sk = emb.cos().to(tdt), emb.sin().to(tdt)
        for layer in range(L):
            cs = hc.update_fused(kn, vn, ck, sk, layer)
            rq = hc.get_queries_buffer(q, layer)
            attention.hogwild_fused(q, cs.loc, cs.keys, cs.values, D ** -0.5, cs.frags, cs.cos, cs.sin, rotated_queries=rq,
                                    out=hc.get_att_buffer(rq, layer), device_lengths=hc.device_lengths)

    K, Wm = min(args.steps, 40), min(args.warmup, 5)

    def timed(fn, n):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e6

    hc_a = make()
    for _ in range(Wm):
        step(hc_a)
    eager_host_us = timed(lambda: step(hc_a), K)
    del hc_a
    hc_b = make()
    hc_b.use_device_lengths(headroom=2 * (K + Wm) + 8)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        for _ in range(Wm):
            step(hc_b)
        eager_dev_us = timed(lambda: step(hc_b), K)
        with torch.cuda.graph(graph, stream=stream):
            step(hc_b)
        for _ in range(Wm):
            graph.replay()
        graph_us = timed(graph.replay, K)
    left = hc_b.device_steps_left()
    assert left >= 0, "replayed beyond the planned lengths"
    kv_bytes = L * sum(seg_lens) * Hkv * 2 * D * 2
    value = kv_bytes / (graph_us * 1e-6) / 1e9
    result = {
        "metric": METRIC + f", attention part of a {L}-layer decode step (key rotation + append, attention, merge per layer)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": Wm, "ms_per_step": round(graph_us / 1e3, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"decode stack: {L} layers, W=4 S=1 Hq=40 Hkv=8 D=128 bf16, segments {seg_lens} per layer, "
                               "lengths in device memory, one HIP graph per step", "kv_bytes_per_step": kv_bytes},
        "roofline": {"bound": "hbm", "achieved": round(value, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(value / PEAK_HBM_GBS, 4), "traffic": None, "kernel": "whole step (3 kernels per layer)",
                     "timing": "wall clock around K graph replays"},
        "extra": {"graph_us_per_layer": round(graph_us / L, 2), "eager_device_lengths_us_per_layer": round(eager_dev_us / L, 2),
                  "eager_host_lengths_us_per_layer": round(eager_host_us / L, 2), "planned_steps_left": left},
    }
    print(json.dumps(result, ensure_ascii=False))


def np_f32():
    import numpy as np
    return np.float32


if __name__ == "__main__":
    main()
