#!/usr/bin/env python3
"""Benchmark of the Hogwild! fused decode-attention step on one MI355X.

A "step" is one call of the fused operator (per-fragment q-RoPE + fragmented-KV GQA attention + LSE
merge) for one decoder layer of the QwQ-32B-shape, 4-worker workload.  Inputs are synthetic, generated
on the CPU from a fixed seed and resident in HBM before the timed region starts.

Cold-cache protocol: the K/V fragments exist in a ring of distinct copies totalling > 640 MB, and
consecutive steps walk the ring, so neither the L2 nor the 256 MiB Infinity Cache can serve a repeat.

Prints ONE JSON line.  `value` = algorithmic KV bytes per step / measured time per step, where the K
steps are replayed from one HIP graph (launch overhead of a Python loop would otherwise dominate a
~10 us step); the eager-loop figure, the hot-cache figure and a plain streaming-read calibration are
reported under "extra".
"""
from __future__ import annotations

import argparse
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

# HBM bytes per launch of the attention kernel measured with rocprofv3 --pmc (FETCH_SIZE and WRITE_SIZE in
# separate runs, each scaled by what the same counter reads for the 256 MiB copy kernel this script launches:
# 0.5 for FETCH_SIZE, 1.0 for WRITE_SIZE): 51.83 MB fetched + 3.03 MB written.  Workloads not measured: None.
MEASURED_TRAFFIC_BYTES = {"c3_qwq32b_w4": 54_860_000}
# the same for hw::paged_attention_kernel at the default paged workload (4 x 12528 tokens, blocks of 16): 205.69 MB + 0.67 MB
MEASURED_PAGED_TRAFFIC_BYTES = {(12528, 16): 206_360_000}
# packed variable-length workload on the same cache: 383.36 MB fetched (1.87 x the algorithmic bytes: L2 and the Infinity
# Cache serve most but not all of the 20 row groups' repeats) + 10.92 MB of split-K partials written
MEASURED_VARLEN_TRAFFIC_BYTES = {(12528, 16): 394_280_000}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--case", type=int, default=3, help="workload configuration 1..5 (3 = headline)")
    ap.add_argument("--splits", type=int, default=0, help="workgroups per kv head (0 = library default)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-rq", action="store_true", help="do not write the rotated-query side output")
    ap.add_argument("--ring-mb", type=int, default=640)
    ap.add_argument("--workload", choices=["fragments", "paged", "varlen", "stack"], default="fragments",
                    help="fragments = the headline fused operator; paged = hogwild_paged_sdpa decode step at the same model shape; "
                         "varlen = hogwild_varlen_paged_sdpa on the same cache with 1 / 8 / 32 / 64 query tokens per sequence; "
                         "stack = the attention part of a 64-layer decode step through HogwildCache (append + attention + merge per "
                         "layer), eagerly and as one HIP graph")
    ap.add_argument("--layers", type=int, default=64, help="stack workload: decoder layers")
    ap.add_argument("--seq-len", type=int, default=12528, help="paged workload: tokens per sequence")
    ap.add_argument("--block-size", type=int, default=16, help="paged workload: tokens per cache block")
    return ap.parse_args()


def make_ring(case, dev, ring_mb):
    """Distinct device copies of the KV fragments; q / locations / cos / sin are shared (tiny)."""
    import torch
    kvb = case.kv_bytes()
    n = max(2, math.ceil(ring_mb * 1e6 / kvb))
    ring = []
    g = torch.Generator().manual_seed(1234)
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


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no multi-GPU part); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from inference_lib_amd import _lib, cases

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.workload in ("paged", "varlen"):
        bench_paged(args, dev)
        return
    if args.workload == "stack":
        bench_stack(args, dev)
        return

    case = cases.baseline_case(args.case)
    kv_bytes = case.kv_bytes()
    cd = case.to(dev)
    ring = make_ring(case, dev, args.ring_mb)
    W, Hq, S, E = cd.q.shape
    tdt = cd.q.dtype

    out = torch.empty((W, Hq, S, E), dtype=tdt, device=dev)
    lse = torch.empty((W, Hq, S), dtype=torch.float32, device=dev)
    rq = None if args.no_rq else torch.empty((case.F, W, Hq, S, E), dtype=tdt, device=dev)
    problems = []
    ws = None
    for keys, vals in ring:
        pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=keys, values=vals, scale=case.scale, out=out,
                          cosines=cd.cos, sines=cd.sin, rq=rq, lse=lse, splits=args.splits)
        if ws is None:
            ws = torch.empty(pr.workspace_bytes(), dtype=torch.uint8, device=dev)
        pr.set_workspace(ws)
        problems.append(pr)
    nring = len(problems)
    plan = _lib.plan(case.lens, W=case.W, S=case.S, Hq=case.Hq, Hkv=case.Hkv, Ev=case.E,
                     num_cus=_lib.lib.hw_device_cus(), splits=args.splits)

    K, Wm = args.steps, args.warmup
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        # ---------------- eager loop (launch-bound from Python; reported under extra) ----------------
        for i in range(Wm):
            problems[i % nring].run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(K):
            problems[i % nring].run()
        torch.cuda.synchronize()
        eager_us = (time.perf_counter() - t0) / K * 1e6

        # ---------------- HIP graph of exactly K steps walking the ring ----------------
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(K):
                problems[i % nring].run()
        for _ in range(max(1, Wm // max(1, K))):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        graph_us = (time.perf_counter() - t0) / K * 1e6

        # ---------------- hot cache: the same KV set every step ----------------
        graph_hot = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph_hot, stream=stream):
            for i in range(K):
                problems[0].run()
        graph_hot.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph_hot.replay()
        torch.cuda.synchronize()
        hot_us = (time.perf_counter() - t0) / K * 1e6

        # ---------------- the same steps with the fragment lengths read from device memory ----------------
        len_dev = torch.tensor(case.lens, dtype=torch.int32, device=dev)
        problems_dl = []
        for keys, vals in ring:
            pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=keys, values=vals, scale=case.scale, out=out,
                              cosines=cd.cos, sines=cd.sin, rq=rq, lse=lse, splits=args.splits, len_dev=len_dev)
            pr.set_workspace(ws)
            problems_dl.append(pr)
        graph_dl = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph_dl, stream=stream):
            for i in range(K):
                problems_dl[i % nring].run()
        graph_dl.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph_dl.replay()
        torch.cuda.synchronize()
        devlen_us = (time.perf_counter() - t0) / K * 1e6

        # ---------------- per-launch duration of the attention kernel (HIP events on its stream) ----------------
        # K launches of the attention kernel alone (merge stage off), replayed as one graph so that the launches
        # follow each other without host submission gaps, bracketed by two HIP events recorded on this stream.
        # (An event pair around a single eagerly launched kernel also measures several microseconds of
        # submission latency; that figure is reported under extra for comparison.)
        graph_k = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph_k, stream=stream):
            for i in range(K):
                problems[i % nring].run(stages=1)
        graph_k.replay()
        torch.cuda.synchronize()
        ea, eb = _lib.Event(), _lib.Event()
        reps = 3
        per = []
        for _ in range(reps):
            ea.record(stream.cuda_stream)
            graph_k.replay()
            eb.record(stream.cuda_stream)
            torch.cuda.synchronize()
            per.append(ea.elapsed_ms(eb) * 1e3 / K)
        kern_us_avg = sum(per) / len(per)
        kern_us_med = sorted(per)[len(per) // 2]

        evs2 = [(_lib.Event(), _lib.Event()) for _ in range(K)]
        for i in range(K):
            pr = problems[i % nring]
            pr.set_events(evs2[i][0].handle, evs2[i][1].handle)
            pr.run()
            pr.set_events(None, None)
        torch.cuda.synchronize()
        d2 = sorted(a.elapsed_ms(b) * 1e3 for a, b in evs2)
        kern_us_eager_med = d2[len(d2) // 2]

        # ---------------- the caller-side steps of a decode step at this shape (latency-bound, tiny) ----------------
        Hkv = cd.keys[0].size(0)
        seg_k = [torch.zeros((Hkv, 256, E), dtype=tdt, device=dev) for _ in range(W)]
        seg_v = [torch.zeros((Hkv, 256, E), dtype=tdt, device=dev) for _ in range(W)]
        k_new = torch.randn((W, S, Hkv, E), device=dev).to(tdt).transpose(1, 2)
        ck = torch.ones((W, S, E), dtype=tdt, device=dev)
        inv = torch.ones(E // 2, dtype=torch.float32, device=dev)
        pos_end = [[1000 + 7 * f + w for w in range(W)] for f in range(case.F)]
        g_a = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g_a, stream=stream):
            for i in range(K):
                _lib.rope_append(k_new, k_new, seg_k, seg_v, [i % 200] * W, cosines=ck, sines=ck)
        g_b = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g_b, stream=stream):
            for i in range(K):
                _lib.build_inputs(pos_end, S, inv, table_dtype=tdt if tdt != torch.float32 else None)
        # what one layer of a decode step launches: key rotation + append, then attention and merge (cold ring)
        g_c = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g_c, stream=stream):
            for i in range(K):
                _lib.rope_append(k_new, k_new, seg_k, seg_v, [i % 200] * W, cosines=ck, sines=ck)
                problems[i % nring].run()
        side = []
        for gr in (g_a, g_b, g_c):
            gr.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            gr.replay()
            torch.cuda.synchronize()
            side.append((time.perf_counter() - t0) / K * 1e6)
        append_us, build_us, layer_us = side

        # ---------------- plain streaming read of the whole ring (achievable HBM rate) ----------------
        big = torch.empty(int(args.ring_mb * 1e6) // 16 * 16, dtype=torch.uint8, device=dev)
        big.random_(0, 255)
        sink = torch.zeros(256, dtype=torch.int32, device=dev)
        e0, e1 = _lib.Event(), _lib.Event()
        s_handle = stream.cuda_stream
        import ctypes as C
        for _ in range(2):
            _lib.check(_lib.lib.hw_stream_read(big.data_ptr(), big.numel(), sink.data_ptr(), C.c_void_p(s_handle)), "hw_stream_read")
        e0.record(s_handle)
        for _ in range(5):
            _lib.check(_lib.lib.hw_stream_read(big.data_ptr(), big.numel(), sink.data_ptr(), C.c_void_p(s_handle)), "hw_stream_read")
        e1.record(s_handle)
        torch.cuda.synchronize()
        stream_gbs = big.numel() * 5 / (e0.elapsed_ms(e1) * 1e-3) / 1e9
        # a plain copy of known size (256 MiB read + 256 MiB written): the reference point that scales the
        # FETCH_SIZE / WRITE_SIZE hardware counters when this command runs under rocprofv3 --pmc
        half = 256 * 1024 * 1024
        for _ in range(2):
            _lib.check(_lib.lib.hw_stream_copy(big.data_ptr() + half, big.data_ptr(), half, C.c_void_p(s_handle)), "hw_stream_copy")
        torch.cuda.synchronize()
        del big

    value = kv_bytes / (graph_us * 1e-6) / 1e9
    achieved = kv_bytes / (kern_us_avg * 1e-6) / 1e9
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
            "workload": f"config {args.case} ({case.name}): W={case.W} S={case.S} Hq={case.Hq} Hkv={case.Hkv} D={case.E} "
                        f"{case.dtype}, fragments={case.lens}",
            "kv_bytes_per_step": kv_bytes,
            "visible_tokens": case.visible_tokens(),
            "cold_cache_ring_sets": nring,
            "workgroups": plan.workgroups,
            "wgs_per_head": plan.wgs_per_head,
            "writes_rotated_q": rq is not None,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": PEAK_HBM_GBS,
            "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM_GBS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(case.name),
            "kernel": "hw::attention_kernel",
            "kernel_us_avg": round(kern_us_avg, 3),
            "kernel_us_median": round(kern_us_med, 3),
            "timing": "two HIP events around a graph replay of K attention-kernel launches (merge stage off), divided by K",
        },
        "extra": {
            "us_per_step": round(graph_us, 3),
            "pct_of_peak": round(100.0 * value / PEAK_HBM_GBS, 2),
            "eager_loop_us_per_step": round(eager_us, 3),
            "kernel_us_median_eager_event_pair": round(kern_us_eager_med, 3),
            "hot_cache_us_per_step": round(hot_us, 3),
            "device_lengths_us_per_step": round(devlen_us, 3),
            "hot_cache_GBps": round(kv_bytes / (hot_us * 1e-6) / 1e9, 1),
            "stream_read_GBps": round(stream_gbs, 1),
            "rope_append_us_per_call": round(append_us, 3),
            "build_inputs_us_per_call": round(build_us, 3),
            "append_plus_attention_us_per_layer": round(layer_us, 3),
            "timing": "K steps replayed as one HIP graph, wall clock between device synchronisations",
        },
    }

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(case, kv_bytes)
    print(json.dumps(result, ensure_ascii=False))


def bench_paged(args, dev):
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
        q_lens = [1, 8, 32, 64]
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
                               scale=scale, out=out, lse=lse, splits=args.splits, cu_seqlens_q=cu)
        if ws is None:
            ws = torch.empty(pr.workspace_bytes(), dtype=torch.uint8, device=dev)
        pr.set_workspace(ws)
        problems.append(pr)
    plan = _lib.paged_plan(W=W, Hq=Hq, Hkv=Hkv, Ev=D, block_size=bs, max_blocks=nblk, num_cus=_lib.lib.hw_device_cus(), S=S,
                           splits=args.splits, total_q=(q.size(1) if varlen else None))
    K, Wm = args.steps, args.warmup
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

        def graph_of(fn):
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr, stream=stream):
                for i in range(K):
                    fn(i)
            gr.replay()
            torch.cuda.synchronize()
            return gr

        g_step = graph_of(lambda i: problems[i % nring].run())
        t0 = time.perf_counter()
        g_step.replay()
        torch.cuda.synchronize()
        graph_us = (time.perf_counter() - t0) / K * 1e6
        g_hot = graph_of(lambda i: problems[0].run())
        t0 = time.perf_counter()
        g_hot.replay()
        torch.cuda.synchronize()
        hot_us = (time.perf_counter() - t0) / K * 1e6
        g_k = graph_of(lambda i: problems[i % nring].run(stages=1))
        ea, eb = _lib.Event(), _lib.Event()
        per = []
        for _ in range(3):
            ea.record(stream.cuda_stream)
            g_k.replay()
            eb.record(stream.cuda_stream)
            torch.cuda.synchronize()
            per.append(ea.elapsed_ms(eb) * 1e3 / K)
        kern_us = sum(per) / len(per)

        # the append that precedes every decode step: one new token per sequence into the paged cache
        ks = torch.randn((W, 1, Hkv, D), device=dev).to(torch.bfloat16).transpose(1, 2)
        seq = torch.full((W,), L - 1, dtype=torch.int32, device=dev)
        g_c = graph_of(lambda i: _lib.copy_to_blocks(ks, ks, kc, vc, tables[i % nring], seq))
        t0 = time.perf_counter()
        g_c.replay()
        torch.cuda.synchronize()
        copy_us = (time.perf_counter() - t0) / K * 1e6

    value = kv_bytes / (graph_us * 1e-6) / 1e9
    achieved = kv_bytes / (kern_us * 1e-6) / 1e9
    result = {
        "metric": "KV-read HBM GB/s (% of peak) + µs/decode step, QwQ-32B shape, 4 sequences, paged KV cache"
                  + (", packed variable-length queries" if varlen else ""),
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": Wm,
        "ms_per_step": round(graph_us * 1e-3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": (f"varlen paged: W={W} sequences x {L} tokens, query tokens per sequence 1/8/32/64, " if varlen else
                                f"paged decode: W={W} sequences x {L} tokens, S={S}, ") + f"Hq={Hq} Hkv={Hkv} D={D} bf16, block_size={bs}, F={F}", "kv_bytes_per_step": kv_bytes, "cold_cache_ring_sets": nring,
                   "workgroups": plan.workgroups, "splits": plan.splits},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4), "traffic": (MEASURED_VARLEN_TRAFFIC_BYTES if varlen else MEASURED_PAGED_TRAFFIC_BYTES).get((L, bs)),
                     "kernel": "hw::paged_attention_kernel",
                     "kernel_us_avg": round(kern_us, 3),
                     "timing": "two HIP events around a graph replay of K attention-kernel launches (merge stage off), divided by K"},
        "extra": {"us_per_step": round(graph_us, 3), "pct_of_peak": round(100.0 * value / PEAK_HBM_GBS, 2),
                  "eager_loop_us_per_step": round(eager_us, 3), "hot_cache_us_per_step": round(hot_us, 3),
                  "copy_to_blocks_us": round(copy_us, 3)},
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
    print(json.dumps(result, ensure_ascii=False))


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


def cpu_baseline(case, kv_bytes):
    """The reference's eager PyTorch path (python/hogwild/attention.py:38-67 + :84-90) restated in
    oracle/, timed on the host cores of this box.  Baseline only."""
    import torch
    from oracle import hogwild_oracle as O
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    args = (case.q, case.locations, case.keys, case.values, case.scale, case.cos, case.sin)
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
    return {
        "value": round(kv_bytes / med / 1e9, 3),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "us_per_step": round(med * 1e6, 1),
        "sample": f"{len(ts)} full steps of the same workload (median), torch fp32 eager restatement of the reference path",
    }


if __name__ == "__main__":
    main()
