#!/usr/bin/env python3
"""Per-kernel throughput of every entry point of libconef_hip.so on the shapes of the benchmark
configurations, against the MI355X HBM peak.  `bench.py` measures the headline step; this script
measures the rest of the hot path the same way: resident inputs, rotating buffers (working set
above the 256 MB Infinity Cache where the shape allows), HIP events on the launch stream.

    python bench_kernels.py [--filter substring] [--iters N]

Prints one line per case: microseconds per call, algorithmic bytes, GB/s, fraction of 8 TB/s.

    python -m conef_amd.build --trace && python bench_kernels.py --phase-trace

prints instead when the workgroups of the two passes of the fused RandomBlock + sketch step reach
their phase boundaries (a build of the same sources that also stores timestamps).
"""
import argparse
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8000.0
A, B = 994443, 609478


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--filter", default="")
    ap.add_argument("--hook-streams", type=int, default=2, help="side streams of the 'N streams' hook-step lines")
    ap.add_argument("--iters", type=int, default=200)
    ap.add_argument("--json", action="store_true")
    ap.add_argument("--phase-trace", action="store_true",
                    help="phase timeline of the binned passes on the flat 25 MB bucket (needs the --trace build)")
    args = ap.parse_args()
    if args.phase_trace:
        return phase_trace()

    import torch
    from conef_amd import _lib
    from conef_amd._plan import SketchPlan

    if not torch.cuda.is_available():
        print("bench_kernels.py needs the GPU", file=sys.stderr)
        sys.exit(2)
    lib = _lib.load()
    dev = torch.device("cuda", 0)
    stream = torch.cuda.current_stream().cuda_stream
    results = []

    def copies(nbytes_per_set, lo=2, hi=64, target=320e6):
        return int(max(lo, min(hi, target // max(nbytes_per_set, 1) + 1)))

    def timeit(name, alg_bytes, make, call, flops=None):
        """make(i) -> state for buffer set i; call(state) enqueues one kernel call."""
        if args.filter and args.filter not in name:
            return
        sets = make()
        n = len(sets)
        for i in range(min(10, args.iters)):
            call(sets[i % n])
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(args.iters):
            call(sets[i % n])
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / args.iters * 1e3
        gbs = alg_bytes / us / 1e3
        rec = {"case": name, "us": round(us, 2), "alg_MB": round(alg_bytes / 1e6, 3), "GBs": round(gbs, 1),
               "frac_hbm": round(gbs / HBM_PEAK, 4), "buffer_sets": n}
        if flops:
            rec["TFLOPs"] = round(flops / us / 1e6, 2)
        results.append(rec)
        if args.json:
            print(json.dumps(rec), flush=True)
        else:
            print("%-58s %9.2f us  %9.3f MB  %8.1f GB/s  %.3f of peak%s" % (
                name, us, alg_bytes / 1e6, gbs, gbs / HBM_PEAK,
                "  %.2f TFLOP/s" % rec["TFLOPs"] if flops else ""), flush=True)

    def rnd(*shape):
        return torch.randn(*shape, device=dev) * 1e-3

    def ck(rc, what):
        if rc != 0:
            raise RuntimeError("%s returned %d" % (what, rc))

    sketch_shapes = [("cfg2 flat bucket", 5, 1_300_000, 0.1), ("cfg3 WRN conv", 640, 5760, 0.2),
                     ("cfg5 BERT ffn", 1024, 4096, 0.1), ("cfg5 BERT attn", 1024, 1024, 0.1),
                     ("cfg4 LSTM embedding", 33278, 650, 0.1), ("cfg1 ResNet-20 conv", 64, 576, 0.5),
                     # rows too long for whole row lists and more than 8 of them: panels / binned row groups
                     ("VGG-16 fc6", 4096, 25088, 0.1), ("64 long rows", 64, 200_000, 0.1)]

    # ------------------------------------------------------------------ count sketch
    for tag, n, d, ss in sketch_shapes:
        w = max(int(d * ss), 1)
        nset = copies(4 * n * d)

        def make(n=n, d=d, w=w, nset=nset):
            return [(rnd(n, d), rnd(n, w), torch.empty(n, w, device=dev)) for _ in range(nset)]

        timeit("cs_query_f32 %s [%d,%d] W=%d" % (tag, n, d, w), 8 * n * d + 4 * n * w, make,
               lambda s, n=n, d=d, w=w: ck(lib.conef_cs_query_f32(s[0].data_ptr(), s[1].data_ptr(), n, d, w, 0.1, A, B,
                                                                    stream), "query"))
        if SketchPlan.applicable(n, d, w):
            plan = SketchPlan(n, d, w, A, B, dev)
            staging = None if plan.in_place else plan.workspace.data_ptr()
            timeit("cs_query_planned_f32 (%s) %s [%d,%d] W=%d" % (
                       "buckets and signs from the plan's table" if plan.in_place else "table, sketch interleaved", tag, n, d, w),
                   8 * n * d + 4 * n * w + 4 * d, make,
                   lambda s, n=n, d=d, w=w, plan=plan, staging=staging: ck(lib.conef_cs_query_planned_f32(
                       s[0].data_ptr(), s[1].data_ptr(), plan.host_ptr, plan.device.data_ptr(), staging, n, d, w, 0.1, A, B,
                       stream), "query planned"))
            timeit("cs_update_planned_f32 (%s) %s [%d,%d] W=%d" % (("binned", "row lists", "row lists in panels")[plan.kind], tag, n, d, w),
                   4 * n * d + 8 * n * w, make,
                   lambda s, n=n, d=d, w=w, plan=plan: ck(lib.conef_cs_update_planned_f32(
                       s[0].data_ptr(), s[1].data_ptr(), s[1].data_ptr(), plan.host_ptr, plan.device.data_ptr(),
                       plan.workspace.data_ptr(), n, d, w, 0.9, A, B, stream), "update planned"))
        if lib.conef_cs_update_inplace_ok(n, d, w):
            timeit("cs_update_f32 (no plan, LDS atomics) %s [%d,%d] W=%d" % (tag, n, d, w), 4 * n * d + 8 * n * w, make,
                   lambda s, n=n, d=d, w=w: ck(lib.conef_cs_update_f32(s[0].data_ptr(), s[1].data_ptr(), s[1].data_ptr(),
                                                                         n, d, w, 0.9, A, B, stream), "update"))
        else:
            timeit("cs_update_f32 (no plan, global atomics) %s [%d,%d] W=%d" % (tag, n, d, w), 4 * n * d + 8 * n * w, make,
                   lambda s, n=n, d=d, w=w: ck(lib.conef_cs_update_f32(s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(),
                                                                         n, d, w, 0.9, A, B, stream), "update atomics"))

    n, d, w = 640, 5760, 1152
    nset = copies(4 * n * d)
    timeit("cs_query_f16 cfg3 [640,5760] W=1152", 8 * n * d + 2 * n * w,
           lambda: [(rnd(n, d), rnd(n, w).half()) for _ in range(nset)],
           lambda s: ck(lib.conef_cs_query_f16(s[0].data_ptr(), s[1].data_ptr(), n, d, w, 0.1, A, B, stream), "q16"))
    timeit("cs_update_f16 cfg3 [640,5760] W=1152", 4 * n * d + 4 * n * w,
           lambda: [(rnd(n, d), rnd(n, w).half()) for _ in range(nset)],
           lambda s: ck(lib.conef_cs_update_f16(s[0].data_ptr(), s[1].data_ptr(), s[1].data_ptr(), n, d, w, 0.9, A, B,
                                                stream), "u16"))
    plan16 = SketchPlan(n, d, w, A, B, dev)
    timeit("cs_update_planned_f16 (row lists) cfg3 [640,5760] W=1152", 4 * n * d + 4 * n * w,
           lambda: [(rnd(n, d), rnd(n, w).half()) for _ in range(nset)],
           lambda s: ck(lib.conef_cs_update_planned_f16(s[0].data_ptr(), s[1].data_ptr(), s[1].data_ptr(),
                                                        plan16.host_ptr, plan16.device.data_ptr(), n, d, w, 0.9, A, B,
                                                        stream), "u16 planned"))
    timeit("cs3_query_f32 cfg3 [640,5760] W=1152", 8 * n * d + 12 * n * w,
           lambda: [(rnd(n, d), rnd(n, w), rnd(n, w), rnd(n, w)) for _ in range(nset)],
           lambda s: ck(lib.conef_cs3_query_f32(s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), s[3].data_ptr(), n,
                                                d, w, 0.1, stream), "q3"))
    timeit("cs3_update_f32 cfg3 [640,5760] W=1152", 4 * n * d + 24 * n * w,
           lambda: [(rnd(n, d), rnd(n, w), rnd(n, w), rnd(n, w), rnd(n, w), rnd(n, w), rnd(n, w)) for _ in range(nset)],
           lambda s: ck(lib.conef_cs3_update_f32(s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), s[3].data_ptr(),
                                                 s[4].data_ptr(), s[5].data_ptr(), s[6].data_ptr(), n, d, w, 0.9,
                                                 stream), "u3"))

    from conef_amd.compressors.CountSketchHash3 import DenseCSHash3
    sk3 = [DenseCSHash3(n, d, 0.2) for _ in range(4)]
    timeit("DenseCSHash3.update on plans (value pass + 3 row-list updates) cfg3 [640,5760] W=1152",
           4 * n * d + 24 * n * w, lambda: [(rnd(n, d), sk3[i % 4]) for i in range(nset)],
           lambda s: s[1].update(s[0], 0.9))

    # ------------------------------------------------------------------ random block
    L = 6_500_000
    k = 650_000
    nset = copies(8 * L)
    timeit("randblock_ef_step_f32 flat 6.5M, block 10%", 16 * L + 4 * k,
           lambda: [(rnd(L), rnd(L), torch.empty(k, device=dev)) for _ in range(nset)],
           lambda s: ck(lib.conef_randblock_ef_step_f32(s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), L, 6413414, k,
                                                        stream), "ef step"))
    n, m = 33278, 650
    L4 = n * m
    k4 = int(0.05 * L4)
    nset = copies(4 * L4)
    timeit("randblock_unbiased_step_f32 cfg4 [33278,650], block 5%", 4 * L4 + 8 * k4,
           lambda: [(rnd(L4), torch.empty(k4, device=dev)) for _ in range(nset)],
           lambda s: ck(lib.conef_randblock_unbiased_step_f32(s[0].data_ptr(), s[1].data_ptr(), L4, 1234567, k4,
                                                              k4 / L4, stream), "unbiased"))
    w4 = 65
    plan4 = SketchPlan(n, m, w4, A, B, dev)
    timeit("randblock_conef_step_planned_f32 (row lists) cfg4 [33278,650] W=65", 8 * L4 + 8 * n * w4 + 4 * k4,
           lambda: [(rnd(n, m), rnd(n, w4), torch.empty(k4, device=dev)) for _ in range(nset)],
           lambda s: ck(lib.conef_randblock_conef_step_planned_f32(
               s[0].data_ptr(), s[1].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), plan4.host_ptr,
               plan4.device.data_ptr(), plan4.workspace.data_ptr(), n, m, w4, 1234567, k4, 0.1, 0.9, A, B, stream),
               "rb conef planned"))
    timeit("randblock_conef_step_f32 (no plan) cfg4 [33278,650] W=65", 8 * L4 + 8 * n * w4 + 4 * k4,
           lambda: [(rnd(n, m), rnd(n, w4), torch.empty(k4, device=dev)) for _ in range(nset)],
           lambda s: ck(lib.conef_randblock_conef_step_f32(s[0].data_ptr(), s[1].data_ptr(), s[1].data_ptr(),
                                                           s[2].data_ptr(), n, m, w4, 1234567, k4, 0.1, 0.9, A, B,
                                                           stream), "rb conef row"))

    # ------------------------------------------------------------------ PowerSGD passes
    for tag, n, m, r, ss in [("cfg3 WRN conv", 640, 5760, 4, 0.2), ("cfg5 BERT ffn", 1024, 4096, 8, 0.1),
                             ("cfg5 BERT ffn", 1024, 4096, 32, 0.1), ("cfg5 BERT vocab", 30522, 1024, 8, 0.1),
                             ("cfg1 ResNet-20 conv", 64, 576, 2, 0.5)]:
        w = max(int(m * ss), 1)
        nset = copies(4 * n * m)

        def make(n=n, m=m, r=r, w=w, nset=nset):
            return [(rnd(n, m), torch.randn(m, r, device=dev), torch.randn(n, r, device=dev), rnd(n, m), rnd(n, w))
                    for _ in range(nset)]

        fl = 2.0 * n * m * r
        shape = "%s [%d,%d] r=%d" % (tag, n, m, r)
        ws = torch.empty(lib.conef_psgd_workspace_bytes(n, m, r), dtype=torch.uint8, device=dev)
        plan = SketchPlan(n, m, w, A, B, dev)
        timeit("psgd_mq_f32 " + shape, 4 * n * m + 4 * (n + m) * r, make,
               lambda s, n=n, m=m, r=r, ws=ws: ck(lib.conef_psgd_mq_f32(s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(),
                                                                        n, m, r, ws.data_ptr(), ws.numel(), stream),
                                                  "mq"), flops=fl)
        timeit("psgd_mq_ef_f32 " + shape, 12 * n * m + 4 * (n + m) * r, make,
               lambda s, n=n, m=m, r=r, ws=ws: ck(lib.conef_psgd_mq_ef_f32(s[0].data_ptr(), s[3].data_ptr(), s[1].data_ptr(),
                                                                           s[2].data_ptr(), n, m, r, ws.data_ptr(),
                                                                           ws.numel(), stream), "mq ef"), flops=fl)
        timeit("psgd_mq_conef_f32 %s W=%d" % (shape, w), 8 * n * m + 4 * n * w + 4 * (n + m) * r, make,
               lambda s, n=n, m=m, r=r, w=w, ws=ws: ck(lib.conef_psgd_mq_conef_f32(
                   s[0].data_ptr(), s[4].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), n, m, r, w, 0.1, A, B,
                   ws.data_ptr(), ws.numel(), stream), "mq conef"), flops=fl)
        timeit("psgd_mq_conef_planned_f32 %s W=%d" % (shape, w), 8 * n * m + 4 * n * w + 4 * (n + m) * r, make,
               lambda s, n=n, m=m, r=r, w=w, plan=plan, ws=ws: ck(lib.conef_psgd_mq_conef_planned_f32(
                   s[0].data_ptr(), s[4].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), plan.host_ptr,
                   plan.device.data_ptr(), n, m, r, w, 0.1, A, B, ws.data_ptr(), ws.numel(), stream),
                   "mq conef planned"), flops=fl)
        timeit("psgd_mtp_f32 " + shape, 4 * n * m + 4 * (n + m) * r, make,
               lambda s, n=n, m=m, r=r, ws=ws: ck(lib.conef_psgd_mtp_f32(s[0].data_ptr(), s[2].data_ptr(), s[1].data_ptr(),
                                                                         n, m, r, ws.data_ptr(), ws.numel(), stream),
                                                  "mtp"), flops=fl)
        timeit("psgd_pqt_f32 " + shape, 4 * n * m + 4 * (n + m) * r, make,
               lambda s, n=n, m=m, r=r: ck(lib.conef_psgd_pqt_f32(s[0].data_ptr(), s[2].data_ptr(), s[1].data_ptr(), n, m,
                                                                  r, stream), "pqt"), flops=fl)
        timeit("psgd_pqt_ef_f32 " + shape, 12 * n * m + 4 * (n + m) * r, make,
               lambda s, n=n, m=m, r=r: ck(lib.conef_psgd_pqt_ef_f32(s[0].data_ptr(), s[3].data_ptr(), s[2].data_ptr(),
                                                                     s[1].data_ptr(), n, m, r, stream), "pqt ef"), flops=fl)
        timeit("psgd_pqt_conef_planned_f32 %s W=%d" % (shape, w), 8 * n * m + 8 * n * w + 4 * (n + m) * r, make,
               lambda s, n=n, m=m, r=r, w=w, plan=plan: ck(lib.conef_psgd_pqt_conef_planned_f32(
                   s[0].data_ptr(), s[2].data_ptr(), s[1].data_ptr(), s[4].data_ptr(), s[4].data_ptr(), plan.host_ptr,
                   plan.device.data_ptr(), n, m, r, w, 0.9, A, B, stream), "pqt conef planned"), flops=fl)
        timeit("psgd_pqt_conef_f32 (no plan) %s W=%d" % (shape, w), 8 * n * m + 8 * n * w + 4 * (n + m) * r, make,
               lambda s, n=n, m=m, r=r, w=w: ck(lib.conef_psgd_pqt_conef_f32(s[0].data_ptr(), s[2].data_ptr(),
                                                                             s[1].data_ptr(), s[4].data_ptr(),
                                                                             s[4].data_ptr(), n, m, r, w, 0.9, A, B,
                                                                             stream), "pqt conef"), flops=fl)

    for rows, r in [(5760, 4), (640, 4), (4096, 8), (1024, 8), (30522, 8), (4096, 32), (576, 2), (1024, 32), (512, 32),
                    (30522, 32), (1024, 16), (4096, 16), (2048, 32), (2048, 16), (256, 32), (64, 32)]:
        ws = torch.empty(lib.conef_psgd_workspace_bytes(rows, 1, r), dtype=torch.uint8, device=dev)
        timeit("gram_schmidt_f32 [%d,%d]" % (rows, r), 8 * rows * r,
               lambda rows=rows, r=r: [(torch.randn(rows, r, device=dev),) for _ in range(8)],
               lambda s, rows=rows, r=r, ws=ws: ck(lib.conef_gram_schmidt_f32(s[0].data_ptr(), rows, r, 0.0, ws.data_ptr(),
                                                                              ws.numel(), stream), "gs"))

    # ------------------------------------------------------------------ top-k
    for numel in (1_048_576, 31_254_528):
        kk = max(1, int(0.2 * numel))
        ws_bytes = lib.conef_topk_workspace_bytes(numel)
        nset = copies(4 * numel, hi=16)
        timeit("topk_sparsify_f32 %d elements, keep 20%%" % numel, 8 * numel,
               lambda numel=numel, ws_bytes=ws_bytes, nset=nset: [(torch.randn(numel, device=dev),
                                                                   torch.empty(ws_bytes, dtype=torch.uint8, device=dev))
                                                                  for _ in range(nset)],
               lambda s, numel=numel, kk=kk: ck(lib.conef_topk_sparsify_f32(s[0].data_ptr(), numel, kk, s[1].data_ptr(),
                                                                            s[1].numel(), stream), "topk"))
    # ------------------------------------------------------------------ whole hook steps
    # One training step's worth of buckets through the Python hooks, per benchmark configuration:
    # host work included (one ctypes call per kernel launch), so small-matrix models show what the
    # launch path costs next to what the kernels cost.
    if not args.filter or "hook" in args.filter:
        hook_steps(args, results)
    if not args.json:
        print("done: %d cases" % len(results))
    teardown()


def phase_trace():
    """Workgroup phase timeline of the staging and accumulate passes, [5, 1300000] bucket, block 650000."""
    import ctypes

    import numpy as np
    import torch
    from conef_amd import _lib
    from conef_amd.build import TRACE_LIBPATH

    if not os.path.exists(TRACE_LIBPATH):
        print("no %s: run `python -m conef_amd.build --trace` first" % TRACE_LIBPATH, file=sys.stderr)
        sys.exit(2)
    _lib.LIBPATH = TRACE_LIBPATH              # before the first load: every entry point comes from the tracing build
    lib = _lib.load()
    lib.conef_trace_read.argtypes = [ctypes.c_void_p]
    lib.conef_trace_read.restype = ctypes.c_int
    from conef_amd.compressors.CountSketch import DenseCS

    n, m, block = 5, 1_300_000, 650_000
    grads = [torch.randn(n, m, device="cuda") * 1e-3 for _ in range(24)]
    sketches = [DenseCS(n, m, 0.1) for _ in range(12)]
    payload = torch.empty(block, device="cuda")
    rng = np.random.RandomState(42)
    buf = np.zeros((2, 1024, 8), dtype=np.uint64)
    rows = {0: [], 1: []}
    for it in range(40):
        sketches[it % 12].randblock_step(grads[it % 24], payload, int(rng.randint(0, n * m)), block, 0.1, 0.9)
        torch.cuda.synchronize()
        if it < 8:
            continue
        _lib.check(lib.conef_trace_read(buf.ctypes.data_as(ctypes.c_void_p)), "conef_trace_read")
        for p in (0, 1):
            t = buf[p].astype(np.int64)
            t = t[t[:, 0] > 0]                   # workgroups of this launch
            rows[p].append((t - t[:, 0].min()) * 0.01)
    names = {0: ["workgroup starts", "its loads are in LDS", "after the barrier", "stores issued"],
             1: ["bin threads start", "first records arrived", "bin image complete", "after the barrier",
                 "lists walked, cells written", "column waves start", "selected block finished", "zeros written"]}
    for p in (0, 1):
        a = np.concatenate(rows[p])              # [launches * workgroups, 8]
        print("pass %s, microseconds after its first workgroup started (%d workgroups per launch)"
              % ("AB"[p], len(rows[p][0])))
        for k, name in enumerate(names[p]):
            v = a[:, k]
            v = v[v >= 0]
            print("  %-30s median %6.2f   p90 %6.2f   max %6.2f" % (name, np.median(v), np.percentile(v, 90), v.max()))
    teardown()


def teardown():
    """Returns every piece of device memory and every stream this process created while the HIP
    runtime is still whole: waits for the device, drops the library's shared pools, then gives
    torch's cached blocks back to the runtime.  Under a profiler that finalises itself in an exit
    handler, whatever is still allocated when the interpreter has gone is freed after the tool."""
    import gc

    import torch
    import conef_amd
    torch.cuda.synchronize()
    conef_amd.release()
    gc.collect()
    torch.cuda.empty_cache()
    torch.cuda.synchronize()


def hook_steps(args, results):
    import time

    import numpy as np
    import torch

    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from _helpers import FakeGradBucket
    from conef_amd.powerSGD_hook import PowerSGDState, powerSGD_hook
    from conef_amd.hPowerSGD_hook import hPowerSGDState, hpowerSGD_hook
    from conef_amd.RandomBlock_hook import RandomBlock_hook, RandomBlockState
    from conef_amd.UnbiasedRandomBlock_hook import UnbiasedRandomBlock_hook, UnbiasedRandomBlockState

    cap = 25 * 1024 * 1024 // 4

    def numel(s):
        return int(np.prod(s))

    def buckets_of(shapes):
        out, cur, size = [], [], 0
        for s in reversed(shapes):
            if cur and size + numel(s) > cap:
                out.append(cur)
                cur, size = [], 0
            cur.append(s)
            size += numel(s)
        if cur:
            out.append(cur)
        return out

    resnet20 = ([(16, 3, 3, 3), (16,), (16,)] + [(16, 16, 3, 3), (16,), (16,)] * 6 + [(32, 16, 3, 3), (32,), (32,)] +
                [(32, 32, 3, 3), (32,), (32,)] * 5 + [(64, 32, 3, 3), (64,), (64,)] + [(64, 64, 3, 3), (64,), (64,)] * 5 +
                [(10, 64), (10,)])
    wrn = [(16, 3, 3, 3)]
    widths = [16, 160, 320, 640]
    for stage in range(3):
        cin, cout = widths[stage], widths[stage + 1]
        for block in range(4):
            a = cin if block == 0 else cout
            wrn += [(a,), (a,), (cout, a, 3, 3), (cout,), (cout,), (cout, cout, 3, 3)]
            if block == 0:
                wrn.append((cout, a, 1, 1))
    wrn += [(640,), (640,), (10, 640), (10,)]
    v, h = 33278, 650
    lstm = [(v, h), (4 * h, h), (4 * h, h), (4 * h,), (4 * h,), (4 * h, h), (4 * h, h), (4 * h,), (4 * h,), (v, h), (v,)]
    hh, ff, vv = 1024, 4096, 30522
    bert = [(vv, hh), (512, hh), (2, hh), (hh,), (hh,)]
    for _ in range(24):
        bert += [(hh, hh), (hh,)] * 4 + [(hh,), (hh,), (ff, hh), (ff,), (hh, ff), (hh,), (hh,), (hh,)]
    bert += [(hh, hh), (hh,), (hh, hh), (hh,), (hh,), (hh,), (vv,), (2, hh), (2,)]

    ns = max(1, args.hook_streams)

    def psgd(rank, ss, streams=None):      # None: the state's own choice (two streams above rank 8)
        return lambda: (PowerSGDState(None, matrix_approximation_rank=rank, start_powerSGD_iter=2,
                                      use_error_compression=True, sketch_size=ss, beta=0.9, hook_streams=streams),
                        powerSGD_hook)

    cases = [
        ("hook cfg1 ResNet-20, PowerSGD r=2 + sketch 50%", resnet20, psgd(2, 0.5)),
        ("hook cfg2 flat 25 MB bucket, RandomBlock 10% + sketch 10%", [(5, 1_300_000)],
         lambda: (RandomBlockState(None, compression_ratio=0.1, start_compression_iter=2, use_error_compression=True,
                                   sketch_size=0.1, beta=0.9), RandomBlock_hook)),
        ("hook cfg3 WRN-28-10, PowerSGD r=4 + sketch 20%", wrn, psgd(4, 0.2)),
        ("hook cfg4 LSTM, UnbiasedRandomBlock 5%", lstm,
         lambda: (UnbiasedRandomBlockState(None, compression_ratio=0.05, start_compression_iter=2),
                  UnbiasedRandomBlock_hook)),
        ("hook cfg4 LSTM, RandomBlock 5% + sketch 10%", lstm,
         lambda: (RandomBlockState(None, compression_ratio=0.05, start_compression_iter=2, use_error_compression=True,
                                   sketch_size=0.1, beta=0.9), RandomBlock_hook)),
        ("hook cfg5 BERT-large, PowerSGD r=8 + sketch 10%", bert, psgd(8, 0.1)),
        ("hook cfg5 BERT-large, PowerSGD r=32 + sketch 10%", bert, psgd(32, 0.1)),
        ("hook cfg5 BERT-large, hPowerSGD r=8 + top-k error", bert,
         lambda: (hPowerSGDState(None, matrix_approximation_rank=8, start_powerSGD_iter=2, use_error_compression=True,
                                 topk_ratio=0.4), hpowerSGD_hook)),
        # the same steps with the buckets spread over side streams (hook_streams, not in the reference)
        ("hook cfg3 WRN-28-10, PowerSGD r=4 + sketch 20%%, %d streams" % ns, wrn, psgd(4, 0.2, ns)),
        ("hook cfg5 BERT-large, PowerSGD r=8 + sketch 10%%, %d streams" % ns, bert, psgd(8, 0.1, ns)),
        ("hook cfg5 BERT-large, PowerSGD r=32 + sketch 10%%, %d streams" % ns, bert, psgd(32, 0.1, ns)),
        ("hook cfg5 BERT-large, hPowerSGD r=8 + top-k error, %d streams" % ns, bert,
         lambda: (hPowerSGDState(None, matrix_approximation_rank=8, start_powerSGD_iter=2, use_error_compression=True,
                                 topk_ratio=0.4, hook_streams=ns), hpowerSGD_hook)),
    ]
    dev = torch.device("cuda", 0)
    for name, shapes, make in cases:
        if args.filter and args.filter not in name and args.filter != "hook":
            continue
        state, hook = make()
        state.iter = 2
        buckets = buckets_of(shapes)
        total = sum(numel(s) for s in shapes)
        grads = [torch.randn(sum(numel(s) for s in b), device=dev) * 1e-3 for b in buckets]

        # bucket objects with their per-parameter views made once, as the reducer's are
        fakes = [FakeGradBucket(g, b, index=i, is_last=i == len(buckets) - 1) for i, (b, g) in enumerate(zip(buckets, grads))]
        for f in fakes:
            f.gradients()

        def step():
            # as the reducer does: every bucket's hook as its gradients are ready, the waits at the end
            futs = [hook(state, f) for f in fakes]
            for f in futs:
                f.wait()

        for _ in range(3):
            step()
        torch.cuda.synchronize()
        # enough repetitions for about 40 ms of timed work (small models: a step is tens of microseconds)
        t_probe = time.perf_counter()
        step()
        torch.cuda.synchronize()
        reps = max(5, min(400, int(0.04 / max(time.perf_counter() - t_probe, 1e-5))))
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(reps):
            step()
        e1.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) / reps * 1e3
        gpu = e0.elapsed_time(e1) / reps
        # what the host spends on issuing one step, with nothing queued in front of it
        issued = 1e9
        for _ in range(3):
            t1 = time.perf_counter()
            step()
            issued = min(issued, (time.perf_counter() - t1) * 1e3)
            torch.cuda.synchronize()
        rec = {"case": name, "ms_per_step_wall": round(wall, 3), "ms_per_step_gpu_events": round(gpu, 3),
               "ms_per_step_host_issue": round(issued, 3),
               "gradient_MB": round(4 * total / 1e6, 1), "buckets": len(buckets),
               "gradient_GBs": round(4 * total / 1e6 / max(wall, gpu), 1)}
        results.append(rec)
        if args.json:
            print(json.dumps(rec), flush=True)
        else:
            print("%-58s %8.3f ms/step wall  %8.3f ms gpu  %8.3f ms host  %8.1f MB gradient in %2d buckets  %7.1f GB/s of gradient" % (
                name, wall, gpu, issued, rec["gradient_MB"], len(buckets), rec["gradient_GBs"]), flush=True)
        del state, hook, fakes, grads, step        # the case's device state goes before the next case (and before exit)


if __name__ == "__main__":
    main()
