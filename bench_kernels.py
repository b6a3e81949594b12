#!/usr/bin/env python3
"""Per-kernel throughput of every entry point of libconef_hip.so on the shapes of the benchmark
configurations, against the MI355X HBM peak.  `bench.py` measures the headline step; this script
measures the rest of the hot path the same way: resident inputs, rotating buffers (working set
above the 256 MB Infinity Cache where the shape allows), HIP events on the launch stream.

    python bench_kernels.py [--filter substring] [--iters N]

Prints one line per case: microseconds per call, algorithmic bytes, GB/s, fraction of 8 TB/s.
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
    ap.add_argument("--iters", type=int, default=200)
    ap.add_argument("--json", action="store_true")
    args = ap.parse_args()

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
                     ("cfg4 LSTM embedding", 33278, 650, 0.1), ("cfg1 ResNet-20 conv", 64, 576, 0.5)]

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
            timeit("cs_update_planned_f32 (%s) %s [%d,%d] W=%d" % ("row lists" if plan.in_place else "binned", tag, n, d, w),
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

    for rows, r in [(5760, 4), (640, 4), (4096, 8), (1024, 8), (30522, 8), (4096, 32), (576, 2)]:
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
        timeit("topk_sparsify_f32 %d elements, keep 20%%" % numel, 7 * 4 * numel,
               lambda numel=numel, ws_bytes=ws_bytes, nset=nset: [(torch.randn(numel, device=dev),
                                                                   torch.empty(ws_bytes, dtype=torch.uint8, device=dev))
                                                                  for _ in range(nset)],
               lambda s, numel=numel, kk=kk: ck(lib.conef_topk_sparsify_f32(s[0].data_ptr(), numel, kk, s[1].data_ptr(),
                                                                            s[1].numel(), stream), "topk"))
    if not args.json:
        print("done: %d cases" % len(results))


if __name__ == "__main__":
    main()
