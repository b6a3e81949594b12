#!/usr/bin/env python3
"""Throughput of the fused ConEF compress + error-feedback step on one MI355X.

Workload (the configuration the headline metric is quoted on): RandomBlock compressor, 10 %
contiguous block, with a count-sketch error compressor at 10 % memory, on one flat fp32 bucket of
6.5 M elements viewed [5, 1_300_000] (sketch [5, 130_000]); gradients N(0, 1e-6) with 1 % heavy-tail
entries Laplace(0, 1e-2); synthetic, seeded.

A "step" is one call of the fused C-ABI entry point `conef_randblock_conef_step_planned_f32` on one
bucket whose gradient already sits in HBM: it adds the unsketched error, extracts the payload
block, leaves the decompressed gradient in place and writes the new sketch.  Every timed step gets a gradient buffer
no earlier step has touched and one of a rotating set of sketch states, so nothing it reads is left
in the 256 MB Infinity Cache from before: the rate is an HBM rate, not a cache rate.  The
same-buffer rate is reported next to it.

Prints ONE JSON line.  `roofline` prices the step against MI355X's 8 TB/s HBM peak with the
algorithmic byte count 8L + 8nW + 4k; `cpu_baseline` times the scalar C oracle on a bounded sample
of the same workload on this box's host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes one step moves come from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this script,
# calibrated on its own 512 MiB copy.  `--write-traffic DIR` condenses the two counter CSVs of
# such runs into this file, stamped with the kernel names, the plan tiling and a hash of the
# kernel sources; a normal run reports the figure only while those still match, else null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "randblock_conef_step_25MB_bucket.traffic.txt")
KERNEL_SOURCES = ("conef_plan.h", "conef_plan.hip", "conef_device.h", "conef_sketch_core.h", "conef_rowlist.h")
STEP_KERNELS = ("conef_binned_stage_kernel", "conef_binned_accumulate_kernel")

N_ROWS, N_COLS = 5, 1_300_000
SKETCH_SIZE = 0.1
RATIO = 0.1
BETA = 0.9
N_BUCKETS = 12           # sketch states / payload buffers in rotation (a fresh 26 MB gradient every step)
MAX_GRAD_BUFFERS = 2000  # 52 GB of gradients at most; beyond that the buffers are stepped on again


def algorithmic_bytes(L, n, w, k):
    """read g (4L) + read sketch (4nW) + write decompressed g (4L) + write sketch (4nW) + write payload (4k)"""
    return 8 * L + 8 * n * w + 4 * k


def kernel_sources_hash():
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "conef_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def read_traffic(chunk_cols, bin_buckets):
    """(bytes per step, note): the recorded HBM traffic if it was measured on these kernel sources
    and this plan tiling, else (None, why)."""
    if not os.path.exists(TRAFFIC_FILE):
        return None, "no traffic record"
    rec = {}
    with open(TRAFFIC_FILE) as f:
        for line in f:
            if "=" in line and not line.lstrip().startswith("#"):
                k, v = line.split("=", 1)
                rec[k.strip()] = v.strip()
    if rec.get("kernel_sources_sha256_16") != kernel_sources_hash():
        return None, "kernel sources changed since the traffic was measured"
    if (int(rec.get("chunk_cols", -1)), int(rec.get("bin_buckets", -1))) != (chunk_cols, bin_buckets):
        return None, "plan tiling differs from the measured one"
    return int(rec["bytes_per_step"]), "rocprofv3 FETCH_SIZE/WRITE_SIZE, see " + os.path.relpath(TRAFFIC_FILE, ROOT)


def write_traffic(pmc_dir, chunk_cols, bin_buckets):
    """Condenses DIR/pmc_FETCH_SIZE_counter_collection.csv and DIR/pmc_WRITE_SIZE_counter_collection.csv
    (rocprofv3 --pmc runs of this script, one counter each) into TRAFFIC_FILE."""
    import csv
    copy_kib = 512 * 1024          # the 512 MiB copy this script performs: reads and writes that much
    per = {}
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        vals = {}
        with open(os.path.join(pmc_dir, "pmc_%s_counter_collection.csv" % counter), newline="") as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] != counter:
                    continue
                name = row["Kernel_Name"]
                key = next((k for k in STEP_KERNELS if k in name), None)
                if key is None and "copyBuffer" in name and int(row["Grid_Size"]) >= 131072:
                    key = "copy"
                if key:
                    vals.setdefault(key, []).append(float(row["Counter_Value"]))
        if "copy" not in vals or any(k not in vals for k in STEP_KERNELS):
            raise SystemExit("%s: kernels or calibration copy missing in %s" % (counter, pmc_dir))
        per[counter] = {k: sum(v) / len(v) for k, v in vals.items()}
        per[counter]["n"] = {k: len(v) for k, v in vals.items()}
    ff = copy_kib / per["FETCH_SIZE"]["copy"]
    wf = copy_kib / per["WRITE_SIZE"]["copy"]
    total = 0.0
    lines = ["# HBM traffic of one fused RandomBlock + count-sketch step on the [5,1300000] bucket.",
             "# Made by: python bench.py --write-traffic <dir with the two rocprofv3 --pmc counter CSVs>",
             "entry_point = conef_randblock_conef_step_planned_f32",
             "chunk_cols = %d" % chunk_cols, "bin_buckets = %d" % bin_buckets,
             "kernel_sources_sha256_16 = %s" % kernel_sources_hash(),
             "calibration_copy_kib = %d" % copy_kib,
             "fetch_size_of_copy_kib = %.1f" % per["FETCH_SIZE"]["copy"], "fetch_factor = %.4f" % ff,
             "write_size_of_copy_kib = %.1f" % per["WRITE_SIZE"]["copy"], "write_factor = %.4f" % wf]
    for k in STEP_KERNELS:
        rd = per["FETCH_SIZE"][k] * ff * 1024
        wr = per["WRITE_SIZE"][k] * wf * 1024
        total += rd + wr
        lines += ["%s.fetch_size_kib = %.1f" % (k, per["FETCH_SIZE"][k]), "%s.write_size_kib = %.1f" % (k, per["WRITE_SIZE"][k]),
                  "%s.dispatches = %d" % (k, per["FETCH_SIZE"]["n"][k]),
                  "%s.read_bytes = %d" % (k, rd), "%s.written_bytes = %d" % (k, wr)]
    lines.append("bytes_per_step = %d" % round(total))
    with open(TRAFFIC_FILE, "w") as f:
        f.write("\n".join(lines) + "\n")
    print("\n".join(lines))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=600)
    ap.add_argument("--warmup", type=int, default=60)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget for the CPU baseline sample")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--write-traffic", metavar="DIR", help="condense the rocprofv3 --pmc CSVs in DIR into "
                    "the tracked traffic record (no GPU needed) and exit")
    args = ap.parse_args()
    if args.write_traffic:
        from conef_amd import _lib
        import numpy as np
        lib = _lib.load()
        w = max(int(N_COLS * SKETCH_SIZE), 1)
        nbytes = lib.conef_plan_bytes(N_ROWS, N_COLS, w, int(os.environ.get("CONEF_PLAN_CHUNK", "0")),
                                      int(os.environ.get("CONEF_PLAN_BIN", "0")))
        buf = np.zeros(nbytes, dtype=np.uint8)
        _lib.check(lib.conef_plan_build_host(buf.ctypes.data, nbytes, N_ROWS, N_COLS, w, 994443, 609478,
                                             int(os.environ.get("CONEF_PLAN_CHUNK", "0")),
                                             int(os.environ.get("CONEF_PLAN_BIN", "0"))), "conef_plan_build_host")
        i32 = buf[:128].view(np.int32)
        write_traffic(args.write_traffic, int(i32[9]), int(i32[11]))
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the ConEF compress+EF step has no cross-GPU part in this build "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from conef_amd import _lib
    from conef_amd.compressors.CountSketch import DenseCS

    if not torch.cuda.is_available():
        print("bench.py needs the GPU; there is no CPU path for the ConEF kernels", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    lib = _lib.load()
    L = N_ROWS * N_COLS
    block = max(1, int(RATIO * L))
    alpha = 1 - BETA

    # ---- resident inputs: one fresh gradient bucket per step (288 GB of HBM make that cheap), a
    # rotating set of sketch states and payload buffers, pre-drawn block offsets
    total_steps = args.warmup + args.steps
    n_grads = min(total_steps, MAX_GRAD_BUFFERS)
    gen = torch.Generator(device="cuda").manual_seed(20240607)

    def device_gradient():
        x = torch.randn(L, generator=gen, device="cuda") * 1e-3
        mask = torch.rand(L, generator=gen, device="cuda") < 0.01
        u = torch.rand(L, generator=gen, device="cuda") - 0.5
        lap = -1e-2 * torch.sign(u) * torch.log1p(-2 * u.abs())
        return torch.where(mask, lap, x).view(N_ROWS, N_COLS).contiguous()

    grads = [device_gradient() for _ in range(n_grads)]
    host_grad0 = grads[0].cpu()
    sketches = [DenseCS(N_ROWS, N_COLS, SKETCH_SIZE) for _ in range(N_BUCKETS)]
    payloads = [torch.empty(block, dtype=torch.float32, device="cuda") for _ in range(N_BUCKETS)]
    W = sketches[0].range
    rng = np.random.RandomState(42)
    starts = [int(rng.choice(L)) for _ in range(total_steps + 64)]
    stream = torch.cuda.current_stream().cuda_stream

    # every sketch of this shape shares one plan (tables) and, on one stream, one staging buffer
    plans = [cs.plan() for cs in sketches]
    planned = plans[0] is not None
    entry = "conef_randblock_conef_step_planned_f32" if planned else "conef_randblock_conef_step_f32"
    # Everything the rotating states will ever allocate exists, and has been written once, before the
    # first step: the second sketch buffer the step writes into, the payloads, the shared staging
    # buffer.  A short run (a handful of warm-up steps for twelve states) then times steady-state
    # steps, not first touches of fresh memory.
    for cs, payload in zip(sketches, payloads):
        (cs.spare_buffer() if planned else cs.next_buffer()).zero_()
        payload.zero_()
    staging_ptr = plans[0].workspace.data_ptr() if planned else 0
    if planned:
        plans[0].workspace.zero_()
    plan_host_ptr, plan_dev_ptr = (plans[0].host_ptr, plans[0].device.data_ptr()) if planned else (0, 0)

    def one_step(i, g, b):
        cs = sketches[b]
        if planned:
            out = cs.spare_buffer()
            rc = lib.conef_randblock_conef_step_planned_f32(
                g.data_ptr(), cs.cs.data_ptr(), out.data_ptr(), payloads[b].data_ptr(), plan_host_ptr,
                plan_dev_ptr, staging_ptr, N_ROWS, N_COLS, W, starts[i], block, alpha, BETA,
                cs.a, cs.b, stream)
            cs.commit(out)
        else:
            out = cs.next_buffer()
            rc = lib.conef_randblock_conef_step_f32(g.data_ptr(), cs.cs.data_ptr(), out.data_ptr(),
                                                    payloads[b].data_ptr(), N_ROWS, N_COLS, W, starts[i], block,
                                                    alpha, BETA, cs.a, cs.b, stream)
            cs.commit(out)
        if rc != 0:
            raise RuntimeError("%s returned %d" % (entry, rc))

    torch.cuda.synchronize()
    for i in range(args.warmup):
        one_step(i, grads[i % n_grads], i % N_BUCKETS)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(args.warmup, total_steps):
        one_step(i, grads[i % n_grads], i % N_BUCKETS)
    ev1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    gpu_ms = ev0.elapsed_time(ev1)
    ms_per_step = max(wall_ms, gpu_ms) / args.steps
    ev_ms_per_step = gpu_ms / args.steps

    # same-buffer (cache-resident) rate, reported for contrast
    same_steps = max(50, args.steps // 4)
    for i in range(10):
        one_step(i, grads[0], 0)
    torch.cuda.synchronize()
    ev0.record()
    for i in range(same_steps):
        one_step(i, grads[0], 0)
    ev1.record()
    torch.cuda.synchronize()
    same_ms = ev0.elapsed_time(ev1) / same_steps

    # practical ceiling: device-to-device copy of a > 256 MB buffer
    big = torch.empty(128 * 1024 * 1024, dtype=torch.float32, device="cuda")
    big2 = torch.empty_like(big)
    for _ in range(3):
        big2.copy_(big)
    torch.cuda.synchronize()
    ev0.record()
    for _ in range(10):
        big2.copy_(big)
    ev1.record()
    torch.cuda.synchronize()
    copy_gbs = 2 * big.numel() * 4 * 10 / (ev0.elapsed_time(ev1) * 1e-3) / 1e9
    del big, big2

    grad_gb = 4 * L / 1e9
    alg_bytes = algorithmic_bytes(L, N_ROWS, W, block)
    if planned:
        hdr = plans[0].header()
        traffic, traffic_note = read_traffic(hdr["chunk_cols"], hdr["bin_buckets"])
    else:
        traffic, traffic_note = None, "unplanned entry point"
    achieved = alg_bytes / (ev_ms_per_step * 1e-3) / 1e9

    result = {
        "metric": "GB/s gradient per ConEF compress+EF step (% HBM roofline), 25MB bucket, 1 GPU",
        "value": round(grad_gb / (ms_per_step * 1e-3), 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "RandomBlock 10% + count-sketch ConEF 10%, flat fp32 bucket [5,1300000] (26 MB), "
                        "sketch [5,130000], block 650000, beta 0.9",
            "entry_point": entry,
            "gradient_buffers": n_grads,
            "sketch_states_rotated": N_BUCKETS,
            "working_set_mb": round((n_grads * 4 * L + N_BUCKETS * (4 * block + 8 * N_ROWS * W)) / 1e6, 1),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "traffic_source": traffic_note,
            "launches_per_step": 2,
            "algorithmic_bytes_per_step": alg_bytes,
            "ms_per_step_hip_events": round(ev_ms_per_step, 5),
            "measured_copy_gbs": round(copy_gbs, 1),
            "frac_of_measured_copy": round(achieved / copy_gbs, 4),
        },
        "same_buffer": {"ms_per_step": round(same_ms, 5), "value": round(grad_gb / (same_ms * 1e-3), 2)},
        "host_wall_ms_per_step": round(wall_ms / args.steps, 5),
    }

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(host_grad0, W, block, alpha, args.cpu_seconds)
    print(json.dumps(result))


def cpu_baseline(grad, W, block, alpha, budget_s):
    """The C oracle's fused step on full 6.5 M-element buckets.  The rows of the sketch are
    independent, so they are spread over host threads (one per row: 5); the result is bit-identical
    to the single-threaded oracle, whose rate is reported next to it."""
    import numpy as np
    from oracle import conef_oracle as oracle

    L = N_ROWS * N_COLS
    x0 = grad.numpy().reshape(N_ROWS, N_COLS)
    payload = np.empty(block, dtype=np.float32)
    threads = max(1, min(N_ROWS, os.cpu_count() or 1))

    def timed(step_fn, budget, cap):
        cs = np.zeros((N_ROWS, W), dtype=np.float32)
        rng = np.random.RandomState(42)
        x = x0.copy()
        step_fn(x, cs, int(rng.choice(L)))     # warm-up
        times = []
        t_begin = time.perf_counter()
        while len(times) < 3 or (time.perf_counter() - t_begin < budget and len(times) < cap):
            x = x0.copy()
            start = int(rng.choice(L))
            t0 = time.perf_counter()
            step_fn(x, cs, start)
            times.append(time.perf_counter() - t0)
        return sorted(times)[len(times) // 2], len(times)

    med1, n1 = timed(lambda x, cs, st: oracle.randblock_conef_step(x, cs, payload, st, block, alpha, BETA),
                     budget_s * 0.4, 60)
    medt, nt = timed(lambda x, cs, st: oracle.randblock_conef_step_threaded(x, cs, payload, st, block, alpha, BETA,
                                                                            threads), budget_s * 0.6, 200)
    return {
        "value": round(4 * L / 1e9 / medt, 4),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": "%d full steps of the same [5,1300000] workload, C oracle with one thread per sketch row, "
                  "median %.1f ms/step; single thread: %d steps, median %.1f ms/step (%.4f GB/s); "
                  "host has %d logical CPUs" % (nt, medt * 1e3, n1, med1 * 1e3, 4 * L / 1e9 / med1, os.cpu_count()),
    }


if __name__ == "__main__":
    main()
