#!/usr/bin/env python3
"""Benchmark of the sparse-dense product path on one MI355X.

One step = one pass of the path over the headline pattern: P = DDS(A,B,S), C = A*S and
G = A_T *^ S at k=256 on the Zipf(1.1) 100000 x 500000 pattern with ~100 M nonzeros
(BASELINE.json configs[1] and configs[2] plus A*S on the same pattern, which the metric names).
Inputs are synthetic, seeded, and resident in HBM before the timed region.

Prints ONE JSON line. `value` is the algorithmic GB/s of the whole step (all three ops);
per-op figures, the roofline object of the DDS kernel and the CPU baseline ride along.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--scale S] [--no-cpu]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def alg_bytes(op, k, nnz, nrows, ncols):
    """Algorithmic bytes of one call: the gathered dense operand is charged once per nonzero,
    the streamed side once per column (row for A*^S), indices/values once."""
    if op in ("dds", "dsmult"):
        return nnz * (4 * k + 8) + ncols * (4 * k + 4) + 4
    if op == "dsmultT":
        return nnz * (4 * k + 8) + nrows * (4 * k + 4) + 4
    raise ValueError(op)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--scale", type=float, default=1.0, help="shrink rows/columns of the pattern (testing)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-sample", type=float, default=1.0, help="fraction of the columns timed on the CPU (1.0 = the whole workload)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch a plain streaming kernel of known size (C = A + B on 3 x 1 GiB) "
                         "before the steps: the scale for rocprofv3 FETCH_SIZE / WRITE_SIZE readings")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the path shards by "
              "columns of S, see DESIGN.md)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from bidmat_amd import gen, hip_abi
    from bidmat_amd.device import DeviceArray

    lib = hip_abi.load()     # raises if the HIP library is not built: no fallback
    ndev = C.c_int(0)
    hip_abi.check(lib.bidmat_device_count(C.byref(ndev)), "device_count")
    if ndev.value < 1:
        raise RuntimeError("no HIP device visible")
    hip_abi.check(lib.bidmat_set_device(0))
    arch = C.create_string_buffer(64)
    cus = C.c_int(0)
    mem = C.c_longlong(0)
    hip_abi.check(lib.bidmat_device_info(arch, 64, C.byref(cus), C.byref(mem)))

    t0 = time.time()
    cfg = gen.config("HEAD", args.scale)
    k, nrows, ncols = cfg["k"], cfg["nrows"], cfg["ncols"]
    ir, jc = cfg["ir"], cfg["jc"]
    nnz = int(ir.size)
    t_gen = time.time() - t0

    d_A = DeviceArray.from_numpy(cfg["A"])          # k x nrows  U(0,1)    (DDS, A*S)
    d_B = DeviceArray.from_numpy(cfg["B"])          # k x ncols  U(0,1)    (DDS)
    d_AT = DeviceArray.from_numpy(cfg["A_T"])       # k x ncols  N(0,1)    (A*^S)
    d_v = DeviceArray.from_numpy(cfg["vals"])       # nnz        U(0,1]
    d_ir = DeviceArray.from_numpy(ir)
    d_jc = DeviceArray.from_numpy(jc)
    d_P = DeviceArray(nnz, np.float32)
    d_C = DeviceArray(k * ncols, np.float32)
    d_G = DeviceArray(k * nrows, np.float32)

    # plan for A*^S: built once per pattern, timed separately
    plan = C.c_void_p()
    hip_abi.check(lib.bidmat_synchronize())
    t0 = time.time()
    hip_abi.check(lib.bidmat_plan_create(nrows, ncols, nnz, d_ir.ptr, d_jc.ptr, k, C.byref(plan)), "plan_create")
    hip_abi.check(lib.bidmat_synchronize())
    t_plan = time.time() - t0

    stream = C.c_void_p()
    hip_abi.check(lib.bidmat_stream_create(C.byref(stream)))

    def ev():
        e = C.c_void_p()
        hip_abi.check(lib.bidmat_event_create(C.byref(e)))
        return e

    def step(marks=None):
        if marks:
            hip_abi.check(lib.bidmat_event_record(marks[0], stream))
        hip_abi.check(lib.bidmat_dds_csc(k, ncols, nnz, d_A.ptr, d_B.ptr, d_ir.ptr, d_jc.ptr, d_P.ptr, 0, stream), "dds")
        if marks:
            hip_abi.check(lib.bidmat_event_record(marks[1], stream))
        hip_abi.check(lib.bidmat_dsmult_csc(k, ncols, nnz, d_A.ptr, d_v.ptr, d_ir.ptr, d_jc.ptr, d_C.ptr, 0, stream), "dsmult")
        if marks:
            hip_abi.check(lib.bidmat_event_record(marks[2], stream))
        hip_abi.check(lib.bidmat_dsmultT_plan(plan, k, d_AT.ptr, d_v.ptr, d_G.ptr, 0, stream), "dsmultT")
        if marks:
            hip_abi.check(lib.bidmat_event_record(marks[3], stream))

    if args.calibrate:
        ncal = 1 << 28                                   # 2^28 floats = 1 GiB per array
        cal = [DeviceArray(ncal, np.float32) for _ in range(3)]
        for c in cal:
            hip_abi.check(lib.bidmat_memset(c.ptr, 0, c.nbytes))
        for _ in range(3):                               # k_apply_full4: reads 2 GiB, writes 1 GiB
            hip_abi.check(lib.bidmat_applyop_flat(cal[0].ptr, cal[1].ptr, cal[2].ptr, ncal, 0, stream))
        hip_abi.check(lib.bidmat_stream_synchronize(stream))
        for c in cal:
            c.free()

    for _ in range(args.warmup):
        step()
    hip_abi.check(lib.bidmat_stream_synchronize(stream))

    marks = [[ev() for _ in range(4)] for _ in range(args.steps)]
    hip_abi.check(lib.bidmat_synchronize())
    t0 = time.perf_counter()
    for s in range(args.steps):
        step(marks[s])
    hip_abi.check(lib.bidmat_stream_synchronize(stream))
    hip_abi.check(lib.bidmat_synchronize())
    wall = time.perf_counter() - t0

    def elapsed(a, b):
        ms = C.c_float(0)
        hip_abi.check(lib.bidmat_event_elapsed_ms(a, b, C.byref(ms)))
        return float(ms.value)

    op_ms = {"dds": [], "dsmult": [], "dsmultT": []}
    for m in marks:
        op_ms["dds"].append(elapsed(m[0], m[1]))
        op_ms["dsmult"].append(elapsed(m[1], m[2]))
        op_ms["dsmultT"].append(elapsed(m[2], m[3]))
    ms_per_step = wall * 1e3 / args.steps

    ops = {}
    total_bytes = 0
    for op in ("dds", "dsmult", "dsmultT"):
        b = alg_bytes(op, k, nnz, nrows, ncols)
        total_bytes += b
        avg = float(np.mean(op_ms[op]))
        ops[op] = {
            "ms_avg": round(avg, 4), "ms_min": round(float(np.min(op_ms[op])), 4),
            "alg_GB": round(b / 1e9, 3),
            "GBps": round(b / avg / 1e6, 1),
            "nnz_per_s": round(nnz / avg * 1e3, 1),
            "GFLOPs": round(2.0 * k * nnz / avg / 1e6, 1),
            "frac_of_hbm_peak": round(b / avg / 1e6 / HBM_PEAK_GBS, 4),
        }
    value = total_bytes / (ms_per_step * 1e-3) / 1e9

    # roofline object: the DDS kernel (the configuration the metric is quoted on)
    dds_avg = float(np.mean(op_ms["dds"]))
    dds_bytes = alg_bytes("dds", k, nnz, nrows, ncols)
    roofline = {
        "kernel": "k_dds<W=4,V=1,LPN=64> (one launch = DDS over the whole pattern)",
        "bound": "hbm", "achieved": round(dds_bytes / dds_avg / 1e6, 1), "peak": HBM_PEAK_GBS,
        "unit": "GB/s", "frac": round(dds_bytes / dds_avg / 1e6 / HBM_PEAK_GBS, 4),
        "traffic": None,
        "bytes_per_launch": dds_bytes, "avg_launch_ms": round(dds_avg, 4),
    }

    out = {
        "metric": "achieved HBM GB/s (algorithmic bytes) for DDS + A*S + A*^S at k=256, ~100M nnz (1 GPU)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]+configs[2] pattern (Zipf(1.1) rows, Poisson(200) columns), "
                               "step = DDS, A*S, A*^S", "k": k, "nrows": nrows, "ncols": ncols, "nnz": nnz,
                   "scale": args.scale},
        "nnz_per_s": round(3 * nnz / (ms_per_step * 1e-3), 1),
        "GFLOPs": round(3 * 2.0 * k * nnz / (ms_per_step * 1e-3) / 1e9, 1),
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "ops": ops,
        "roofline": roofline,
        "plan": {"build_ms": round(t_plan * 1e3, 2), "segments": lib.bidmat_plan_segments(plan),
                 "bytes": lib.bidmat_plan_bytes(plan)},
        "device": {"arch": arch.value.decode(), "compute_units": cus.value, "mem_GiB": round(mem.value / 2**30, 1)},
        "gen_s": round(t_gen, 2),
    }

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg, args.cpu_sample)

    print(json.dumps(out))


def cpu_baseline(cfg, frac):
    """The CPU restatement of the reference's loops (oracle/, threads as the reference splits
    them) on the first `frac` of the columns of the same workload."""
    import oracle
    k, nrows, ncols = cfg["k"], cfg["nrows"], cfg["ncols"]
    nc = max(1, int(ncols * frac))
    jc = cfg["jc"][: nc + 1].copy()
    nnz = int(jc[-1])
    ir = cfg["ir"][:nnz]
    vals = cfg["vals"][:nnz]
    threads = oracle.max_threads()
    A, B, AT = cfg["A"], cfg["B"][: k * nc], cfg["A_T"][: k * nc]
    t = {}
    t0 = time.perf_counter(); oracle.dds(A, B, k, ir, jc, nthreads=threads); t["dds"] = time.perf_counter() - t0
    t0 = time.perf_counter(); oracle.fsmult(A, k, vals, ir, jc, nthreads=threads); t["dsmult"] = time.perf_counter() - t0
    t0 = time.perf_counter(); oracle.fsmultT(AT, k, nrows, vals, ir, jc, nthreads=threads); t["dsmultT"] = time.perf_counter() - t0
    total_b = sum(alg_bytes(op, k, nnz, nrows, nc) for op in t)
    total_s = sum(t.values())
    return {
        "value": round(total_b / total_s / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": "first %d of %d columns (%d nnz) of the same workload; DDS, A*S, A*^S each once; A*^S "
                  "uses min(cores, k/32) threads as the reference does" % (nc, ncols, nnz),
        "seconds": {op: round(s, 3) for op, s in t.items()},
        "nnz_per_s": round(3 * nnz / total_s, 1),
    }


if __name__ == "__main__":
    main()
