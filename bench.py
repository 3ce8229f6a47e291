#!/usr/bin/env python3
"""Benchmark of the sparse-dense product path on one MI355X.

Default workload ("headline"): one step = one pass of the path over the headline pattern:
P = DDS(A,B,S), C = A*S and G = A_T *^ S at k=256 on the Zipf(1.1) 100000 x 500000 pattern with
~100 M nonzeros (BASELINE.json configs[1] and configs[2] plus A*S on the same pattern, which
the metric names). Inputs are synthetic, seeded, and resident in HBM before the timed region.

Prints ONE JSON line. `value` is the algorithmic GB/s of the whole step (the gathered dense operand
charged once per nonzero, so caches can push it above the HBM peak); per-op figures, the roofline
object of the DDS kernel (with a bound that cannot exceed 1: compulsory bytes at the HBM peak, or
the same kernel's rate on an L2-resident operand, measured live), the CPU baseline and the check of
every timed output against the CPU oracle ride along.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|headline|C1|C4|C5]
                  [--scale S] [--no-cpu] [--calibrate]

The other workloads (C1: A*S k=32; C4: A*S k=1024 with Pareto columns; C5: the NMF update
chain at k=128, ~400 M nonzeros) are the remaining BASELINE.json configurations; the default run
times each over a few steps, checks it against the oracle and reports it under `workloads`
(`value` is always the headline's). "next" times the callers either side of the
path on the headline pattern (tile products, S*A / S^T*A, sparse op edge vector, file load);
"footprint" sweeps the gather kernels over the gathered footprint (where L1 / L2 / HBM serve).
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
# L2-miss bytes per launch of the roofline kernel at full scale (fabric side of L2: Infinity Cache
# and HBM together), from rocprofv3 FETCH_SIZE x 2.0 plus WRITE_SIZE x 1.0 (KiB per dispatch; the
# factors are what the same counters read for the streaming kernel of --calibrate, which moves a
# known 2 GiB + 1 GiB). A profiler cannot run inside this script, so each figure names the summary
# under profiles/ it was taken from and the sha256 (first 16 hex digits) of the kernel sources it
# was taken on (concatenated); it is reported only for that exact workload and dropped (null) as soon as the
# kernel source differs.
MEASURED_TRAFFIC = {
    ("headline", "dsmultT", 100003320): (34.5e9, ("bidmat_amd/csrc/spmm.hip", "bidmat_amd/csrc/dense_rows.hip"), "3675babc718fa305",
                                         "profiles/headline_kernel_trace_and_hbm_counters.txt"),
    ("C4", "dsmult", 38900534): (163.1e9, ("bidmat_amd/csrc/spmm.hip",), "d18cc32221214df7",
                                 "profiles/other_workloads_kernel_trace_and_hbm_counters.txt"),
}


def measured_traffic(workload, op, nnz):
    import hashlib
    rec = MEASURED_TRAFFIC.get((workload, op, nnz))
    if rec is None:
        return None, None
    nbytes, srcs, sha, where = rec
    try:
        m = hashlib.sha256()
        for src in srcs:
            m.update(open(os.path.join(ROOT, src), "rb").read())
        cur = m.hexdigest()[:16]
    except OSError:
        return None, None
    return (nbytes, where) if cur == sha else (None, None)


def alg_bytes(op, k, nnz, nrows, ncols):
    """Algorithmic bytes of one call: the gathered dense operand is charged once per nonzero,
    the streamed side once per column (row for A*^S), indices/values once."""
    if op in ("dds", "dsmult", "dds_op"):
        return nnz * (4 * k + 8) + ncols * (4 * k + 4) + 4 + (4 * nnz if op == "dds_op" else 0)
    if op == "dsmultT":
        return nnz * (4 * k + 8) + nrows * (4 * k + 4) + 4
    if op == "fused":              # the chain as the reference runs it: DDS with the elementwise op, then A*^S
        return alg_bytes("dds_op", k, nnz, nrows, ncols) + alg_bytes("dsmultT", k, nnz, nrows, ncols)
    if op == "ewise":              # elementwise on the nonzero values: two reads, one write
        return 12 * nnz
    if op == "rowsum":             # dense row sums of a k x ncols matrix
        return 4 * k * ncols + 4 * k
    raise ValueError(op)


def compulsory_bytes(op, k, nnz, nrows, ncols):
    """Every array of the call read or written exactly once (what an infinite cache would leave)."""
    if op in ("dds", "dds_op"):    # A, B, ir, jc, P (+ V)
        return 4 * k * (nrows + ncols) + 8 * nnz + 4 * (ncols + 1) + (4 * nnz if op == "dds_op" else 0)
    if op == "dsmult":             # A, values, ir, jc, C
        return 4 * k * (nrows + ncols) + 8 * nnz + 4 * (ncols + 1)
    if op == "dsmultT":            # A, values, column of each nonzero, row pointer, C
        return 4 * k * (nrows + ncols) + 8 * nnz + 4 * (nrows + 1)
    if op == "fused":              # both dense operands, values, column of each nonzero, row pointer, G
        return 4 * k * (2 * nrows + ncols) + 8 * nnz + 4 * (nrows + 1)
    return alg_bytes(op, k, nnz, nrows, ncols)


def flops(op, k, nnz, ncols):
    """The reference's own accounting (GMat.scala:1057,1092; GSMat.scala:665; length for the
    elementwise op and the reduction)."""
    if op in ("dds", "dsmult", "dsmultT", "dds_op"):
        return 2.0 * k * nnz + (nnz if op == "dds_op" else 0)
    if op == "fused":
        return 4.0 * k * nnz + nnz
    if op == "ewise":
        return float(nnz)
    return float(k) * ncols


def uncacheable_gather_bytes(ir, nrows, k, cache_bytes=32 << 20):
    """Bytes of row gathers that even an ideal cache of `cache_bytes` (all eight 4 MiB L2s holding disjoint rows,
    always the most frequent ones) would have to fetch from beyond L2: every gather of a row outside the
    cache_bytes / 4k most frequent rows. A kernel that walks S column by column cannot order these
    gathers away, so they bound its time at the rate of the memory side."""
    cnt = np.bincount(ir, minlength=nrows)
    keep = min(nrows, max(1, cache_bytes // (4 * k)))
    if keep >= nrows:
        return 0
    top = np.partition(cnt, nrows - keep)[nrows - keep:].sum()
    return int(cnt.sum() - top) * 4 * k


def op_bounds(kind, k, nnz, nrows, ncols, l2_rate_GBps, uncacheable, heavy_nnz=None):
    """Lower bounds on the time of one op in ms. compulsory: every array once at the HBM peak; l2_resident:
    all gathered bytes at the rate the same kernel reaches when every gather hits L2; uncacheable: the gathers
    an ideal 32 MiB L2 cannot hold, at the HBM peak. A*^S walks the plan's order, which an ideal-cache model of
    S's rows does not describe: its third term is the bound of that schedule, heavy-row gathers (reused inside
    a column panel) at the L2-resident rate plus light-row gathers (each dense column once per nonzero, no
    reuse) at the HBM peak."""
    terms = {"compulsory_ms": compulsory_bytes(kind, k, nnz, nrows, ncols) / (HBM_PEAK_GBS * 1e6)}
    gathered = nnz * 4.0 * k
    if l2_rate_GBps:
        terms["l2_resident_ms"] = gathered / (l2_rate_GBps * 1e6)
    if kind in ("dsmultT", "fused"):
        if heavy_nnz is not None and l2_rate_GBps:
            terms["plan_schedule_ms"] = heavy_nnz * 4.0 * k / (l2_rate_GBps * 1e6) + (nnz - heavy_nnz) * 4.0 * k / (HBM_PEAK_GBS * 1e6)
    elif uncacheable is not None:
        terms["uncacheable_ms"] = uncacheable / (HBM_PEAK_GBS * 1e6)
    return terms


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all", choices=["all", "headline", "C1", "C4", "C5", "next", "footprint"],
                    help="all (default): the headline workload as the timed `value`, plus short runs of C1, C4 and C5 "
                         "reported under `workloads`; any other name: that workload alone")
    ap.add_argument("--footprint-k", type=int, default=256, help="k of the footprint sweep")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink rows/columns of the pattern (testing)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU legs (baseline timing and verification)")
    ap.add_argument("--cpu-sample", type=float, default=1.0,
                    help="fraction of the columns timed on the CPU (1.0 = the whole workload)")
    ap.add_argument("--sections", default="probe,shaped,operator,graph,stored,chains",
                    help="side measurements around the timed steps, comma-separated: probe (L2-resident and streaming "
                         "rates for the bounded roofline), shaped (reference-shaped entries, repeated and fresh patterns), "
                         "operator (the GMat / GSMat operator layer), graph (HIP-graph replay), "
                         "stored (values stored in the plan), chains (the LDA / NMF factor updates as two calls and as one launch); 'none' runs the timed steps only, which keeps a profiler's "
                         "per-kernel averages clean")
    ap.add_argument("--set", action="append", default=[], metavar="NAME=VALUE",
                    help="library option set before anything runs (bidmat_set_option), repeatable")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch a plain streaming kernel of known size (C = A + B on 3 x 1 GiB) "
                         "before the steps: the scale for rocprofv3 FETCH_SIZE / WRITE_SIZE readings")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the path shards by "
              "columns of S; a multi-GPU figure is not part of this build)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from bidmat_amd import hip_abi

    lib = hip_abi.load()     # raises if the HIP library is not built: there is no fallback
    ndev = C.c_int(0)
    hip_abi.check(lib.bidmat_device_count(C.byref(ndev)), "device_count")
    if ndev.value < 1:
        raise RuntimeError("no HIP device visible")
    hip_abi.check(lib.bidmat_set_device(0))
    for item in args.set:
        oname, _, oval = item.partition("=")
        hip_abi.check(lib.bidmat_set_option(oname.encode(), int(oval)), "set_option " + item)

    sections = set() if args.sections == "none" else set(args.sections.split(","))
    if args.workload == "footprint":
        return footprint_sweep(lib, args)
    if args.workload == "next":
        return next_rows(lib, args)

    main_name = "headline" if args.workload == "all" else args.workload
    out = run_workload(lib, main_name, args.steps, args.warmup, args.scale, sections, not args.no_cpu, args.cpu_sample,
                       args.calibrate)
    if args.workload == "all":
        # the other configurations of the path, each timed over a few steps and checked against the oracle;
        # their CPU baselines run on labelled column samples so that the whole run stays within minutes
        out["workloads"] = {}
        for name, steps, sample in (("C1", 200, 1.0), ("C4", 10, 0.02), ("C5", 5, 0.005)):
            w = run_workload(lib, name, steps, 2, args.scale, {"probe"} & sections, not args.no_cpu, sample, False)
            out["workloads"][name] = {key: w[key] for key in ("metric", "value", "unit", "ms_per_step", "steps", "config", "ops", "roofline",
                                                              "alg_frac_of_hbm_peak", "plan", "cpu_baseline", "verified", "rowsum", "chain_forms")
                                      if key in w}
            hip_abi.check(lib.bidmat_release_caches())
        out["verified"] = bool(out.get("verified")) and all(w.get("verified") for w in out["workloads"].values()) \
            if not args.no_cpu else None
    print(json.dumps(out))
    if not args.no_cpu and not out["verified"]:
        print("bench.py: the timed outputs differ from the CPU oracle beyond 1e-4", file=sys.stderr)
        sys.exit(1)


def _without_dense_block(lib, call, stream, d_out):
    """The output of one A*^S call made with option dense_rows = 0 (every row through the plan's segments)."""
    from bidmat_amd import hip_abi
    before = lib.bidmat_get_option(b"dense_rows")
    hip_abi.check(lib.bidmat_set_option(b"dense_rows", 0))
    try:
        hip_abi.check(call())
        hip_abi.check(lib.bidmat_stream_synchronize(stream) if stream else lib.bidmat_synchronize())
    finally:
        hip_abi.check(lib.bidmat_set_option(b"dense_rows", before))
    return d_out.numpy()


def run_workload(lib, name, steps, warmup, scale, sections, cpu, cpu_sample, calibrate):
    """Times `steps` steps of one workload with inputs resident in HBM and returns its record."""
    from bidmat_amd import gen, hip_abi
    from bidmat_amd.device import DeviceArray

    arch = C.create_string_buffer(64)
    cus = C.c_int(0)
    mem = C.c_longlong(0)
    hip_abi.check(lib.bidmat_device_info(arch, 64, C.byref(cus), C.byref(mem)))

    t0 = time.time()
    cfg = gen.config("HEAD" if name == "headline" else name, scale)
    k, nrows, ncols = cfg["k"], cfg["nrows"], cfg["ncols"]
    ir, jc = cfg["ir"], cfg["jc"]
    nnz = int(ir.size)
    t_gen = time.time() - t0

    stream = C.c_void_p()
    hip_abi.check(lib.bidmat_stream_create(C.byref(stream)))
    h2d = {"bytes": 0, "s": 0.0}

    def up(a):       # host -> device copy of an input, timed (pageable host memory)
        t = time.perf_counter()
        d = DeviceArray.from_numpy(a)
        h2d["s"] += time.perf_counter() - t
        h2d["bytes"] += a.nbytes
        return d

    d_ir, d_jc = up(ir), up(jc)
    d_v = up(cfg["vals"])
    keep = [d_ir, d_jc, d_v]
    plan = C.c_void_p()
    t_plan = [None, None]

    def build_plan():
        # first build in the process (pays one-off costs: kernel loading, workspace growth), then
        # the build a caller sees from the second pattern on
        for i in range(2):
            if plan.value:
                hip_abi.check(lib.bidmat_plan_destroy(plan))
            hip_abi.check(lib.bidmat_synchronize())
            t = time.time()
            hip_abi.check(lib.bidmat_plan_create(nrows, ncols, nnz, d_ir.ptr, d_jc.ptr, k, C.byref(plan)), "plan_create")
            hip_abi.check(lib.bidmat_synchronize())
            t_plan[i] = time.time() - t

    def ev():
        e = C.c_void_p()
        hip_abi.check(lib.bidmat_event_create(C.byref(e)))
        return e

    # ---- the ops of one step: (name, kind, launcher). Every workload goes through a plan: the plan
    # holds what depends on the pattern alone, so no call builds or allocates anything.
    build_plan()
    outputs = {}
    stage_marks = None       # one event per step, recorded between the two stages of A*^S
    if name == "headline":
        d_A, d_B, d_AT = (up(cfg[x]) for x in ("A", "B", "A_T"))
        d_P, d_C, d_G = DeviceArray(nnz, np.float32), DeviceArray(k * ncols, np.float32), DeviceArray(k * nrows, np.float32)
        keep += [d_A, d_B, d_AT, d_P, d_C, d_G]
        outputs = {"dds": d_P, "dsmult": d_C, "dsmultT": d_G}
        stage_marks = [ev() for _ in range(steps)]
        cur = {"step": 0}
        ops = [
            ("dds", "dds", lambda: lib.bidmat_dds_plan(plan, k, d_A.ptr, d_B.ptr, d_ir.ptr, d_jc.ptr, None, 0, d_P.ptr, 0, stream)),
            ("dsmult", "dsmult", lambda: lib.bidmat_dsmult_plan(plan, k, d_A.ptr, d_v.ptr, d_ir.ptr, d_jc.ptr, d_C.ptr, 0, stream)),
            ("dsmultT", "dsmultT", lambda: lib.bidmat_dsmultT_plan_staged(plan, k, d_AT.ptr, d_v.ptr, d_G.ptr, 0, stream,
                                                                          stage_marks[cur["step"] % steps])),
        ]
        workload = "configs[1]+configs[2] pattern (Zipf(1.1) rows, Poisson(200) columns), step = DDS, A*S, A*^S"
        metric = "algorithmic GB/s (gathered operand charged once per nonzero) and nnz/s for DDS + A*S + A*^S at k=256, ~100M nnz (1 GPU)"
        roof_op = "dsmultT"
        roof_kernel = ("stage 1 of A*^S, the time-dominant part of the step: k_gather_axpy_sv<4,1,64,true> (the gathers of the pattern in plan "
                       "order) + k_dense_mfma<8,4> (the plan's densest rows as a dense block on the matrix cores) + k_dense_fold, "
                       "timed as one stretch of the stream; bytes and time are those of the three launches together")
    elif name in ("C1", "C4"):
        d_A = up(cfg["A"])
        d_C = DeviceArray(k * ncols, np.float32)
        keep += [d_A, d_C]
        outputs = {"dsmult": d_C}
        ops = [("dsmult", "dsmult", lambda: lib.bidmat_dsmult_plan(plan, k, d_A.ptr, d_v.ptr, d_ir.ptr, d_jc.ptr, d_C.ptr, 0, stream))]
        workload = "configs[0]: A*S, k=32, 50 nnz per column" if name == "C1" else \
            "configs[3]: A*S, k=1024, Pareto(1.5) column lengths in [1,50000]"
        metric = "algorithmic GB/s (gathered operand charged once per nonzero) for A*S (%s)" % name
        roof_op = "dsmult"
        roof_kernel = "k_gather_axpy<W=4,V=1,LPN=8>" if name == "C1" else "k_gather_axpy<W=4,V=4,LPN=64>"
    else:  # C5: Q = V ./ DDS(W,H,V) in one launch; G = H *^ Q; rs = sum(H,2)
        d_W, d_H = up(cfg["W"]), up(cfg["H"])
        d_Q, d_G, d_rs = DeviceArray(nnz, np.float32), DeviceArray(k * nrows, np.float32), DeviceArray(k, np.float32)
        d_rs2 = DeviceArray(k * nrows, np.float32)
        keep += [d_W, d_H, d_Q, d_G, d_rs, d_rs2]
        outputs = {"dds_op": d_Q, "dsmultT": d_G}
        # V, the data matrix, is the same in every iteration of the update: its values are stored in the
        # plan once (like the plan itself, outside the step) and the fused DDS streams them from there
        hip_abi.check(lib.bidmat_plan_set_values(plan, d_v.ptr, stream))
        # One walk over the plan's rows does the whole chain: every nonzero's column of H is gathered once and serves
        # the dot product and the accumulation; Q stays in registers (the two calls it replaces, and the variant that
        # also writes Q, are timed beside it under `chain_forms`).
        two_calls = [
            ("dds_op", lambda: lib.bidmat_dds_plan_stored(plan, k, d_W.ptr, d_H.ptr, d_ir.ptr, d_jc.ptr, 3, d_Q.ptr, stream)),
            ("dsmultT", lambda: lib.bidmat_dsmultT_plan(plan, k, d_H.ptr, d_Q.ptr, d_G.ptr, 0, stream)),
        ]
        ops = [("dds_dsmultT", "fused",
                lambda: lib.bidmat_dds_dsmultT_plan(plan, k, d_W.ptr, d_H.ptr, None, 3, None, d_G.ptr, 0, stream))]
        workload = "configs[4]: NMF update chain Q = V ./ DDS(W,H,V), G = H *^ Q in one launch over the plan's rows (dense row sums timed apart)"
        metric = "algorithmic GB/s (the chain's two gathers per nonzero charged as the reference runs them) for the NMF update chain at k=128, ~400M nnz"
        roof_op, roof_kernel = "dds_dsmultT", "k_fused_rows<W=4,V=1,LPN=32> + k_reduce_segments"

    def step(marks=None):
        for i, (opname, _, fn) in enumerate(ops):
            if marks:
                hip_abi.check(lib.bidmat_event_record(marks[i], stream))
            hip_abi.check(fn(), opname)
        if marks:
            hip_abi.check(lib.bidmat_event_record(marks[len(ops)], stream))

    if calibrate:
        ncal = 1 << 28                                   # 2^28 floats = 1 GiB per array
        cal = [DeviceArray(ncal, np.float32) for _ in range(3)]
        for c in cal:
            hip_abi.check(lib.bidmat_memset(c.ptr, 0, c.nbytes))
        for _ in range(3):                               # k_apply_full4: reads 2 GiB, writes 1 GiB
            hip_abi.check(lib.bidmat_applyop_flat(cal[0].ptr, cal[1].ptr, cal[2].ptr, ncal, 0, stream))
        hip_abi.check(lib.bidmat_stream_synchronize(stream))
        for c in cal:
            c.free()

    for _ in range(warmup):
        step()
    hip_abi.check(lib.bidmat_stream_synchronize(stream))

    marks = [[ev() for _ in range(len(ops) + 1)] for _ in range(steps)]
    hip_abi.check(lib.bidmat_synchronize())
    t0 = time.perf_counter()
    for s in range(steps):
        if stage_marks:
            cur["step"] = s
        step(marks[s])
    hip_abi.check(lib.bidmat_stream_synchronize(stream))
    hip_abi.check(lib.bidmat_synchronize())
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / steps

    def elapsed(a, b):
        ms = C.c_float(0)
        hip_abi.check(lib.bidmat_event_elapsed_ms(a, b, C.byref(ms)))
        return float(ms.value)

    per_op, total_bytes, total_flops = {}, 0, 0.0
    for i, (opname, kind, _) in enumerate(ops):
        t = [elapsed(m[i], m[i + 1]) for m in marks]
        b = alg_bytes(kind, k, nnz, nrows, ncols)
        total_bytes += b
        total_flops += flops(kind, k, nnz, ncols)
        avg = float(np.mean(t))
        per_op[opname] = {
            "ms_avg": round(avg, 4), "ms_median": round(float(np.median(t)), 4), "ms_min": round(float(np.min(t)), 4),
            "alg_GB": round(b / 1e9, 3), "compulsory_GB": round(compulsory_bytes(kind, k, nnz, nrows, ncols) / 1e9, 3),
            "alg_GBps": round(b / avg / 1e6, 1), "nnz_per_s": round(nnz / avg * 1e3, 1),
            "GFLOPs": round(flops(kind, k, nnz, ncols) / avg / 1e6, 1),
            "alg_frac_of_hbm_peak": round(b / avg / 1e6 / HBM_PEAK_GBS, 4),
        }
    if stage_marks:
        t1 = [elapsed(marks[s][2], stage_marks[s]) for s in range(steps)]
        t2 = [elapsed(stage_marks[s], marks[s][3]) for s in range(steps)]
        per_op["dsmultT"]["stage1_gather_ms_avg"] = round(float(np.mean(t1)), 4)
        per_op["dsmultT"]["stage2_reduce_ms_avg"] = round(float(np.mean(t2)), 4)
    value = total_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- what bounds every op, measured on this device in this run: the rate of the same gather kernels
    # when the gathered rows fit in L2 (the ceiling of a kernel whose every gather is served by L2), the
    # plain streaming rate of the device, and from the pattern itself the gathers no L2 could hold.
    heavy_nnz = lib.bidmat_plan_heavy_nnz(plan) if any(o[1] in ("dsmultT", "fused") for o in ops) else None
    uncache = uncacheable_gather_bytes(ir, nrows, k) if "probe" in sections else None
    live = {}
    if "probe" in sections:
        for kind in sorted({("dds" if o[1] in ("dds", "dds_op") else "dsmult") for o in ops}):
            live[kind] = live_rates(lib, stream, k, kind)
    for opname, kind, _ in ops:
        lr = live.get("dds" if kind in ("dds", "dds_op") else "dsmult")
        terms = op_bounds(kind, k, nnz, nrows, ncols, lr["l2_resident_gather_GBps"] if lr else None, uncache, heavy_nnz)
        bound = max(v for key, v in terms.items() if key != "plan_schedule_ms")
        per_op[opname]["bound_terms_ms"] = {key: round(v, 4) for key, v in terms.items()}
        per_op[opname]["bound_ms"] = round(bound, 4)
        per_op[opname]["frac_of_bound"] = round(bound / per_op[opname]["ms_avg"], 4)
        if "plan_schedule_ms" in terms:
            per_op[opname]["frac_of_plan_schedule_bound"] = round(terms["plan_schedule_ms"] / per_op[opname]["ms_avg"], 4)
    r = per_op[roof_op]
    # the dominant kernel's own launch time where the step marks it (stage 1 of A*^S), else its op's time
    r_avg = r.get("stage1_gather_ms_avg", r["ms_avg"])
    roof_kind = [o[1] for o in ops if o[0] == roof_op][0]
    r_bytes = alg_bytes(roof_kind, k, nnz, nrows, ncols)
    if "stage1_gather_ms_avg" in r:
        # stage 1 alone: per nonzero one gathered column, its index and its value; per segment one partial sum written
        r_bytes = nnz * (4 * k + 8) + lib.bidmat_plan_segments(plan) * (4 * k + 4) + 4
    lr = live.get("dds" if roof_op in ("dds", "dds_op") else "dsmult")
    traffic, traffic_src = measured_traffic(name, roof_op, nnz)
    roofline = {
        "kernel": roof_kernel, "bound": "hbm", "achieved": round(r_bytes / r_avg / 1e6, 1), "peak": HBM_PEAK_GBS,
        "unit": "GB/s", "frac": round(r_bytes / r_avg / 1e6 / HBM_PEAK_GBS, 4),
        "frac_basis": "ALGORITHMIC bytes / time / 8 TB/s: every gathered row is charged per nonzero although L1/L2 serve "
                      "most of them, so this can exceed 1; the bounded utilisation figure is frac_of_bound",
        "traffic": traffic, "traffic_source": traffic_src,
        "bytes_per_launch": r_bytes, "avg_launch_ms": round(r_avg, 4),
        "compulsory_bytes": compulsory_bytes(roof_kind, k, nnz, nrows, ncols), "gathered_bytes": nnz * 4 * k,
        "uncacheable_gather_bytes": uncache if roof_op not in ("dsmultT", "dds_dsmultT") else None,
        "heavy_row_nnz": heavy_nnz if roof_op in ("dsmultT", "dds_dsmultT") else None,
        "l2_resident_gather_GBps": lr["l2_resident_gather_GBps"] if lr else None, "l2_resident_probe": lr["probe"] if lr else None,
        "stream_GBps": lr["stream_GBps"] if lr else None,
        "bound_ms": r.get("bound_ms"), "frac_of_bound": round(r["bound_ms"] / r_avg, 4) if r.get("bound_ms") else None,
        "frac_of_plan_schedule_bound": round(r["bound_terms_ms"]["plan_schedule_ms"] / r_avg, 4)
        if r.get("bound_terms_ms", {}).get("plan_schedule_ms") else None,
        "bound_basis": "max(compulsory bytes / 8 TB/s, gathered bytes / rate of the same kernel with an L2-resident operand, "
                       "gathers that an ideal 32 MiB L2 cannot hold / 8 TB/s); plan_schedule: heavy-row gathers at the L2-resident "
                       "rate + light-row gathers at 8 TB/s",
    }
    if traffic:
        # L2-miss (fabric-side) bytes over time: Infinity Cache and HBM together, not an HBM fraction
        roofline["l2_miss_GBps"] = round(traffic / r_avg / 1e6, 1)

    out = {
        "metric": metric, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": workload, "k": k, "nrows": nrows, "ncols": ncols, "nnz": nnz, "scale": scale},
        "nnz_per_s": round(len([o for o in ops if o[1] != "ewise"]) * nnz / (ms_per_step * 1e-3), 1),
        "GFLOPs": round(total_flops / (ms_per_step * 1e-3) / 1e9, 1),
        "alg_frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "ops": per_op, "roofline": roofline,
        "api_form": "every op of the timed step goes through a plan handle (bidmat_*_plan); what callers without a handle get "
                    "is under reference_shaped_ms_incl_clear and operator_api_ms",
        "device": {"arch": arch.value.decode(), "compute_units": cus.value, "mem_GiB": round(mem.value / 2**30, 1)},
        "gen_s": round(t_gen, 2),
        # informational: what one step would cost if every input crossed PCIe first (never `value`)
        "h2d": {"GB": round(h2d["bytes"] / 1e9, 3), "s": round(h2d["s"], 3),
                "GBps": round(h2d["bytes"] / h2d["s"] / 1e9, 2),
                "step_GBps_incl_h2d": round(total_bytes / (ms_per_step * 1e-3 + h2d["s"]) / 1e9, 1)},
    }
    out["plan"] = {"first_build_ms": round(t_plan[0] * 1e3, 2), "build_ms": round(t_plan[1] * 1e3, 2),
                   "segments": lib.bidmat_plan_segments(plan), "bytes": lib.bidmat_plan_bytes(plan),
                   "column_overflow_segments": lib.bidmat_plan_overflow_segments(plan)}
    if "dsmultT" in per_op:
        # what a caller with a fresh pattern on every call (a BIDMach minibatch) pays for A*^S
        per_op["dsmultT_incl_plan_ms"] = round(per_op["dsmultT"]["ms_avg"] + t_plan[1] * 1e3, 4)
    if name == "C5":
        # the chain's other forms: the two calls the fused launch replaces, and the fused launch that also writes Q
        forms = {n + "_ms": round(_timed(lib, f, stream, 3, warm=1), 4) for n, f in two_calls}
        forms["two_calls_ms"] = round(forms["dds_op_ms"] + forms["dsmultT_ms"], 4)
        # the bits of the one launch are those of the two calls walking the plan's segments for every row: the A*^S
        # call is repeated once without the plan's dense block (which adds the most frequent rows' terms in another order)
        g_two = _without_dense_block(lib, two_calls[1][1], stream, d_G)
        q_two = d_Q.numpy()
        fq = lambda: lib.bidmat_dds_dsmultT_plan(plan, k, d_W.ptr, d_H.ptr, None, 3, d_Q.ptr, d_G.ptr, 0, stream)
        hip_abi.check(lib.bidmat_memset(d_Q.ptr, 0, d_Q.nbytes))
        forms["one_launch_also_writing_Q_ms"] = round(_timed(lib, fq, stream, 3, warm=1), 4)
        forms["one_launch_same_bits_as_two_calls"] = bool(np.array_equal(g_two.view(np.uint32), d_G.numpy().view(np.uint32)) and
                                                          np.array_equal(q_two.view(np.uint32), d_Q.numpy().view(np.uint32)))
        del g_two, q_two
        # the gathers alone, for scale: A*^S with the plan's stored values (V, not Q: a timing, not a result of the chain)
        forms["dsmultT_alone_values_in_plan_order_ms"] = round(_timed(
            lib, lambda: lib.bidmat_dsmultT_plan(plan, k, d_H.ptr, None, d_rs2.ptr, 0, stream), stream, 3, warm=1), 4)
        out["chain_forms"] = forms
        per_op["dds_dsmultT_incl_plan_ms"] = round(per_op["dds_dsmultT"]["ms_avg"] + t_plan[1] * 1e3, 4)
    if name == "C5":      # the dense row sums of H, timed apart from the chain
        e0, e1 = ev(), ev()
        hip_abi.check(lib.bidmat_reduce2op(k, ncols, d_H.ptr, d_rs.ptr, 0.0, 0))
        hip_abi.check(lib.bidmat_event_record(e0, None))
        for _ in range(5):
            hip_abi.check(lib.bidmat_reduce2op(k, ncols, d_H.ptr, d_rs.ptr, 0.0, 0))
        hip_abi.check(lib.bidmat_event_record(e1, None))
        hip_abi.check(lib.bidmat_synchronize())
        t = elapsed(e0, e1) / 5
        b = alg_bytes("rowsum", k, nnz, nrows, ncols)
        out["rowsum"] = {"ms_avg": round(t, 4), "GBps": round(b / t / 1e6, 1),
                         "frac_of_hbm_peak": round(b / t / 1e6 / HBM_PEAK_GBS, 4)}

    # the outputs of the timed steps, checked below
    results = {opname: d.numpy() for opname, d in outputs.items()} if cpu else {}

    if name == "headline" and "shaped" in sections:
        out["reference_shaped_ms_incl_clear"] = shaped_entries(lib, k, nrows, ncols, nnz, d_ir, d_jc, d_v, d_A, d_B, d_AT,
                                                               d_P, d_C, d_G)
    if name == "headline" and "operator" in sections:
        out["operator_api_ms"] = operator_layer(cfg)

    if name == "headline" and "chains" in sections:
        # The two factor updates of an LDA / NMF step on this pattern, each as the two calls the reference's
        # operators make (DDS with the elementwise op fused, then the product) and as one launch that gathers once:
        # E-step Q = V ./ DDS(A,B,S), C = A * Q (by columns); M-step G = B *^ Q (by the plan's rows).
        d_Q2, d_C2, d_G2 = DeviceArray(nnz, np.float32), DeviceArray(k * ncols, np.float32), DeviceArray(k * nrows, np.float32)
        ch = {}
        ch["e_step_dds_op_ms"] = round(_timed(lib, lambda: lib.bidmat_dds_plan(plan, k, d_A.ptr, d_B.ptr, d_ir.ptr, d_jc.ptr, d_v.ptr, 3, d_Q2.ptr, 0, stream), stream, 5), 4)
        ch["e_step_dsmult_ms"] = round(_timed(lib, lambda: lib.bidmat_dsmult_plan(plan, k, d_A.ptr, d_Q2.ptr, d_ir.ptr, d_jc.ptr, d_C2.ptr, 0, stream), stream, 5), 4)
        ch["e_step_two_calls_ms"] = round(ch["e_step_dds_op_ms"] + ch["e_step_dsmult_ms"], 4)
        c_two_plan = d_C2.numpy()              # what the two plan calls left
        ch["e_step_one_launch_ms"] = round(_timed(lib, lambda: lib.bidmat_dds_dsmult_csc(k, ncols, nnz, d_A.ptr, d_B.ptr, d_ir.ptr, d_jc.ptr, d_v.ptr, 3, None, d_C2.ptr, 0, stream), stream, 5), 4)
        ch["e_step_one_launch_through_plan_ms"] = round(_timed(lib, lambda: lib.bidmat_dds_dsmult_plan(plan, k, d_A.ptr, d_B.ptr, d_ir.ptr, d_jc.ptr, d_v.ptr, 3, None, d_C2.ptr, 0, stream), stream, 5), 4)
        ch["e_step_through_plan_same_bits_as_two_calls"] = bool(np.array_equal(c_two_plan.view(np.uint32), d_C2.numpy().view(np.uint32)))
        del c_two_plan
        ch["m_step_dsmultT_ms"] = round(_timed(lib, lambda: lib.bidmat_dsmultT_plan(plan, k, d_B.ptr, d_Q2.ptr, d_G2.ptr, 0, stream), stream, 5), 4)
        ch["m_step_two_calls_ms"] = round(ch["e_step_dds_op_ms"] + ch["m_step_dsmultT_ms"], 4)
        g_two = _without_dense_block(lib, lambda: lib.bidmat_dsmultT_plan(plan, k, d_B.ptr, d_Q2.ptr, d_G2.ptr, 0, stream), stream, d_G2)
        ch["m_step_one_launch_ms"] = round(_timed(lib, lambda: lib.bidmat_dds_dsmultT_plan(plan, k, d_A.ptr, d_B.ptr, d_v.ptr, 3, None, d_G2.ptr, 0, stream), stream, 5), 4)
        ch["m_step_one_launch_same_bits_as_two_calls"] = bool(np.array_equal(g_two.view(np.uint32), d_G2.numpy().view(np.uint32)))
        del g_two
        for d in (d_Q2, d_C2, d_G2):
            d.free()
        out["chain_forms"] = ch

    if name == "headline" and "stored" in sections:
        # Callers whose values stay fixed over several calls (the data matrix of an LDA minibatch) can
        # store them in the plan, in plan order: A*^S, A*S and the sparse row sums then stream them.
        d_rs = DeviceArray(nrows, np.float32)
        keep.append(d_rs)
        sv = {"set_values_ms": round(_timed(lib, lambda: lib.bidmat_plan_set_values(plan, d_v.ptr, stream), stream, 5), 4),
              "dsmultT_ms": round(_timed(lib, lambda: lib.bidmat_dsmultT_plan(plan, k, d_AT.ptr, None, d_G.ptr, 0, stream), stream, 5), 4),
              "spsum_rows_ms": round(_timed(lib, lambda: lib.bidmat_spsum_rows_plan(plan, None, d_rs.ptr, 0, stream), stream, 5), 4),
              "spsum_rows_fresh_values_ms": round(_timed(lib, lambda: lib.bidmat_spsum_rows_csc(nrows, nnz, d_ir.ptr, d_v.ptr, d_rs.ptr, 0, stream), stream, 5), 4),
              "spsum_rows_fresh_values_through_plan_ms": round(_timed(lib, lambda: lib.bidmat_spsum_rows_plan(plan, d_v.ptr, d_rs.ptr, 0, stream), stream, 5), 4)}
        if lib.bidmat_dsmult_plan(plan, k, d_A.ptr, None, d_ir.ptr, d_jc.ptr, d_C.ptr, 0, stream) == 0:
            sv["dsmult_ms"] = round(_timed(lib, lambda: lib.bidmat_dsmult_plan(plan, k, d_A.ptr, None, d_ir.ptr, d_jc.ptr, d_C.ptr, 0, stream), stream, 5), 4)
        out["values_stored_in_plan"] = sv

    if name in ("C1", "headline") and "graph" in sections:
        # the same step recorded once into a HIP graph and replayed with one launch per step
        if stage_marks:
            ops[2] = ("dsmultT", "dsmultT", lambda: lib.bidmat_dsmultT_plan(plan, k, d_AT.ptr, d_v.ptr, d_G.ptr, 0, stream))
        gx = C.c_void_p()
        hip_abi.check(lib.bidmat_graph_begin_capture(stream))
        step()
        hip_abi.check(lib.bidmat_graph_end_capture(stream, C.byref(gx)))
        reps = 200 if name == "C1" else steps
        for _ in range(3):
            hip_abi.check(lib.bidmat_graph_launch(gx, stream))
        e0, e1 = ev(), ev()
        hip_abi.check(lib.bidmat_event_record(e0, stream))
        for _ in range(reps):
            hip_abi.check(lib.bidmat_graph_launch(gx, stream))
        hip_abi.check(lib.bidmat_event_record(e1, stream))
        hip_abi.check(lib.bidmat_stream_synchronize(stream))
        out["graph_replay"] = {"ms_per_step": round(elapsed(e0, e1) / reps, 4), "steps": reps}
        hip_abi.check(lib.bidmat_graph_destroy(gx))

    # device memory back before the CPU legs (and the next workload)
    hip_abi.check(lib.bidmat_synchronize())
    hip_abi.check(lib.bidmat_plan_destroy(plan))
    for d in keep:
        d.free()
    hip_abi.check(lib.bidmat_stream_destroy(stream))

    if cpu:
        out["cpu_baseline"] = cpu_baseline(name, cfg, cpu_sample)
        checks = verify_outputs(name, cfg, results)
        for opname, c in checks.items():
            if opname in per_op:
                per_op[opname].update(c)
            else:                       # an output of a fused launch: filed under the launch
                per_op[ops[0][0]]["check_" + opname] = c
        out["verified"] = bool(checks) and all(c["max_err_measure"] <= 1e-4 for c in checks.values())
    return out


def shaped_entries(lib, k, nrows, ncols, nnz, d_ir, d_jc, d_v, d_A, d_B, d_AT, d_P, d_C, d_G):
    """What unchanged call sites get: the blocking entries with the reference's argument lists (per-nonzero
    column array, no column pointer, no plan handle), each preceded by the clear of its output that
    GSMult / GSMultT / DDS do; wall clock around clear + call. `repeated`: the same device arrays call after
    call (from the second call on the entries find the pattern's cached plan). `fresh`: a pattern the
    library has not seen, in new device arrays, on every call (a new minibatch): DDS and A*S run the plain
    kernels, A*^S builds its row plan inside the call."""
    from bidmat_amd import hip_abi
    from bidmat_amd.device import DeviceArray
    d_ic = DeviceArray(nnz, np.int32)
    hip_abi.check(lib.bidmat_csc_expand_cols(ncols, nnz, d_jc.ptr, d_ic.ptr, None))
    hip_abi.check(lib.bidmat_synchronize())

    def calls(ir_ptr, ic_ptr):
        return (("dds", d_P, lambda: lib.bidmat_dds(k, nnz, d_A.ptr, d_B.ptr, ir_ptr, ic_ptr, d_P.ptr)),
                ("dsmult", d_C, lambda: lib.bidmat_dsmult(k, ncols, nnz, d_A.ptr, d_v.ptr, ir_ptr, ic_ptr, d_C.ptr)),
                ("dsmultT", d_G, lambda: lib.bidmat_dsmultT(k, ncols, nnz, d_AT.ptr, d_v.ptr, ir_ptr, ic_ptr, d_G.ptr)))

    def timed(outbuf, call, what):
        hip_abi.check(lib.bidmat_synchronize())
        t0 = time.perf_counter()
        hip_abi.check(lib.bidmat_memset(outbuf.ptr, 0, outbuf.nbytes))
        hip_abi.check(call(), what)
        return (time.perf_counter() - t0) * 1e3

    hip_abi.check(lib.bidmat_release_caches())
    repeated, first = {}, {}
    for opname, outbuf, call in calls(d_ir.ptr, d_ic.ptr):
        ts = [timed(outbuf, call, opname) for _ in range(7)]
        first[opname] = [round(t, 3) for t in ts[:3]]      # 1st: plain kernel / plan build; 2nd: column side built
        repeated[opname] = round(float(np.median(ts[3:])), 3)
    fresh = {}
    for opname in ("dds", "dsmult", "dsmultT"):
        ts = []
        for r in range(4):
            # another pattern of the same size and statistics in device arrays of its own (the columns rotated by a
            # different amount every time: the cache goes by the content of the index arrays, not by their addresses);
            # the values stay where they are - these calls are timed, not checked
            c0 = 1000 * (len(fresh) * 4 + r + 1)
            j0 = np.zeros(1, np.int32)
            hip_abi.check(lib.bidmat_memcpy_d2h(j0.ctypes.data, d_jc.ptr + 4 * c0, 4))
            j0 = int(j0[0])
            f_ir, f_ic = DeviceArray(nnz, np.int32), DeviceArray(nnz, np.int32)
            for dst, src in ((f_ir, d_ir), (f_ic, d_ic)):
                hip_abi.check(lib.bidmat_memcpy_d2d(dst.ptr, src.ptr + 4 * j0, 4 * (nnz - j0)))
                hip_abi.check(lib.bidmat_memcpy_d2d(dst.ptr + 4 * (nnz - j0), src.ptr, 4 * j0))
            hip_abi.check(lib.bidmat_index_shift(f_ic.ptr, nnz - j0, -c0, None))
            hip_abi.check(lib.bidmat_index_shift(f_ic.ptr + 4 * (nnz - j0), j0, ncols - c0, None))
            _, outbuf, call = [c for c in calls(f_ir.ptr, f_ic.ptr) if c[0] == opname][0]
            ts.append(timed(outbuf, call, opname))
            f_ir.free(); f_ic.free()
        fresh[opname] = round(float(np.median(ts[1:])), 3)
    hip_abi.check(lib.bidmat_release_caches())
    d_ic.free()
    return {"repeated_pattern": repeated, "fresh_pattern": fresh, "first_three_calls": first}


def operator_layer(cfg):
    """The same three products through the GMat / GSMat operator layer (libbidmathost, the stand-in for the
    Scala classes): wall clock around each blocking operator call with the output matrix reused, median of
    five calls after the two that build the pattern's plan."""
    from bidmat_amd import mats
    k, nrows, ncols = cfg["k"], cfg["nrows"], cfg["ncols"]
    mats.Mat.set("ioneBased", 0)
    try:
        S = mats.GSMat.from_csc(nrows, ncols, cfg["vals"], cfg["ir"], cfg["jc"])
        gA = mats.GMat.from_numpy(cfg["A"].reshape(nrows, k).T)
        gB = mats.GMat.from_numpy(cfg["B"].reshape(ncols, k).T)
        gAT = mats.GMat.from_numpy(cfg["A_T"].reshape(ncols, k).T)
        res = {}
        for opname, first, again in (
                ("DDS", lambda: mats.DDS(gA, gB, S), lambda o: mats.DDS(gA, gB, S, o)),
                ("GSMult (A*S)", lambda: gA.GSMult(S), lambda o: gA.GSMult(S, o)),
                ("GSMultT (A*^S)", lambda: gAT.GSMultT(S), lambda o: gAT.GSMultT(S, o))):
            o = first()
            ts = []
            for _ in range(7):
                t0 = time.perf_counter()
                again(o)
                ts.append((time.perf_counter() - t0) * 1e3)
            res[opname] = round(float(np.median(ts[2:])), 3)
            del o
        return res
    finally:
        mats.Mat.set("ioneBased", 1)


def live_rates(lib, stream, k, op):
    """Two reference rates of this device, measured with the library's own kernels:
    the DDS / A*S kernel on 100 000 columns x 200 nonzeros whose rows are uniform over 2 MiB of the
    gathered operand (half of one XCD's L2: every gather is an L2 hit, or an L1 hit), as algorithmic
    gather bytes per second, and a streaming add over 3 x 256 MiB."""
    from bidmat_amd import hip_abi
    from bidmat_amd.device import DeviceArray
    ncols, L = 100000, 200
    R = max(16, (2 << 20) // (4 * k))
    nnz = ncols * L
    rng = np.random.default_rng(0)
    d_A = DeviceArray.from_numpy(rng.random(k * R, dtype=np.float32))
    d_B = DeviceArray.from_numpy(rng.random(k * ncols, dtype=np.float32))
    d_v = DeviceArray.from_numpy(rng.random(nnz, dtype=np.float32))
    d_jc = DeviceArray.from_numpy((np.arange(ncols + 1) * L).astype(np.int32))
    d_ir = DeviceArray.from_numpy(rng.integers(0, R, size=nnz).astype(np.int32))
    if op == "dds":
        d_o = DeviceArray(nnz, np.float32)
        fn = lambda: lib.bidmat_dds_csc(k, ncols, nnz, d_A.ptr, d_B.ptr, d_ir.ptr, d_jc.ptr, d_o.ptr, 0, stream)
    else:
        d_o = DeviceArray(k * ncols, np.float32)
        fn = lambda: lib.bidmat_dsmult_csc(k, ncols, nnz, d_A.ptr, d_v.ptr, d_ir.ptr, d_jc.ptr, d_o.ptr, 0, stream)
    t = _timed(lib, fn, stream, 5)
    gather = nnz * 4.0 * k / t / 1e6
    n = 1 << 26
    s = [DeviceArray(n, np.float32) for _ in range(3)]
    for x in s:
        hip_abi.check(lib.bidmat_memset(x.ptr, 0, x.nbytes))
    t2 = _timed(lib, lambda: lib.bidmat_applyop_flat(s[0].ptr, s[1].ptr, s[2].ptr, n, 0, stream), stream, 5)
    for x in [d_A, d_B, d_v, d_jc, d_ir, d_o] + s:
        x.free()
    return {"l2_resident_gather_GBps": round(gather, 1), "stream_GBps": round(12.0 * n / t2 / 1e6, 1),
            "probe": "%s kernel, k=%d, %d columns x %d nonzeros, rows uniform over %d rows (2 MiB), %.3f ms" % (op, k, ncols, L, R, t)}


def _timed(lib, fn, stream, reps, warm=2):
    from bidmat_amd import hip_abi
    for _ in range(warm):
        hip_abi.check(fn())
    e0, e1 = C.c_void_p(), C.c_void_p()
    hip_abi.check(lib.bidmat_event_create(C.byref(e0)))
    hip_abi.check(lib.bidmat_event_create(C.byref(e1)))
    hip_abi.check(lib.bidmat_event_record(e0, stream))
    for _ in range(reps):
        hip_abi.check(fn())
    hip_abi.check(lib.bidmat_event_record(e1, stream))
    hip_abi.check(lib.bidmat_stream_synchronize(stream))
    hip_abi.check(lib.bidmat_synchronize())
    ms = C.c_float(0)
    hip_abi.check(lib.bidmat_event_elapsed_ms(e0, e1, C.byref(ms)))
    return ms.value / reps


def footprint_sweep(lib, args):
    """DDS and A*S at k = --footprint-k (256) on 100 000 columns x 200 nonzeros whose rows are uniform over R rows:
    R KiB of gathered footprint, so the sweep shows what L1, L2, the Infinity Cache and HBM deliver."""
    from bidmat_amd import hip_abi
    from bidmat_amd.device import DeviceArray
    k, ncols, L = args.footprint_k, 100000, 200
    nnz = ncols * L
    rng = np.random.default_rng(0)
    stream = C.c_void_p()
    hip_abi.check(lib.bidmat_stream_create(C.byref(stream)))
    k_rows_max = 1 << 20                      # A holds 2^20 rows of 256 floats: fewer rows fit when k is larger
    d_A = DeviceArray.from_numpy(rng.random(256 * k_rows_max, dtype=np.float32))
    d_B = DeviceArray.from_numpy(rng.random(k * ncols, dtype=np.float32))
    d_v = DeviceArray.from_numpy(rng.random(nnz, dtype=np.float32))
    d_jc = DeviceArray.from_numpy((np.arange(ncols + 1) * L).astype(np.int32))
    d_P, d_C = DeviceArray(nnz, np.float32), DeviceArray(k * ncols, np.float32)
    rows = []
    for R in (16, 64, 256, 1024, 2048, 4096, 8192, 16384, 65536, 262144, 1048576):
        if R * k > k_rows_max * 256:
            break
        d_ir = DeviceArray.from_numpy(rng.integers(0, R, size=nnz).astype(np.int32))
        t_dds = _timed(lib, lambda: lib.bidmat_dds_csc(k, ncols, nnz, d_A.ptr, d_B.ptr, d_ir.ptr, d_jc.ptr, d_P.ptr, 0, stream), stream, 5)
        t_as = _timed(lib, lambda: lib.bidmat_dsmult_csc(k, ncols, nnz, d_A.ptr, d_v.ptr, d_ir.ptr, d_jc.ptr, d_C.ptr, 0, stream), stream, 5)
        b = nnz * (4 * k + 8)
        rows.append({"rows": R, "footprint_KiB": R * k * 4 // 1024, "dds_ms": round(t_dds, 3),
                     "dds_TBps": round(b / t_dds / 1e9, 2), "dsmult_ms": round(t_as, 3),
                     "dsmult_TBps": round(b / t_as / 1e9, 2)})
        d_ir.free()
    print(json.dumps({"metric": "gather throughput vs gathered footprint (algorithmic TB/s), k=%d, 20M nnz" % k,
                      "unit": "TB/s", "n_gpus": 1, "sweep": rows}))


def next_rows(lib, args):
    """The callers either side of the path, on the headline pattern (k = p = 256)."""
    import tempfile
    from bidmat_amd import gen, hip_abi, mats
    from bidmat_amd.device import DeviceArray
    cfg = gen.config("HEAD", args.scale)
    k, nrows, ncols = cfg["k"], cfg["nrows"], cfg["ncols"]
    ir, jc, vals = cfg["ir"], cfg["jc"], cfg["vals"]
    nnz = int(ir.size)
    stream = None            # these entries are the blocking, reference-shaped ones or take the default stream
    d_ir, d_jc, d_v = DeviceArray.from_numpy(ir), DeviceArray.from_numpy(jc), DeviceArray.from_numpy(vals)
    d_ic = DeviceArray(nnz, np.int32)
    hip_abi.check(lib.bidmat_csc_expand_cols(ncols, nnz, d_jc.ptr, d_ic.ptr, None))
    d_A, d_AT = DeviceArray.from_numpy(cfg["A"]), DeviceArray.from_numpy(cfg["A_T"])
    d_C, d_G = DeviceArray(k * ncols, np.float32), DeviceArray(k * nrows, np.float32)
    hip_abi.check(lib.bidmat_memset(d_C.ptr, 0, d_C.nbytes))
    hip_abi.check(lib.bidmat_memset(d_G.ptr, 0, d_G.nbytes))
    out = {}
    reps = max(1, args.steps // 2)
    # tile products over the middle half of the rows and columns (reference-shaped, blocking)
    r0, nr_, c0, nc_ = nrows // 4, nrows // 2, ncols // 4, ncols // 2
    inside = int(np.count_nonzero((ir[jc[c0]:jc[c0 + nc_]] >= r0) & (ir[jc[c0]:jc[c0 + nc_]] < r0 + nr_)))
    t = _timed(lib, lambda: lib.bidmat_dsmultTile(k, nc_, nr_, nnz, d_A.ptr + 4 * k * r0, k, d_v.ptr, d_ir.ptr, d_ic.ptr,
                                                   r0, c0, d_C.ptr, k), stream, reps, 1)
    out["dsmultTile"] = {"ms": round(t, 3), "nnz_in_tile": inside, "GBps": round((inside * 4 * k + int(jc[c0 + nc_] - jc[c0]) * 8 + nc_ * 4 * k) / t / 1e6, 1)}
    t = _timed(lib, lambda: lib.bidmat_dsmultTileT(k, nr_, nc_, nnz, d_AT.ptr + 4 * k * c0, k, d_v.ptr, d_ir.ptr, d_ic.ptr,
                                                    r0, c0, d_G.ptr, k), stream, reps, 1)
    out["dsmultTileT"] = {"ms": round(t, 3), "nnz_in_tile": inside, "GBps": round((inside * 4 * k + nnz * 8 + nr_ * 4 * k) / t / 1e6, 1)}
    # S^T * A and S * A with p = 256 dense columns
    p = k
    plan = C.c_void_p()
    hip_abi.check(lib.bidmat_plan_create(nrows, ncols, nnz, d_ir.ptr, d_jc.ptr, p, C.byref(plan)))
    d_X = DeviceArray.from_numpy(gen.normal(nrows * p, 71))
    d_Y = DeviceArray(ncols * p, np.float32)
    t = _timed(lib, lambda: lib.bidmat_sdtmult_csc(nrows, ncols, nnz, p, d_v.ptr, d_ir.ptr, d_jc.ptr, d_X.ptr, nrows, d_Y.ptr, ncols, None), stream, reps, 1)
    b = alg_bytes("dsmult", p, nnz, nrows, ncols) + 8 * p * (nrows + ncols)
    out["SDTMult (S^T*A)"] = {"ms": round(t, 3), "GBps": round(b / t / 1e6, 1)}
    t = _timed(lib, lambda: lib.bidmat_sdmult_plan(plan, p, d_v.ptr, d_Y.ptr, ncols, d_X.ptr, nrows, None), stream, reps, 1)
    b = alg_bytes("dsmultT", p, nnz, nrows, ncols) + 8 * p * (nrows + ncols)
    out["SDMult (S*A)"] = {"ms": round(t, 3), "GBps": round(b / t / 1e6, 1)}
    # sparse op edge vectors (in place on a copy of the values)
    d_w = DeviceArray.from_numpy(vals)
    d_row, d_col = DeviceArray.from_numpy(gen.uniform(ncols, 72, 0.5, 1.5)), DeviceArray.from_numpy(gen.uniform(nrows, 73, 0.5, 1.5))
    t = _timed(lib, lambda: lib.bidmat_sdoprow(nrows, ncols, nnz, d_w.ptr, d_ic.ptr, d_row.ptr, ncols, 2), stream, reps, 1)
    out["sdoprow"] = {"ms": round(t, 3), "GBps": round(12.0 * nnz / t / 1e6, 1)}
    t = _timed(lib, lambda: lib.bidmat_sdopcol(nrows, ncols, nnz, d_w.ptr, d_ir.ptr, d_col.ptr, nrows, 2), stream, reps, 1)
    out["sdopcol"] = {"ms": round(t, 3), "GBps": round(12.0 * nnz / t / 1e6, 1)}
    # pattern utilities: transpose on the device, a column range as a matrix of its own, dense image skipped (too large)
    d_tv, d_tir, d_tjc = DeviceArray(nnz, np.float32), DeviceArray(nnz, np.int32), DeviceArray(nrows + 1, np.int32)
    t0 = time.perf_counter()
    for _ in range(3):
        hip_abi.check(lib.bidmat_csc_transpose(nrows, ncols, nnz, d_v.ptr, d_ir.ptr, d_jc.ptr, d_tv.ptr, d_tir.ptr, d_tjc.ptr))
    t = (time.perf_counter() - t0) / 3 * 1e3
    out["GSMat.t (device)"] = {"ms": round(t, 3), "Mnnz_per_s": round(nnz / t / 1e3, 1)}
    c1, c2 = ncols // 4, ncols // 2
    start, cnt = C.c_int(), C.c_int()
    hip_abi.check(lib.bidmat_csc_colslice_range(ncols, c1, c2, d_jc.ptr, C.byref(start), C.byref(cnt)))
    d_sjc, d_sic = DeviceArray(c2 - c1 + 1, np.int32), DeviceArray(cnt.value, np.int32)
    t = _timed(lib, lambda: lib.bidmat_csc_colslice(c1, c2, start.value, cnt.value, d_jc.ptr, d_ir.ptr, d_v.ptr, d_sjc.ptr,
                                                    d_tir.ptr, d_sic.ptr, d_tv.ptr, stream), stream, reps, 1)
    out["colslice (quarter of the columns)"] = {"ms": round(t, 3), "GBps": round(20.0 * cnt.value / t / 1e6, 1)}
    # file -> device (pinned, double-buffered) against host arrays -> device (pageable copies)
    with tempfile.TemporaryDirectory() as tmp:
        f = os.path.join(tmp, "pattern.smat")
        mats.saveSMat(f, nrows, ncols, vals, ir + 1, jc + 1)
        size = os.path.getsize(f)
        t0 = time.perf_counter()
        g = mats.loadGSMat(f)
        t_load = time.perf_counter() - t0
        ir1, jc1 = ir + 1, jc + 1                        # host arrays carry base 1, like a host SMat
        g2 = mats.GSMat.from_csc(nrows, ncols, vals, ir1, jc1)       # first call: staging buffers, kernel loading
        t0 = time.perf_counter()
        g2 = mats.GSMat.from_csc(nrows, ncols, vals, ir1, jc1)
        t_from = time.perf_counter() - t0
        t0 = time.perf_counter()
        back = g2.to_csc()                               # incl. SparseMat.check on the host copy
        t_to = time.perf_counter() - t0
        assert np.array_equal(back[1], ir1) and np.array_equal(back[2], jc1) and np.array_equal(back[0], vals)
        out["loadGSMat"] = {"file_GB": round(size / 1e9, 3), "s": round(t_load, 3), "GBps": round(size / t_load / 1e9, 2)}
        out["GSMat.fromSMat"] = {"s": round(t_from, 3), "GBps": round(size / t_from / 1e9, 2)}
        out["GSMat.toSMat"] = {"s": round(t_to, 3), "GBps": round(size / t_to / 1e9, 2)}
        del g, g2
    print(json.dumps({"metric": "callers either side of the path on the headline pattern", "unit": "GB/s", "n_gpus": 1,
                      "config": {"k": k, "nrows": nrows, "ncols": ncols, "nnz": nnz, "scale": args.scale}, "ops": out}))


def cpu_baseline(workload, cfg, frac):
    """The CPU restatement of the reference's loops (oracle/, threads split as the reference
    splits them) on the first `frac` of the columns of the same workload, best of two runs."""
    import oracle
    k, nrows, ncols = cfg["k"], cfg["nrows"], cfg["ncols"]
    nc = max(1, int(ncols * frac))
    jc = cfg["jc"][: nc + 1].copy()
    nnz = int(jc[-1])
    ir = cfg["ir"][:nnz]
    vals = cfg["vals"][:nnz]
    threads = oracle.max_threads()

    def best(fn, reps=2):
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return min(ts)

    t = {}
    if workload == "headline":
        A, B, AT = cfg["A"], cfg["B"][: k * nc], cfg["A_T"][: k * nc]
        t["dds"] = best(lambda: oracle.dds(A, B, k, ir, jc, nthreads=threads))
        t["dsmult"] = best(lambda: oracle.fsmult(A, k, vals, ir, jc, nthreads=threads))
        t["dsmultT"] = best(lambda: oracle.fsmultT(AT, k, nrows, vals, ir, jc, nthreads=threads))
    elif workload in ("C1", "C4"):
        t["dsmult"] = best(lambda: oracle.fsmult(cfg["A"], k, vals, ir, jc, nthreads=threads))
    else:
        W, H = cfg["W"], cfg["H"][: k * nc]
        r, q = [None], [None]

        def dds():
            r[0] = oracle.dds(W, H, k, ir, jc, nthreads=threads)[0]

        def ew():
            q[0] = oracle.applyop(vals, r[0], 3)
        t["dds"] = best(dds, 1)
        t["ewise"] = best(ew, 1)
        t["dsmultT"] = best(lambda: oracle.fsmultT(H, k, nrows, q[0], ir, jc, nthreads=threads), 1)
    total_b = sum(alg_bytes(op, k, nnz, nrows, nc) for op in t)
    total_s = sum(t.values())
    return {
        "value": round(total_b / total_s / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": "first %d of %d columns (%d nnz) of the same workload, every op of the step, best of two "
                  "runs; A*^S uses min(cores, k/32) threads as the reference does" % (nc, ncols, nnz),
        "seconds": {op: round(s, 3) for op, s in t.items()},
        "nnz_per_s": round(len([o for o in t if o != "ewise"]) * nnz / total_s, 1),
    }


def _error_fields(x, ref64, sumabs):
    """Pure relative error and the path's error measure min(|x-ref|/|ref|, |x-ref|/sum|terms|) of a
    result against the fp64-accumulated CPU result, as maxima over all values."""
    x = np.asarray(x, dtype=np.float64)
    err = np.abs(x - ref64)
    with np.errstate(divide="ignore", invalid="ignore"):
        rel = np.where(err == 0, 0.0, err / np.abs(ref64))
        scaled = np.where(err == 0, 0.0, err / sumabs)
    rel = np.where(np.isnan(rel), np.inf, rel)
    measure = np.minimum(rel, np.where(np.isnan(scaled), np.inf, scaled))
    return {"max_rel_err": float(rel.max(initial=0.0)), "max_err_measure": float(measure.max(initial=0.0)),
            "checked_values": int(x.size)}


def _sub_csc(ir, jc, vals, cols):
    lens = jc[cols + 1] - jc[cols]
    sjc = np.zeros(cols.size + 1, dtype=np.int32)
    sjc[1:] = np.cumsum(lens)
    idx = np.concatenate([np.arange(jc[c], jc[c + 1]) for c in cols]) if cols.size else np.zeros(0, np.int64)
    return (vals[idx] if vals is not None else None), ir[idx], sjc, idx


def _rows_sub_csc(ir, jc, vals, rows, nrows):
    pos = np.full(nrows, -1, dtype=np.int64)
    pos[rows] = np.arange(rows.size)
    keep = np.flatnonzero(pos[ir] >= 0)
    ic = np.searchsorted(jc, keep, side="right") - 1
    sjc = np.zeros(jc.size, dtype=np.int32)
    sjc[1:] = np.cumsum(np.bincount(ic, minlength=jc.size - 1))
    return vals[keep], pos[ir[keep]].astype(np.int32), sjc


def verify_outputs(workload, cfg, results):
    """The outputs the timed steps left on the device against the CPU oracle's fp64-accumulated
    results: every value for the headline workload and configs[0]; for the 40 M / 400 M-nonzero
    workloads, whose full CPU results take minutes, all values of a random sample of columns (rows
    for A*^S). Returns per op: max_rel_err, max_err_measure, checked_values."""
    import oracle
    k, nrows, ncols = cfg["k"], cfg["nrows"], cfg["ncols"]
    ir, jc, vals = cfg["ir"], cfg["jc"], cfg["vals"]
    th = oracle.max_threads()
    out = {}
    rng = np.random.default_rng(0)
    if workload == "headline":
        ref, sa = oracle.dds_f64(cfg["A"], cfg["B"], k, ir, jc, nthreads=th)
        out["dds"] = _error_fields(results["dds"], ref, sa)
        ref, sa = oracle.fsmult_f64(cfg["A"], k, vals, ir, jc, nthreads=th)
        out["dsmult"] = _error_fields(results["dsmult"], ref, sa)
        ref, sa = oracle.fsmultT_f64(cfg["A_T"], k, nrows, vals, ir, jc, nthreads=th)
        out["dsmultT"] = _error_fields(results["dsmultT"], ref, sa)
    elif workload == "C1":
        ref, sa = oracle.fsmult_f64(cfg["A"], k, vals, ir, jc, nthreads=th)
        out["dsmult"] = _error_fields(results["dsmult"], ref, sa)
    elif workload == "C4":
        lens = np.diff(jc)
        cols = np.unique(np.concatenate([rng.integers(0, ncols, 2000), np.argsort(lens)[-5:], [0, ncols - 1]]))
        sv, sir, sjc, _ = _sub_csc(ir, jc, vals, cols)
        ref, sa = oracle.fsmult_f64(cfg["A"], k, sv, sir, sjc, nthreads=th)
        out["dsmult"] = _error_fields(results["dsmult"].reshape(ncols, k)[cols].ravel(), ref, sa)
        out["dsmult"]["checked"] = "%d sampled columns incl. the 5 longest" % cols.size
    else:   # C5: Q = V ./ DDS(W,H,V), G = H *^ Q
        W, H = cfg["W"], cfg["H"]
        Q, G = results["dds_op"], results["dsmultT"]
        cols = np.unique(rng.integers(0, ncols, 2000))
        sv, sir, sjc, idx = _sub_csc(ir, jc, vals, cols)
        r64, sa = oracle.dds_f64(W, H.reshape(ncols, k)[cols].ravel(), k, sir, sjc, nthreads=th)
        # all terms of R are positive: the error of Q = V/R relative to Q is the error of R relative to R
        want = sv.astype(np.float64) / r64
        out["dds_op"] = _error_fields(Q[idx], want, np.abs(want))
        out["dds_op"]["checked"] = "%d sampled columns" % cols.size
        rows = np.unique(np.concatenate([rng.integers(0, nrows, 500), [0, 1, nrows - 1]]))
        rv, rir, rjc = _rows_sub_csc(ir, jc, Q, rows, nrows)
        ref, sa = oracle.fsmultT_f64(H, k, rows.size, rv, rir, rjc, nthreads=th)
        out["dsmultT"] = _error_fields(G.reshape(nrows, k)[rows].ravel(), ref, sa)
        out["dsmultT"]["checked"] = "%d sampled rows, fed with the device's own Q" % rows.size
    return out


if __name__ == "__main__":
    main()
