#!/usr/bin/env python3
"""Benchmark of the CSR SpMV / SpMM / csr2csc path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the hot path (one mcsparseSpMV / mcsparseSpMM / mcsparseCsr2cscEx2 call
through the C ABI) over one synthetic operand set that is already resident in HBM.  Several
independent copies of all operands are rotated so the 256 MB Infinity Cache cannot hold a
matrix between steps.  The default workload is the configuration the metric is quoted on:
fp64 CSR SpMV, 1,048,576 rows x 16 nonzeros per row.  The last line of stdout is one compact JSON
object (about 2 KB) with the headline figures; the default invocation also measures the other
configurations (50 timed steps each, inside a wall-clock budget) and lists them under "others" of
that line as workload: [ms_per_step, roofline.frac].  The full object of every workload measured
goes to stderr, one JSON line each, and to bench_details.json in the results directory (see write_details).

Workloads: mixed (1 M rows of 16 and 64 rows of 100000, fp32), c1 (5-pt Laplacian 256^2 fp32), c2 (default), c3 / c3t (power-law fp32, op N / T),
c4-8 / c4-64 / c4-256 (27-pt stencil 128^3 SpMM, row-major B and C), c4-64-col (the same with
column-major B and C, the layout of csrmm2), c5 (csr2csc on the c3 matrix), c5-coo (csr2coo on it),
c5-spmv (A^T x from the converted CSC).  Probes: copy (a plain device copy, the yardstick of the
traffic counters), gather-probe (16.8 M random 8-byte reads through mcsparseDgthr: what the x[col]
reads of c2 cost on their own, from an 8 MB table and from one that fits every L2), stream-probe (the library's own
streaming kernels reading, writing and copying 1 GiB buffers: what the memory takes by itself; the default run holds
the headline against these rates as roofline.stream_ceiling_frac).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
RESULTS_DIR = "gpurun_out"  # where the full objects of a run are kept, when it exists

OTHERS = ["c4-64", "c3", "c3t", "c5", "c5-spmv", "c5-coo", "c4-8", "c4-256", "c4-64-col", "c1",
          "c2-alg2", "c3-alg2", "c3t-alg2", "c2-direct", "c3-direct", "c3t-direct", "c4-64-direct", "mixed-direct"]
OTHERS_BUDGET_S = 200.0  # wall-clock budget of the default invocation for the workloads above
OTHER_STEPS = {"c5": 20}  # timed steps of the workloads above: 50 unless named here (a step of c5 takes milliseconds)
OTHERS_WITH_CPU = ("c4-64", "c3", "c3t", "c5")  # the OpenMP port is timed beside these (and beside the headline)
SPIN_UP_S = 0.03  # every workload runs its steps for this long before the warmup steps (see run_workload)


def measured_traffic():
    """{(workload, preprocess state): (bytes per step, file)} from the "traffic" lines of the counter summaries under
    profiles/: FETCH_SIZE and WRITE_SIZE counts of all kernels of one step, each scaled by what the same counter
    reads on a 1 GiB copy (2 KiB and 1 KiB per count, profiles/copy_kernel_counter_calibration.txt).  Constants
    taken from those summaries, not counters read during the run."""
    out = {}
    directory = os.path.join(ROOT, "profiles")
    if not os.path.isdir(directory):
        return out
    for name in sorted(os.listdir(directory)):
        if not name.endswith(".txt"):
            continue
        with open(os.path.join(directory, name)) as f:
            for line in f:
                parts = line.split()
                if len(parts) == 5 and parts[0] == "traffic" and parts[2].startswith("state="):
                    fetch = float(parts[3].split("=", 1)[1])
                    write = float(parts[4].split("=", 1)[1])
                    out[(parts[1], int(parts[2].split("=", 1)[1]))] = (int((fetch * 2 + write) * 1024),
                                                                        "profiles/" + name)
    return out


MEASURED_TRAFFIC = measured_traffic()


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=None)
    p.add_argument("--warmup", type=int, default=None)
    p.add_argument("--workload", default="c2")
    p.add_argument("--copies", type=int, default=None, help="independent operand sets rotated between steps")
    p.add_argument("--scale", type=float, default=1.0, help="shrink the workload (for dry runs); 1.0 = as specified")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-preprocess", action="store_true",
                   help="skip mcsparseSpMV_preprocess / mcsparseSpMM_preprocess (the reference has neither)")
    p.add_argument("--no-others", action="store_true", help="default invocation: measure the headline workload only")
    p.add_argument("--family", type=int, default=0, help="force the SpMV kernel family (1 vector, 2 merge)")
    p.add_argument("--lanes", type=int, default=0, help="force lanes per row of the vector family")
    p.add_argument("--band-bytes", type=int, default=0, help="band width of mcsparseSpMV_preprocess (0 = default)")
    p.add_argument("--alg2", action="store_true",
                   help="MCSPARSE_SPMV_CSR_ALG2 for the SpMV workloads (a name ending in -alg2 says the same): "
                        "preprocess builds the banded copy whose sums repeat bit for bit, instead of the "
                        "faster copy in column order that the default algorithm gets")
    p.add_argument("--cache", default=None, help="directory to keep generated matrices in between runs")
    return p.parse_args()


class Matrices:
    """Generated matrices, kept for the workloads that share one (c3, c3t, c5*)."""

    def __init__(self, wl, scale, cache):
        self.wl, self.s, self.cache, self.have = wl, scale, cache, {}

    def get(self, key):
        if key in self.have:
            return self.have[key]
        wl, s = self.wl, self.s
        if key == "laplacian":
            a = wl.laplacian_5pt(max(4, int(256 * s)), dtype=np.float32)
        elif key == "uniform":
            a = wl.uniform_rows(m=max(64, int((1 << 20) * s)), per_row=16, dtype=np.float64)
        elif key == "power_law":
            a = cached(self.cache, "power_law_%g" % s, lambda: wl.power_law(
                m=max(64, int((1 << 22) * s)), max_len=max(8, int(200000 * min(1.0, s * 4))), dtype=np.float32))
        elif key == "mixed":
            a = wl.mixed_rows(m=max(4096, int((1 << 20) * s)), long_len=max(64, int(100000 * min(1.0, s * 4))),
                              dtype=np.float32)
        elif key == "stencil":
            a = wl.stencil_27pt(max(4, int(round(128 * s ** (1 / 3)))), dtype=np.float32)
        else:
            raise KeyError(key)
        self.have = {key: a}  # one at a time: the power-law matrix alone is 1.4 GB on the host
        return a


def describe(name):
    """(matrix key, kind, op is T, dense columns, alpha, beta, description) of a workload."""
    if name.endswith("-alg2"):
        d = describe(name[:-5])
        return d[:6] + (d[6] + ", MCSPARSE_SPMV_CSR_ALG2 (reproducible bits)",)
    if name.endswith("-direct"):
        d = describe(name[:-7])
        return d[:6] + (d[6] + ", no preprocess call (the two calls the reference's API has)",)
    if name == "c1":
        return "laplacian", "spmv", False, 0, 1.0, 0.0, "fp32 CSR SpMV, 5-pt Laplacian 256x256"
    if name == "c2":
        return "uniform", "spmv", False, 0, 1.5, 0.5, "fp64 CSR SpMV, 1048576 rows x 16 nnz/row uniform"
    pl = "fp32 CSR SpMV, 4194304 rows power-law (Zipf 1.8, <=200000 nnz/row)"
    if name == "c3":
        return "power_law", "spmv", False, 0, 1.0, 0.0, pl
    if name == "c3t":
        return "power_law", "spmv", True, 0, 1.0, 0.0, pl + ", op T"
    if name == "c5":
        return "power_law", "csr2csc", False, 0, 1.0, 0.0, "csr2csc (values + structure) of the fp32 power-law matrix"
    if name == "c5-coo":
        return "power_law", "csr2coo", False, 0, 1.0, 0.0, "csr2coo of the power-law matrix"
    if name == "c5-spmv":
        return ("power_law", "spmv-csc", False, 0, 1.0, 0.0,
                "fp32 SpMV op T from the CSC produced by csr2csc (power-law matrix)")
    if name == "mixed":
        return ("mixed", "spmv", False, 0, 1.0, 0.0,
                "fp32 CSR SpMV, 1048576 rows x 16 nnz/row uniform + 64 rows of 100000")
    if name.startswith("c3-spmm-"):  # not among the others of the default run
        return ("power_law", "spmm", False, int(name.split("-")[2]), 1.0, 0.0,
                "fp32 CSR SpMM, the power-law matrix of c3, B and C row-major N=%d" % int(name.split("-")[2]))
    if name.startswith("c4-"):
        parts = name.split("-")
        n_cols = int(parts[1])
        col_major = len(parts) > 2 and parts[2] == "col"
        return ("stencil", "spmm-col" if col_major else "spmm", False, n_cols, 1.0, 0.0,
                "fp32 CSR SpMM, 27-pt stencil 128^3, B and C %s N=%d" % ("column-major" if col_major else "row-major",
                                                                      n_cols))
    raise KeyError(name)


def run_workload(name, args, ctx, steps=None, warmup=None, with_cpu=True):
    """Measures one workload; returns the JSON object of its line."""
    torch, api, wl, handle, stream = ctx["torch"], ctx["api"], ctx["wl"], ctx["handle"], ctx["stream"]
    key, kind, op_t, n_cols, alpha, beta, desc = describe(name)
    alg = api.SPMV_CSR_ALG2 if (args.alg2 or name.endswith("-alg2")) else api.SPMV_ALG_DEFAULT
    if args.alg2 and not name.endswith("-alg2") and kind in ("spmv", "spmv-csc"):
        desc += ", MCSPARSE_SPMV_CSR_ALG2 (reproducible bits)"
    a = ctx["matrices"].get(key)
    op = api.OP_T if op_t else api.OP_N
    s = args.scale

    def dev(v):
        return torch.from_numpy(np.ascontiguousarray(v)).cuda()

    dt = a.val.dtype
    vb = dt.itemsize
    ct = api.maca_type(dt)
    tdt = torch.float32 if vb == 4 else torch.float64
    if kind in ("spmv", "spmv-csc"):
        algo_bytes = wl.spmv_bytes(a, vb)
        flops = 2 * a.nnz
        extra_read = a.m * vb if beta != 0 else 0
    elif kind in ("spmm", "spmm-col"):
        algo_bytes = wl.spmm_bytes(a, n_cols, vb)
        flops = 2 * a.nnz * n_cols
        extra_read = 0
    elif kind == "csr2csc":
        algo_bytes = (a.m + 1) * 4 + (a.n + 1) * 4 + 2 * a.nnz * (4 + vb)
        flops, extra_read = 0, 0
    else:
        algo_bytes = (a.m + 1) * 4 + 4 * a.nnz
        flops, extra_read = 0, 0

    # enough copies that the rotated footprint exceeds the 256 MB Infinity Cache several times
    copies = args.copies or max(2, min(8, int(np.ceil(1.2e9 / max(algo_bytes, 1)))))
    if algo_bytes > 8e8:
        copies = args.copies or 2
    if steps is None:
        steps = args.steps if args.steps is not None else (200 if algo_bytes < 6e8 else 40)
    if warmup is None:
        warmup = args.warmup if args.warmup is not None else (20 if algo_bytes < 6e8 else 5)

    rng = np.random.default_rng(12345)
    sets = []
    preprocess_ms = []

    def timed(call, what):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        api.check(call(), what)
        torch.cuda.synchronize()
        preprocess_ms.append((time.perf_counter() - t0) * 1e3)

    def spmv_buffer(st, the_op, fmt_is_csr):
        """Scratch of an SpMV set: with preprocessing, the larger buffer the banded copy lives in."""
        use_pre = not args.no_preprocess and not name.endswith("-direct") and not (args.family or args.lanes)
        if use_pre:
            rc, size = api.spmv_preprocess_buffer_size(handle, the_op, alpha, st["mat"], st["vx"], beta, st["vy"], ct,
                                                       alg=alg)
        else:
            rc, size = api.spmv_buffer_size(handle, the_op, alpha, st["mat"], st["vx"], beta, st["vy"], ct)
        api.check(rc, "mcsparseSpMV_bufferSize")
        st["buf"] = torch.empty(size, dtype=torch.uint8, device="cuda")
        if use_pre:
            timed(lambda: api.spmv_preprocess(handle, the_op, alpha, st["mat"], st["vx"], beta, st["vy"], ct, st["buf"],
                                              alg=alg),
                  "mcsparseSpMV_preprocess")

    for c in range(copies):
        st = {"ptr": dev(a.ptr), "col": dev(a.col), "val": dev(a.val)}
        if kind == "spmv":
            xs, ys = (a.n, a.m) if op == api.OP_N else (a.m, a.n)
            st["x"] = dev(rng.uniform(-1, 1, xs).astype(dt))
            st["y"] = dev(rng.uniform(-1, 1, ys).astype(dt))
            st["mat"] = api.SpMat(a.m, a.n, a.nnz, st["ptr"], st["col"], st["val"], base=a.base)
            if args.family or args.lanes:
                st["mat"].set_plan(args.family, args.lanes)
            if args.band_bytes:
                st["mat"].set_band_bytes(args.band_bytes)
            st["vx"], st["vy"] = api.DnVec(st["x"]), api.DnVec(st["y"])
            spmv_buffer(st, op, True)
        elif kind in ("spmm", "spmm-col"):
            row_major = kind == "spmm"
            order = api.ORDER_ROW if row_major else api.ORDER_COL
            shape_b, shape_c = ((a.n, n_cols), (a.m, n_cols)) if row_major else ((n_cols, a.n), (n_cols, a.m))
            st["B"] = dev(rng.uniform(-1, 1, shape_b).astype(dt))
            st["C"] = torch.zeros(shape_c, dtype=tdt, device="cuda")
            st["mat"] = api.SpMat(a.m, a.n, a.nnz, st["ptr"], st["col"], st["val"], base=a.base)
            st["mB"] = api.DnMat(a.n, n_cols, n_cols if row_major else a.n, st["B"], order=order)
            st["mC"] = api.DnMat(a.m, n_cols, n_cols if row_major else a.m, st["C"], order=order)
            rc, size = api.spmm_buffer_size(handle, api.OP_N, api.OP_N, alpha, st["mat"], st["mB"], beta, st["mC"], ct)
            api.check(rc, "mcsparseSpMM_bufferSize")
            st["buf"] = torch.empty(size, dtype=torch.uint8, device="cuda")
            if not args.no_preprocess and not name.endswith("-direct"):
                timed(lambda: api.spmm_preprocess(handle, api.OP_N, api.OP_N, alpha, st["mat"], st["mB"], beta,
                                                  st["mC"], ct, st["buf"]), "mcsparseSpMM_preprocess")
        elif kind in ("csr2csc", "spmv-csc"):
            st["o_val"] = torch.zeros(a.nnz, dtype=tdt, device="cuda")
            st["o_ptr"] = torch.zeros(a.n + 1, dtype=torch.int32, device="cuda")
            st["o_row"] = torch.zeros(a.nnz, dtype=torch.int32, device="cuda")
            rc, size = api.csr2csc_buffer_size(handle, a.m, a.n, a.nnz, st["val"], st["ptr"], st["col"], st["o_val"],
                                               st["o_ptr"], st["o_row"], ct, api.ACTION_NUMERIC, a.base)
            api.check(rc, "mcsparseCsr2cscEx2_bufferSize")
            st["buf"] = torch.empty(size, dtype=torch.uint8, device="cuda")
            if kind == "spmv-csc":
                api.check(api.csr2csc(handle, a.m, a.n, a.nnz, st["val"], st["ptr"], st["col"], st["o_val"],
                                      st["o_ptr"], st["o_row"], ct, api.ACTION_NUMERIC, a.base, st["buf"]))
                torch.cuda.synchronize()
                del st["buf"], st["ptr"], st["col"], st["val"]
                st["x"] = dev(rng.uniform(-1, 1, a.m).astype(dt))
                st["y"] = dev(rng.uniform(-1, 1, a.n).astype(dt))
                st["mat"] = api.SpMat(a.m, a.n, a.nnz, st["o_ptr"], st["o_row"], st["o_val"], base=a.base,
                                      fmt=api.FORMAT_CSC)
                if args.family or args.lanes:
                    st["mat"].set_plan(args.family, args.lanes)
                if args.band_bytes:
                    st["mat"].set_band_bytes(args.band_bytes)
                st["vx"], st["vy"] = api.DnVec(st["x"]), api.DnVec(st["y"])
                spmv_buffer(st, api.OP_T, False)
        else:
            st["coo"] = torch.zeros(a.nnz, dtype=torch.int32, device="cuda")
        sets.append(st)

    def step(i):
        st = sets[i % copies]
        if kind == "spmv":
            rc = api.spmv(handle, op, alpha, st["mat"], st["vx"], beta, st["vy"], ct, st["buf"], alg=alg)
        elif kind == "spmv-csc":
            rc = api.spmv(handle, api.OP_T, alpha, st["mat"], st["vx"], beta, st["vy"], ct, st["buf"], alg=alg)
        elif kind in ("spmm", "spmm-col"):
            rc = api.spmm(handle, api.OP_N, api.OP_N, alpha, st["mat"], st["mB"], beta, st["mC"], ct, st["buf"])
        elif kind == "csr2csc":
            rc = api.csr2csc(handle, a.m, a.n, a.nnz, st["val"], st["ptr"], st["col"], st["o_val"], st["o_ptr"],
                             st["o_row"], ct, api.ACTION_NUMERIC, a.base, st["buf"])
        else:
            rc = api.xcsr2coo(handle, st["ptr"], a.nnz, a.m, st["coo"], a.base)
        if rc != 0:
            raise api.McsparseError(rc, "step")

    # the first call on a structure (row-length analysis of a descriptor that has no plan yet)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(copies):
        step(i)
    torch.cuda.synchronize()
    first_pass_ms = (time.perf_counter() - t0) * 1e3 / copies

    # A device that has been idle runs its first 10 to 20 ms of work slower (the clocks come up, the page
    # tables of the rotated operand copies fill): SpMM with 64 columns 0.55 ms per step straight after 3
    # warmup steps and 0.50 ms from the 30th step on.  The steps are therefore repeated for SPIN_UP_S before
    # the warmup steps proper; the count goes into the output line.
    spin_up_steps = 0
    t_spin = time.perf_counter()
    while time.perf_counter() - t_spin < SPIN_UP_S:
        for i in range(max(copies, 4)):
            step(spin_up_steps + i)
        spin_up_steps += max(copies, 4)
        torch.cuda.synchronize()

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()

    # The timed region: exactly `steps` steps between two synchronisations, with one HIP event at each end
    # and none inside (an event record is a packet of its own on the stream: a pair around every step costs
    # about 5 us per step, which is 6 % of a step of the headline workload).
    region = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    region[0].record(stream)
    for i in range(steps):
        step(i)
    region[1].record(stream)
    torch.cuda.synchronize()
    wall_s = time.perf_counter() - t0
    ms_per_step = wall_s * 1e3 / steps
    region_ms = region[0].elapsed_time(region[1]) / steps
    # The same steps once more with an event pair around each, for the spread between steps (the pairs
    # themselves keep a step's first kernel from starting under the last one's tail: about 2 us per step).
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for i in range(steps):
        ev[i][0].record(stream)
        step(i)
        ev[i][1].record(stream)
    torch.cuda.synchronize()
    dev_ms = np.array([e0.elapsed_time(e1) for e0, e1 in ev])
    dev_avg_ms = float(dev_ms.mean())

    value = algo_bytes / (ms_per_step * 1e-3) / 1e9
    achieved = algo_bytes / (region_ms * 1e-3) / 1e9
    mat0 = sets[0].get("mat")
    plan = mat0.plan() if mat0 is not None and kind in ("spmv", "spmv-csc") else None
    banded = mat0.spmv_preprocess_state() if mat0 is not None and kind in ("spmv", "spmv-csc") else None
    copy_state = banded[0] if banded and banded[0] in (2, 3) else 0
    base_name = name[:-5] if name.endswith("-alg2") else name[:-7] if name.endswith("-direct") else name
    traffic = MEASURED_TRAFFIC.get((base_name, copy_state)) if s == 1.0 else None
    if name.endswith("-direct") and kind.startswith("spmm"):
        traffic = None  # the counters on file are those of the scheduled kernel

    out = {
        "metric": "CSR SpMV/SpMM achieved HBM GB/s (% of MI355X peak) + GFLOP/s at 1 GPU",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "spin_up_steps_before_warmup": spin_up_steps,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64" if vb == 8 else "f32",
        "data": "synthetic",
        "config": {"workload": "%s: %s" % (name, desc), "rows": a.m, "cols": a.n, "nnz": a.nnz,
                   "dense_cols": n_cols, "alpha": alpha, "beta": beta, "operand_copies_rotated": copies,
                   "max_row_nnz": int(a.row_lengths().max()), "scale": s},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "gflops": round(flops / (ms_per_step * 1e-3) / 1e9, 2),
        "algorithmic_bytes_per_step": int(algo_bytes),
        "extra_bytes_not_counted": int(extra_read),
        "first_call_ms": round(first_pass_ms, 4),
        "preprocess_ms": round(min(preprocess_ms), 4) if preprocess_ms else None,
        "device_ms_per_step": {"mean": round(dev_avg_ms, 5), "median": round(float(np.median(dev_ms)), 5),
                               "min": round(float(dev_ms.min()), 5),
                               "timed_region_mean": round(region_ms, 5),
                               "how": "timed_region_mean (what roofline.achieved uses): two HIP events around the "
                                      "timed region / steps; mean, median, min: event pairs around every step in a "
                                      "second pass of the same steps"},
        "spmv_plan": {"family": plan[0], "lanes_per_row": plan[1]} if plan else None,
        "spmv_preprocess": {"state": banded[0], "bands": banded[1], "rows_per_tile": banded[2]} if banded else None,
        "spmm_schedule": mat0.spmm_schedule()[0] if mat0 is not None and kind.startswith("spmm") else None,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": traffic[0] if traffic else None,
                     "traffic_source": ("constant from " + traffic[1]) if traffic else None},
    }
    del sets
    torch.cuda.empty_cache()
    if with_cpu and not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(kind, a, alpha, beta, n_cols, algo_bytes, op_t)
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (got --gpus %d)" % args.gpus,
              file=sys.stderr)
        return 2

    import torch
    from mcsparse_amd import api
    from mcsparse_amd import workloads as wl

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream()
    handle = api.Handle(stream=stream.cuda_stream)
    name = args.workload
    if name == "copy":
        # plain device copy of known size: the yardstick the rocprofv3 FETCH_SIZE / WRITE_SIZE
        # counters are scaled by
        return copy_probe(torch, args)
    if name == "gather-probe":
        return gather_probe(torch, api, handle, args)
    if name == "stream-probe":
        print(json.dumps(stream_probe(torch, api, handle, stream, steps=args.steps or 40)))
        return 0
    try:
        describe(name)
    except (KeyError, ValueError, IndexError):
        print("unknown workload %r" % name, file=sys.stderr)
        return 2

    ctx = {"torch": torch, "api": api, "wl": wl, "handle": handle, "stream": stream,
           "matrices": Matrices(wl, args.scale, args.cache)}
    t_start = time.perf_counter()
    out = run_workload(name, args, ctx)

    # A run of the headline workload (with or without --steps / --warmup, which apply to it alone) also measures
    # the other configurations, each with fewer steps, while the wall-clock budget lasts; what does not fit is named
    # under "others_skipped".  --no-others, or any flag that changes how the headline runs, leaves them out.
    default_run = (name == "c2" and not args.no_others and not args.no_preprocess and not args.alg2 and
                   not args.no_cpu_baseline and args.scale == 1.0 and
                   not (args.family or args.lanes or args.band_bytes or args.copies))
    details = [out]
    if default_run or name == "c2":
        # The same bytes at the rates the memory gives streaming kernels of this library (measured in this run): what
        # a kernel that only streamed its algorithmic bytes, reads at the read rate and writes at the write rate,
        # would reach, and the headline as a fraction of that.
        probe = stream_probe(torch, api, handle, stream, steps=20)
        details.append(probe)
        a_bytes = out["algorithmic_bytes_per_step"]
        writes = out["config"]["rows"] * (8 if out["dtype"] == "f64" else 4)
        floor_ms = ((a_bytes - writes) / probe["read_GBps"] + writes / probe["write_GBps"]) / 1e6
        out["roofline"]["stream_ceiling"] = {"read_GBps": probe["read_GBps"], "write_GBps": probe["write_GBps"],
                                             "copy_GBps": probe["copy_GBps"],
                                             "algorithmic_bytes_at_these_rates_ms": round(floor_ms, 5)}
        out["roofline"]["stream_ceiling_frac"] = round(floor_ms / (a_bytes / out["roofline"]["achieved"] / 1e6), 4)
    if default_run:
        others, skipped = {}, []
        for w in OTHERS:
            if time.perf_counter() - t_start > OTHERS_BUDGET_S:
                skipped.append(w)
                continue
            r = run_workload(w, args, ctx, steps=OTHER_STEPS.get(w, 50), warmup=5, with_cpu=w in OTHERS_WITH_CPU)
            details.append(r)
            others[w] = [r["ms_per_step"], r["roofline"]["frac"]]
        out["others"] = others
        out["others_are"] = "workload: [ms_per_step, roofline.frac]"
        out["others_skipped"] = skipped
    write_details(details)
    print(compact_line(out))
    return 0


HEADLINE_KEYS = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                 "vs_baseline", "dtype", "data", "config", "pct_of_hbm_peak", "gflops", "algorithmic_bytes_per_step",
                 "preprocess_ms", "roofline", "cpu_baseline", "others", "others_are", "others_skipped")


def compact_line(out):
    """The one JSON line a run ends with: the headline keys only, short enough (about 2 KB) that a reader who keeps
    the last few KB of the output still has all of it.  Everything else a workload measured goes to write_details."""
    line = {k: out[k] for k in HEADLINE_KEYS if k in out}
    return json.dumps(line, separators=(",", ":"))


def write_details(objects):
    """Every workload's full object: one JSON line each on stderr, and the list as bench_details.json in the
    directory named by BENCH_DETAILS_DIR (default: RESULTS_DIR beside this script, when it exists)."""
    for o in objects:
        print(json.dumps(o), file=sys.stderr)
    directory = os.environ.get("BENCH_DETAILS_DIR") or os.path.join(ROOT, RESULTS_DIR)
    if os.path.isdir(directory):
        try:
            with open(os.path.join(directory, "bench_details.json"), "w") as f:
                json.dump(objects, f, indent=1)
        except OSError:
            pass


def stream_probe(torch, api, handle, stream, steps=40, gib=1):
    """What the memory takes by itself: the library's own streaming kernels (mcsparseXstreamProbe: a contiguous
    16 KB per workgroup, four 16-byte accesses per thread) reading, writing and copying buffers of 1 GiB, rotated over
    four so that the 256 MB Infinity Cache holds none of them.  GB/s per mode, between two events on the stream."""
    nbytes = gib << 30
    bufs = [torch.empty(nbytes, dtype=torch.uint8, device="cuda") for _ in range(4)]
    for b in bufs:
        b.fill_(1)
    sink = torch.zeros(1 << 20, dtype=torch.int32, device="cuda")
    out = {"workload": "stream-probe", "buffer_bytes": nbytes, "buffers_rotated": len(bufs), "steps": steps}

    def run(mode, i):
        src, dst = bufs[i % 4], bufs[(i + 1) % 4]
        api.check(api.stream_probe(handle, mode, src if mode != 1 else None, dst if mode != 0 else None, nbytes,
                                   sink if mode == 0 else None), "mcsparseXstreamProbe")

    for mode, name, moved in ((0, "read", nbytes), (1, "write", nbytes), (2, "copy", 2 * nbytes)):
        for i in range(8):
            run(mode, i)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(steps):
            run(mode, i)
        e1.record(stream)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        out[name + "_GBps"] = round(moved / ms / 1e6, 1)
        out[name + "_ms"] = round(ms, 4)
    del bufs
    torch.cuda.empty_cache()
    return out


def copy_probe(torch, args):
    n = 1 << 28  # 1 GiB of fp32 read, 1 GiB written per step
    src = torch.ones(n, dtype=torch.float32, device="cuda")
    dst = torch.zeros(n, dtype=torch.float32, device="cuda")
    steps = args.steps or 10
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        dst.copy_(src)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    print(json.dumps({"workload": "copy", "bytes_read_per_step": 4 * n, "bytes_written_per_step": 4 * n,
                      "steps": steps, "ms_per_step": round(ms, 4), "GBps": round(8 * n / ms / 1e6, 1)}))
    return 0


def gather_probe(torch, api, handle, args):
    """x_val[i] = y[x_ind[i]] for as many uniformly random indices as c2 has nonzeros, from a table
    the size of c2's x, from one band of the banded layout (2 MiB) and from one that fits every L2:
    the cost of the gathers of a random-column SpMV with everything else (row offsets, values, sums)
    taken away.  mcsparseDgthr runs eight independent gathers per thread, like the SpMV kernels.
    Second part: the same gathers from the 2 MiB table with the indices sorted inside blocks, so that
    a block holds 1, 4, 16 indices per 128-byte line (what sorting a tile by column does to an SpMV)."""
    count = 1 << 24
    steps = args.steps or 20
    rng = np.random.default_rng(7)
    out = {"workload": "gather-probe", "gathers": count, "element_bytes": 8, "steps": steps, "tables": [],
           "sorted_blocks": []}
    stream = torch.cuda.current_stream()

    def measure(ind_host, table_elems):
        ind = torch.from_numpy(ind_host).cuda()
        table = torch.rand(table_elems, dtype=torch.float64, device="cuda")
        dst = torch.zeros(count, dtype=torch.float64, device="cuda")
        for _ in range(3):
            api.check(api.gthr(handle, count, table, dst, ind, 0))
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(steps):
            api.check(api.gthr(handle, count, table, dst, ind, 0))
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / steps

    for table_elems in (1 << 17, 1 << 18, 1 << 20):
        us = measure(rng.integers(0, table_elems, count, dtype=np.int32), table_elems)
        out["tables"].append({"table_MB": table_elems * 8 / 1e6, "us_per_call": round(us, 1),
                              "gathers_per_us": round(count / us, 1),
                              "streamed_bytes_per_call": count * (4 + 8)})
    table_elems = 1 << 18
    ind = rng.integers(0, table_elems, count, dtype=np.int32)
    for block in (1 << 14, 1 << 16, 1 << 18, count):
        us = measure(np.sort(ind.reshape(-1, block), axis=1).reshape(-1), table_elems)
        out["sorted_blocks"].append({"table_MB": table_elems * 8 / 1e6, "block": block,
                                     "indices_per_line": block * 16 / table_elems, "us_per_call": round(us, 1)})
    print(json.dumps(out))
    return 0


def cached(directory, key, make):
    """Generated matrices are deterministic; keeping them on disk only saves generation time."""
    from mcsparse_amd import workloads as wl
    if not directory:
        return make()
    path = os.path.join(directory, key + ".npz")
    if os.path.exists(path):
        with np.load(path) as z:
            return wl.Csr(int(z["m"]), int(z["n"]), z["ptr"], z["col"], z["val"], int(z["base"]))
    a = make()
    os.makedirs(directory, exist_ok=True)
    np.savez(path, m=a.m, n=a.n, ptr=a.ptr, col=a.col, val=a.val, base=a.base)
    return a


def host_cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(kind, a, alpha, beta, n_cols, algo_bytes, op_t):
    """Times the oracle's OpenMP port of the same semantics on the host cores (reported only).

    The port is compiled for the host it runs on (-march=native) when a compiler is at hand, and
    the operands are copied into pages that the OpenMP threads touch first, with the schedule of
    the compute loops."""
    import oracle
    tuned = oracle.use_native_build()
    threads = oracle.max_threads()
    rng = np.random.default_rng(1)
    dt = a.val.dtype
    ft = oracle.first_touch_copy
    ptr, col, val = ft(a.ptr), ft(a.col), ft(a.val)
    if kind == "spmv" and not op_t:
        x = ft(rng.uniform(-1, 1, a.n).astype(dt))
        y = ft(rng.uniform(-1, 1, a.m).astype(dt))
        dyn = int(a.row_lengths().max()) > 4096

        def run():
            oracle.spmv_omp(a.m, a.base, ptr, col, val, alpha, beta, x, y, dynamic=dyn)
        sample = "whole workload per repetition"
    elif kind == "spmv":
        # op T as the reference does it: transpose on every call, then the row loop
        x = ft(rng.uniform(-1, 1, a.m).astype(dt))
        y = ft(rng.uniform(-1, 1, a.n).astype(dt))

        def run():
            cp, ri, cv = oracle.csr2csc(a.m, a.n, a.base, ptr, col, val, method="omp")
            oracle.spmv_omp(a.n, a.base, cp, ri, cv, alpha, beta, x, y, dynamic=True)
        sample = "whole workload per repetition (csr2csc + row loop over the transpose)"
    elif kind == "spmv-csc":
        cp, ri, cv = oracle.csr2csc(a.m, a.n, a.base, ptr, col, val, method="omp")
        cp, ri, cv = ft(cp), ft(ri), ft(cv)
        x = ft(rng.uniform(-1, 1, a.m).astype(dt))
        y = ft(rng.uniform(-1, 1, a.n).astype(dt))
        dyn = int(np.diff(cp.astype(np.int64)).max()) > 4096

        def run():
            oracle.spmv_omp(a.n, a.base, cp, ri, cv, alpha, beta, x, y, dynamic=dyn)
        sample = "whole workload per repetition (row loop over the transposed matrix)"
    elif kind == "csr2csc":
        def run():
            oracle.csr2csc(a.m, a.n, a.base, ptr, col, val, method="omp")
        sample = "whole workload per repetition (per-thread column counts, scan, stable placement)"
    elif kind == "csr2coo":
        def run():
            oracle.csr2coo_omp(a.m, a.base, ptr, a.nnz)
        sample = "whole workload per repetition"
    elif kind == "spmm":
        B = ft(rng.uniform(-1, 1, (a.n, n_cols)).astype(dt))
        C = ft(np.zeros((a.m, n_cols), dtype=dt))

        def run():
            oracle.spmm_omp_f32(a.m, n_cols, a.base, ptr, col, val, alpha, beta, B, C)
        sample = "whole workload per repetition"
    else:
        return {"value": None, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": "no OpenMP port of this workload"}
    for _ in range(2):
        run()
    times = []
    t_end = time.perf_counter() + 8.0
    while len(times) < 10 and (time.perf_counter() < t_end or len(times) < 3):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {"value": round(algo_bytes / med / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "host_cpu": host_cpu_model(), "build": "-O3 -march=native" if tuned else "-O3 -march=x86-64-v3",
            "sample": "%s; median of %d (%.3f ms); operands first touched by the OpenMP threads" % (
                sample, len(times), med * 1e3)}


if __name__ == "__main__":
    sys.exit(main())
