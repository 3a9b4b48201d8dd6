#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: hyb SpMM (fp32, feature width 128) on a seeded
synthetic power-law graph with 2,449,029 nodes and ~61.9M edges, the configuration the
headline metric is quoted on.

  python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one launch of the fused hyb SpMM kernel over the whole graph (all ELL buckets of
all column partitions), inputs resident in HBM.  Following the reference's time_evaluator
loop (examples/spmm/bench_spmm.py:229, src/runtime/profiling.cc:742-797) the output is not
re-zeroed between timed steps; correctness is checked on a separate first call.

Prints ONE JSON line.  `value` is GFLOP/s = 2*nnz*feat / wall time per step.  `roofline`
prices the same kernel against HBM bandwidth with the algorithmic byte count
8*nnz + 4*(m+1) + 4*n*feat + 4*m*feat (indices and values once, X once, Y once) and the
per-launch duration measured with HIP events on the launch stream.  `cpu_baseline` times the
C restatement of the reference's unscheduled CPU loop nest on one host core over a bounded
row sample of the same graph.  `extra` carries the same kernel on the graph with power-law
columns (its own roofline block), the CSR row-split comparator, SDDMM, BSR, RGMS, TC-SpMM and the
host format passes.  Small kernels are timed three ways: `us_per_call` (events around every call:
what a Python caller sees, launch overhead included), `us_back_to_back` (one event pair around a
run of calls) and `us_graph` (a captured HIP graph of 20 launches replayed: device time only,
the figure a rocprofv3 kernel trace shows).

Exit status 3 when a correctness check of the first call fails (the JSON line is still printed).
"""
import argparse
import ctypes
import glob
import hashlib
import json
import os
import re
import subprocess
import sys
import time

import numpy as np

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
ROOT = os.path.dirname(os.path.abspath(__file__))

# ---- bandwidth probes: a small library of this benchmark's own (bench_probes.hip), not part of
# the product library
PROBES_SRC = os.path.join(ROOT, "bench_probes.hip")
PROBES_LIB = os.path.join(ROOT, "libbench_probes.so")


def build_probes():
    cmd = [os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "-O3", "-std=c++17", "-fPIC", "-shared",
           "--offload-arch=gfx950", "-munsafe-fp-atomics", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-x", "hip", PROBES_SRC, "-o", PROBES_LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on bench_probes.hip:\n" + r.stdout + r.stderr)
    return PROBES_LIB


PROBE_SYMBOLS = ("bench_probe_copy", "bench_probe_gather", "bench_probe_atomic_rows", "bench_probe_mfma_f16",
                 "bench_probe_bsr_lds")


def load_probes():
    """The probe library, built first when it is missing, older than its source, or lacks a symbol
    this file binds (a checkout that kept a library from an older bench_probes.hip)."""
    stale = (not os.path.exists(PROBES_LIB)
             or os.path.getmtime(PROBES_LIB) < os.path.getmtime(PROBES_SRC))
    if not stale:
        have = ctypes.CDLL(PROBES_LIB)
        stale = not all(hasattr(have, name) for name in PROBE_SYMBOLS)
        del have
    if stale:
        build_probes()
    L = ctypes.CDLL(PROBES_LIB)
    VP, I64, I32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32
    L.bench_probe_copy.restype, L.bench_probe_copy.argtypes = I32, [VP, VP, I64, VP]
    L.bench_probe_gather.restype, L.bench_probe_gather.argtypes = I32, [VP, I64, I32, I64, VP, VP]
    L.bench_probe_atomic_rows.restype, L.bench_probe_atomic_rows.argtypes = I32, [VP, I64, I64, VP]
    L.bench_probe_mfma_f16.restype = I32
    L.bench_probe_mfma_f16.argtypes = [I32, I32, I32, VP, ctypes.POINTER(ctypes.c_double), VP]
    L.bench_probe_bsr_lds.restype, L.bench_probe_bsr_lds.argtypes = I32, [I32, VP, VP]
    return L


def measured_traffic(workload):
    """HBM-side bytes per launch of a kernel as measured with rocprofv3 --pmc (FETCH_SIZE,
    WRITE_SIZE, scaled by a plain copy of known size).  The summaries under profiles/ carry one
    line per measured workload,
        traffic-bytes-per-launch: workload=<signature> bytes=<float> kernel-source-sha1=<sha1> [kernel-source=<file>]
    where the sha1 is that of the kernel's source file under sparsetir_amd/csrc/ (spmm.hip when the
    line names none) when the counters were taken.  Returns (bytes, note); bytes is None when
    nothing was measured for this workload or the kernel source has changed since."""
    pat = re.compile(r"traffic-bytes-per-launch:\s+workload=(\S+)\s+bytes=(\S+)\s+kernel-source-sha1=(\w+)"
                     r"(?:\s+kernel-source=(\S+))?")
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.md"))):
        for line in open(path):
            mt = pat.search(line)
            if mt and mt.group(1) == workload:
                src = mt.group(4) or "spmm.hip"
                with open(os.path.join(ROOT, "sparsetir_amd", "csrc", src), "rb") as f:
                    now = hashlib.sha1(f.read()).hexdigest()
                if mt.group(3) != now:
                    return None, f"stale: {src} changed since {os.path.basename(path)} was taken"
                return float(mt.group(2)), os.path.basename(path)
    return None, "not measured for this workload"


def side_roofline(bound, achieved, tag):
    """The roofline block of a side kernel: `achieved` in TFLOP/s against the dense fp16 MFMA peak
    (bound "mfma") or in GB/s of algorithmic bytes against the HBM peak (bound "hbm"); traffic
    from the profile line of workload `tag`, if one exists for the kernel source as it is now."""
    peak = MFMA_F16_PEAK_TFLOPS if bound == "mfma" else HBM_PEAK_GBS
    traffic, note = measured_traffic(tag)
    return {"bound": bound, "achieved": achieved, "peak": peak, "unit": "TFLOP/s" if bound == "mfma" else "GB/s",
            "frac": achieved / peak, "traffic": traffic, "traffic_source": note}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--feat", type=int, default=128)
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the graph (testing only)")
    ap.add_argument("--columns", default="uniform", choices=["uniform", "symmetric"])
    ap.add_argument("--parts", type=int, default=None, help="column partitions")
    ap.add_argument("--buckets", type=str, default=None, help="comma separated ELL widths")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip CSR / SDDMM side measurements")
    ap.add_argument("--profile", action="store_true",
                    help="few launches per kernel and no graph replays: for runs under rocprofv3 --pmc, "
                         "which serialises and slows every launch")
    ap.add_argument("--lds-probes", action="store_true",
                    help="only launch the LDS access-class kernels of the BSR tile body (bench_probes.hip), for a "
                         "run under rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_ACTIVE_INST_LDS SQ_INSTS_LDS")
    ap.add_argument("--cpu-rows", type=int, default=10**9,
                    help="rows in the cpu_baseline sample (default: every row, about 6 s on one core)")
    return ap.parse_args()


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def time_steps(fn, steps, warmup, torch):
    """Wall time of `steps` launches bracketed by synchronize, plus the mean launch duration
    from HIP events recorded on the launch stream around each launch."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        fn()
        stops[i].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    dev_ms = [s.elapsed_time(e) for s, e in zip(starts, stops)]
    return wall, float(np.mean(dev_ms)) / 1e3, float(np.min(dev_ms)) / 1e3


PROFILE_RUN = False  # set by --profile


def time_small(fn, calls, warmup, torch, graph=True):
    """Three timings of a short kernel, in microseconds: events around every call (the median over
    the calls: a single call now and then waits tens of milliseconds for the host), one event pair
    around a run of calls (the median of three such runs), and a captured graph of 20 launches
    replayed (device time only)."""
    if PROFILE_RUN:
        calls, warmup, graph = 3, 1, False
    for _ in range(warmup):
        fn()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(calls)]
    for a, b in pairs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    per_call = float(np.median([a.elapsed_time(b) for a, b in pairs])) / 1e3
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    batches = []
    for _ in range(1 if PROFILE_RUN else 3):  # the median of three runs: clocks drift between neighbours
        e0.record()
        for _ in range(calls):
            fn()
        e1.record()
        e1.synchronize()
        batches.append(e0.elapsed_time(e1) * 1e3 / calls)
    out = {"us_per_call": per_call * 1e6, "us_back_to_back": sorted(batches)[len(batches) // 2]}
    if graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()  # plans are complete before capture begins
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(20):
                fn()
        g.replay()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(5):
            g.replay()
        e1.record()
        e1.synchronize()
        out["us_graph"] = e0.elapsed_time(e1) * 1e3 / 100
        del g
    else:
        out["us_graph"] = None
    return out




def config2_sweep(torch, dev, ops, st, datasets, time_steps):
    """Config 2: hyb SpMM (2 column partitions, widths 1..512) against CSR row-split on the
    169k-node graph, feature widths 32/64/128/256."""
    g = datasets.config2()
    m, n, nnz = g["m"], g["n"], len(g["indices"])
    parts, buckets = g["num_col_parts"], g["buckets"]
    d_ptr, d_idx = torch.from_numpy(g["indptr"]).to(dev), torch.from_numpy(g["indices"]).to(dev)
    rows, cols, mask = st.column_part_hyb(m, n, d_ptr, d_idx, parts, buckets)
    triples, nrows = [], []
    for p in range(parts):
        for b in range(len(buckets)):
            triples += [mask[p][b].reshape(-1).float(), rows[p][b], cols[p][b].reshape(-1)]
            nrows.append(int(rows[p][b].shape[0]))
    # ... and the decomposition format.suggest_decomposition gives for this GPU (one partition)
    sparts, sbuckets = st.suggest_decomposition(m, n, nnz, 128)
    srows, scols, smask = st.column_part_hyb(m, n, d_ptr, d_idx, sparts, sbuckets)
    striples, snrows = [], []
    for b in range(len(sbuckets)):
        striples += [smask[0][b].reshape(-1).float(), srows[0][b], scols[0][b].reshape(-1)]
        snrows.append(int(srows[0][b].shape[0]))
    ones = torch.ones(nnz, device=dev)
    out = {"nodes": m, "edges": nnz, "num_col_parts": parts,
           "suggested_decomposition": {"num_col_parts": sparts, "buckets": sbuckets}}
    for feat in (32, 64, 128, 256):
        x = torch.randn(n * feat, device=dev)
        c = torch.zeros(m * feat, device=dev)
        hyb = ops.build_hyb_csrmm(m, n, feat, parts, buckets, nrows)
        shyb = ops.build_hyb_csrmm(m, n, feat, sparts, sbuckets, snrows)
        csr = ops.build_csrmm(m, n, feat, nnz)
        reps = 3 if PROFILE_RUN else 50
        _, dh, _ = time_steps(lambda: hyb(x, c, *triples), reps, 2, torch)
        _, ds, _ = time_steps(lambda: shyb(x, c, *striples), reps, 2, torch)
        _, dc, _ = time_steps(lambda: csr(ones, x, c, d_ptr, d_idx), reps, 2, torch)
        byts = 8.0 * nnz + 4.0 * (m + 1) + 4.0 * n * feat + 4.0 * m * feat
        out[f"feat{feat}"] = {"hyb_us": dh * 1e6, "csr_us": dc * 1e6, "hyb_gflops": 2.0 * nnz * feat / dh / 1e9,
                              "hyb_alg_GBps": byts / dh / 1e9, "hyb_suggested_us": ds * 1e6,
                              "hyb_suggested_alg_GBps": byts / ds / 1e9,
                              "roofline": side_roofline("hbm", byts / dh / 1e9, f"config2/p{parts}/f{feat}")}
    if not PROFILE_RUN:
        # the same graph cut into 1 ... 16 column partitions (widths 1..512), as the plan runs them
        # (phases up to 4 partitions, rows merged across partitions above), at 128 and 256 features
        sweep = {}
        for sp in (1, 2, 4, 8, 16):
            prow, pcol, pmask = st.column_part_hyb(m, n, d_ptr, d_idx, sp, buckets)
            ptriples, pnrows, slots = [], [], 0
            for p in range(sp):
                for b in range(len(buckets)):
                    ptriples += [pmask[p][b].reshape(-1).float(), prow[p][b], pcol[p][b].reshape(-1)]
                    pnrows.append(int(prow[p][b].shape[0]))
                    slots += int(pcol[p][b].numel())
            entry = {"slots_per_edge": slots / nnz, "ell_rows_per_row": sum(pnrows) / m}
            for feat in (128, 256):
                x = torch.randn(n * feat, device=dev)
                c = torch.zeros(m * feat, device=dev)
                f = ops.build_hyb_csrmm(m, n, feat, sp, buckets, pnrows)
                _, dp, _ = time_steps(lambda: f(x, c, *ptriples), 50, 2, torch)
                entry[f"feat{feat}_us"] = dp * 1e6
            sweep[f"parts{sp}"] = entry
        out["partition_sweep"] = sweep
    return out


def side_kernels(torch, dev, ops, st, datasets, time_steps):
    """BSR SpMM (config 4 and scaled-up shapes), RGMS (config 5), TC-SpMM and the host format
    passes: time, flop rate against the dense fp16 MFMA peak, algorithmic bytes against the HBM
    peak.  Rates use the back-to-back time; see time_small for the three timings."""
    out = {}

    def bsr(tag, mb, nb, blk, density, feat, dtype, calls=100):
        cfg = datasets.config4(seed=3, mb=mb, nb=nb, blk=blk, density=density, feat=32)
        nnzb = len(cfg["indices"])
        a = torch.from_numpy(cfg["data"]).to(dev).to(dtype).reshape(-1)
        x = torch.randn(nb * blk * feat, device=dev).to(dtype)
        y = torch.zeros(mb * blk * feat, device=dev, dtype=dtype)
        ip, ix = torch.from_numpy(cfg["indptr"]).to(dev), torch.from_numpy(cfg["indices"]).to(dev)
        f = ops.build_bsrmm(mb, nb, nnzb, blk, feat, dtype)
        tm = time_small(lambda: f(a, x, y, ip, ix), calls, 5, torch)
        d = tm["us_back_to_back"] / 1e6
        flops = 2.0 * nnzb * blk * blk * feat
        byts = 2.0 * nnzb * blk * blk + 4 * nnzb + 4 * (mb + 1) + 2.0 * nb * blk * feat + 2.0 * mb * blk * feat
        out[tag] = dict(tm, us=d * 1e6, tflops=flops / d / 1e12,
                        frac_of_mfma_peak=flops / d / 1e12 / MFMA_F16_PEAK_TFLOPS, alg_GBps=byts / d / 1e9,
                        frac_of_hbm_peak=byts / d / 1e9 / HBM_PEAK_GBS, nnzb=nnzb, algorithmic_bytes=byts,
                        shape=[mb * blk, nb * blk, feat], blk=blk, dtype=str(dtype).split(".")[-1],
                        roofline=side_roofline("mfma", flops / d / 1e12, tag))

    bsr("bsr_config4_f16", 128, 128, 32, 0.10, 512, torch.float16)
    bsr("bsr_config4_bf16", 128, 128, 32, 0.10, 512, torch.bfloat16)
    # config 4's weight against 16 times the activation columns: X stays in L2, the launch is long
    bsr("bsr_config4_weight_f8192_f16", 128, 128, 32, 0.10, 8192, torch.float16, calls=50)
    bsr("bsr_16384x16384_f4096_f16", 512, 512, 32, 0.10, 4096, torch.float16, calls=20)
    bsr("bsr_16384x16384_blk64_f4096_f16", 256, 256, 64, 0.10, 4096, torch.float16, calls=20)
    bsr("bsr_16384x16384_blk128_f4096_f16", 128, 128, 128, 0.10, 4096, torch.float16, calls=20)
    # 16 x 16 blocks, the granularity of the reference's schedule (bsr_spmm.py:379-380): 16-row slices on 16x16x32
    bsr("bsr_16384x16384_blk16_f4096_f16", 1024, 1024, 16, 0.10, 4096, torch.float16, calls=10)

    cfg = datasets.config5()
    R, n, fin, fout = cfg["num_rels"], cfg["n"], cfg["feat_in"], cfg["feat_out"]
    buckets, group = cfg["buckets"], 256
    rb = [group // b for b in buckets]
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    E = len(cfg["indices1"])
    st.csf_to_ell3d(*csf, rb, buckets)  # first call: page faults of the output arrays
    t0 = time.perf_counter()
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rb, buckets)
    fmt_s = time.perf_counter() - t0
    slots5 = int(sum(c.size for c in cols))
    out["csf_to_ell3d_config5_host"] = {"ms": fmt_s * 1e3, "edges": E, "slots": slots5, "threads": 1,
                                        "alg_GBps": (8.0 * E + 4.0 * sum(r.size for r in rows) + 8.0 * slots5)
                                        / fmt_s / 1e9}
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    # the same pass on the GPU (CSF arrays resident): per call, allocations and the sizing round trip included
    d_csf = [t(a) for a in csf]
    dev_out = st.csf_to_ell3d(*d_csf, rb, buckets)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        dev_out = st.csf_to_ell3d(*d_csf, rb, buckets)
    torch.cuda.synchronize()
    dev_s = (time.perf_counter() - t0) / 5
    same = all(bool((a.cpu() == torch.from_numpy(b)).all()) for ga, gb in zip(dev_out, (ptr, rows, cols, mask))
               for a, b in zip(ga, gb))
    out["csf_to_ell3d_config5_device"] = {"ms": dev_s * 1e3, "equals_host_arrays": same,
                                          "alg_GBps": (8.0 * E + 4.0 * sum(r.size for r in rows) + 8.0 * slots5)
                                          / dev_s / 1e9}
    del dev_out, d_csf
    triples, mids = [], []
    for k in range(len(buckets)):
        triples += [t(mask[k].astype(np.float16).ravel()), t(rows[k].ravel()), t(cols[k].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[k]))))
    w = t(cfg["w"].astype(np.float16).ravel())
    x = t(cfg["x"].astype(np.float16).ravel())
    y = torch.zeros(n * fout, device=dev)
    flops = 2.0 * E * fin * fout + 2.0 * E * fout
    byts = 8.0 * E + 2.0 * n * fin + 2.0 * R * fin * fout + 4.0 * n * fout
    # "rgms_config5": the operator as the reference uses it -- its A_k is the 0/1 mask, written once,
    # which the plan is told (static_weights); "..._weights_may_change": the default plan, which
    # reads the weights at every launch and keeps the padding slots
    # (a throwaway plan first: the first index build of a process also loads the sort's code objects
    # and grows the allocator's pools, 11 ms that belong to no plan)
    ops.build_rgms(n, n, R, fin, fout, rb, buckets, [c.shape[0] for c in cols])(w, x, y, *triples, *mids)
    y.zero_()
    for tag, static in (("rgms_config5", True), ("rgms_config5_weights_may_change", False)):
        f = ops.build_rgms(n, n, R, fin, fout, rb, buckets, [c.shape[0] for c in cols], static_weights=static)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        f(w, x, y, *triples, *mids)   # the first launch of a plan builds its edge index
        torch.cuda.synchronize()
        first_s = time.perf_counter() - t0
        tm = time_small(lambda: f(w, x, y, *triples, *mids), 50, 3, torch)
        d = tm["us_back_to_back"] / 1e6
        out[tag] = dict(tm, us=d * 1e6, first_call_ms=first_s * 1e3, tflops=flops / d / 1e12,
                        alg_GBps=byts / d / 1e9, frac_of_hbm_peak=byts / d / 1e9 / HBM_PEAK_GBS, edges=E,
                        algorithmic_bytes=byts, roofline=side_roofline("mfma", flops / d / 1e12, tag),
                        ell_rows=int(sum(r.size for r in rows)), static_weights=static,
                        accumulation="32-row output tiles written once; tiles cut by a share boundary add with atomics")

    # an fp16 Y: the reference's operator built with dtype "float16" (bench_rgcn_tensorcore.py:564-607)
    f = ops.build_rgms(n, n, R, fin, fout, rb, buckets, [c.shape[0] for c in cols], static_weights=True,
                       out_dtype=torch.float16)
    y16 = torch.zeros(n * fout, device=dev, dtype=torch.float16)
    f(w, x, y16, *triples, *mids)
    tm = time_small(lambda: f(w, x, y16, *triples, *mids), 50, 3, torch)
    d = tm["us_back_to_back"] / 1e6
    out["rgms_config5_f16_out"] = dict(tm, us=d * 1e6, tflops=flops / d / 1e12, static_weights=True,
                                       algorithmic_bytes=byts - 2.0 * n * fout,
                                       roofline=side_roofline("mfma", flops / d / 1e12, "rgms_config5_f16_out"))
    del f, y16

    # The same layer with 130 relations (the reference's BGS and AM graphs have 200 to 270 with their
    # inverses): W is twice what the LDS of a compute unit holds, so the plan runs two ranges of
    # relations one after the other.  The ELL3D arrays come from the device format pass.
    cfg_r = datasets.config5(seed=5, num_rels=130)
    Rr = cfg_r["num_rels"]
    d_csf = [t(cfg_r[k]) for k in ("indptr0", "indices0", "indptr1", "indices1")]
    ptr_r, rows_r, cols_r, mask_r = st.csf_to_ell3d(*d_csf, rb, buckets)
    triples_r, mids_r = [], []
    rel_ids = torch.arange(Rr, dtype=torch.int32, device=dev)
    for k in range(len(buckets)):
        triples_r += [mask_r[k].reshape(-1).half(), rows_r[k].reshape(-1), cols_r[k].reshape(-1)]
        mids_r.append(torch.repeat_interleave(rel_ids, (ptr_r[k][1:] - ptr_r[k][:-1]).long()))
    w_r = t(cfg_r["w"].astype(np.float16).ravel())
    x_r = t(cfg_r["x"].astype(np.float16).ravel())
    f = ops.build_rgms(n, n, Rr, fin, fout, rb, buckets, [c.shape[0] for c in cols_r], static_weights=True)
    f(w_r, x_r, y, *triples_r, *mids_r)
    tm = time_small(lambda: f(w_r, x_r, y, *triples_r, *mids_r), 50, 3, torch)
    Er = int(cfg_r["indices1"].shape[0])
    tf_r = (2.0 * Er * fin * fout + 2.0 * Er * fout) / tm["us_back_to_back"] / 1e6
    out["rgms_130_relations"] = dict(tm, us=tm["us_back_to_back"], edges=Er, num_rels=Rr, static_weights=True,
                                     tflops=tf_r, launches_per_call=2,
                                     roofline=side_roofline("mfma", tf_r, "rgms_130_relations"))
    del d_csf, triples_r, mids_r, w_r, x_r, f

    # SpMM over the condensed format (t = 32, g = 16) on the config-2 graph, fp16 in, fp32 out
    g2 = datasets.config2()
    st.condense(g2["indptr"], g2["indices"], 32, 16)
    t0 = time.perf_counter()
    gptr, tiles, cmask = st.condense(g2["indptr"], g2["indices"], 32, 16)
    fmt_s = time.perf_counter() - t0
    out["condense_config2_host"] = {"ms": fmt_s * 1e3, "edges": int(len(g2["indices"])), "groups": int(tiles.shape[0]),
                                    "threads": 1}
    # the same pass on the GPU (CSR arrays resident): per call, allocations and the sizing round trip included
    d_ptr2, d_idx2 = t(g2["indptr"]), t(g2["indices"])
    dev_out = st.condense(d_ptr2, d_idx2, 32, 16)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        dev_out = st.condense(d_ptr2, d_idx2, 32, 16)
    torch.cuda.synchronize()
    dev_s = (time.perf_counter() - t0) / 5
    out["condense_config2_device"] = {
        "ms": dev_s * 1e3,
        "equals_host_arrays": all(bool((a.cpu() == torch.from_numpy(b)).all())
                                  for a, b in zip(dev_out, (gptr, tiles, cmask)))}
    del dev_out, d_ptr2, d_idx2
    mb2, nnzb2, f2 = len(gptr) - 1, tiles.shape[0], 128
    tc = ops.build_tcspmm(mb2, nnzb2, f2, 32, 16, g2["n"], torch.float32)
    a2, b2 = t(cmask.astype(np.float16).ravel()), torch.randn(g2["n"] * f2, device=dev).half()
    c2 = torch.zeros(mb2 * 32 * f2, device=dev)
    gp, ti = t(gptr), t(tiles.ravel())
    tc(a2, b2, c2, gp, ti)  # makes the operator's plan
    torch.cuda.synchronize()
    tm = time_small(lambda: tc(a2, b2, c2, gp, ti), 50, 5, torch)
    d = tm["us_back_to_back"] / 1e6
    nnz2 = len(g2["indices"])
    out["tcspmm_config2_feat128"] = {"us_per_call": tm["us_per_call"], "us_graph": tm["us_graph"], "us": d * 1e6, "useful_gflops": 2.0 * nnz2 * f2 / d / 1e9,
                                     "mfma_tflops": 2.0 * nnzb2 * 32 * 16 * f2 / d / 1e12, "groups": int(nnzb2),
                                     "mask_density": float(nnz2) / (nnzb2 * 32 * 16),
                                     "roofline": side_roofline("mfma", 2.0 * nnzb2 * 32 * 16 * f2 / d / 1e12,
                                                               "tcspmm_config2_feat128")}
    # the reference's own form of this operator writes fp16 (bench_tc_spmm.py: fp16 accumulator fragments)
    tc16 = ops.build_tcspmm(mb2, nnzb2, f2, 32, 16, g2["n"], torch.float16)
    c16 = torch.zeros(mb2 * 32 * f2, device=dev, dtype=torch.float16)
    t0 = time.perf_counter()
    tc16(a2, b2, c16, gp, ti)  # makes the operator's plan (the long row tiles, longest first, in pieces)
    torch.cuda.synchronize()
    first_ms = (time.perf_counter() - t0) * 1e3
    tm = time_small(lambda: tc16(a2, b2, c16, gp, ti), 50, 5, torch)
    out["tcspmm_config2_feat128_f16_out"] = {"us_per_call": tm["us_per_call"], "us_graph": tm["us_graph"],
                                             "us": tm["us_back_to_back"], "first_call_ms": first_ms,
                                             "useful_gflops": 2.0 * nnz2 * f2 / tm["us_back_to_back"] / 1e3,
                                             "plan": "made from the group counts at the first call",
                                             "roofline": side_roofline(
                                                 "mfma", 2.0 * nnzb2 * 32 * 16 * f2 / tm["us_back_to_back"] / 1e6,
                                                 "tcspmm_config2_feat128_f16_out")}
    # the tile sizes the reference condenses with (tile_size = mma_m: 8 by default, 16;
    # examples/spmm/bench_tc_spmm.py:584-585,670) beside 32, fp16 out, condensed on the GPU
    d_ptr2, d_idx2 = t(g2["indptr"]), t(g2["indices"])
    sizes = {}
    for tsz in (8, 16, 32):
        gptr_t, tiles_t, mask_t = st.condense(d_ptr2, d_idx2, tsz, 16)
        mb_t, nnzb_t = int(gptr_t.shape[0]) - 1, int(tiles_t.shape[0])
        f_t = ops.build_tcspmm(mb_t, nnzb_t, f2, tsz, 16, g2["n"], torch.float16)
        a_t, ti_t = mask_t.reshape(-1).half(), tiles_t.reshape(-1)
        c_t = torch.zeros(mb_t * tsz * f2, device=dev, dtype=torch.float16)
        f_t(a_t, b2, c_t, gptr_t, ti_t)
        tm = time_small(lambda: f_t(a_t, b2, c_t, gptr_t, ti_t), 50, 5, torch)
        us = tm["us_back_to_back"]
        # the matrix cores multiply 16-row operands for tiles of 8 rows
        mfma_tf = 2.0 * nnzb_t * max(tsz, 16) * 16 * f2 / us / 1e6
        sizes[f"tile{tsz}"] = {"us": us, "us_graph": tm["us_graph"], "row_tiles": mb_t, "groups": nnzb_t,
                               "mask_density": float(nnz2) / (nnzb_t * tsz * 16),
                               "useful_gflops": 2.0 * nnz2 * f2 / us / 1e3, "mfma_tflops": mfma_tf,
                               "roofline": side_roofline("mfma", mfma_tf, f"tcspmm_config2_tile{tsz}")}
        del f_t, a_t, ti_t, c_t, gptr_t, tiles_t, mask_t
    out["tcspmm_config2_tile_sizes"] = sizes
    del d_ptr2, d_idx2
    # the entry point without a plan, as a TVM process binds it
    from sparsetir_amd import _lib as stlib
    L16 = stlib.lib()
    vp = lambda v: ctypes.c_void_p(v.data_ptr())

    def plain(out_code, c):
        stlib.check(L16.stir_tc_spmm_f16(out_code, mb2, 32, 16, f2, nnzb2, vp(a2), vp(b2), vp(c), vp(gp), vp(ti),
                                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))

    tm = time_small(lambda: plain(0, c16), 50, 5, torch)
    out["tcspmm_config2_feat128_f16_out_no_plan"] = {"us_per_call": tm["us_per_call"], "us_graph": tm["us_graph"],
                                                     "us": tm["us_back_to_back"]}
    tm = time_small(lambda: plain(2, c2), 50, 5, torch)
    out["tcspmm_config2_feat128_no_plan"] = {"us_per_call": tm["us_per_call"], "us_graph": tm["us_graph"],
                                             "us": tm["us_back_to_back"]}

    # fp32 forms: ELL3D buckets with 32-slot groups (the reference's composable fp32 setting) and the
    # CSF traversal; W is [R, fout, fin]
    w32 = t(np.ascontiguousarray(cfg["w"].transpose(0, 2, 1)).ravel())
    x32 = t(cfg["x"].ravel())
    byts32 = 8.0 * E + 4.0 * n * fin + 4.0 * R * fin * fout + 4.0 * n * fout
    rb32 = [32 // b for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"],
                                            rb32, buckets)
    triples, mids = [], []
    for k in range(len(buckets)):
        triples += [t(mask[k].astype(np.float32).ravel()), t(rows[k].ravel()), t(cols[k].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[k]))))
    # the operator's default: every 64-row tile of Y summed on chip from an edge index, no atomics
    f32 = ops.build_rgms_f32(n, n, R, fin, fout, rb32, buckets, [c.shape[0] for c in cols])
    f32(w32, x32, y, *triples, *mids)  # builds its edge index
    tm = time_small(lambda: f32(w32, x32, y, *triples, *mids), 20, 2, torch)
    d = tm["us_back_to_back"] / 1e6
    out["rgms_f32_ell3d_config5"] = {"us_per_call": tm["us_per_call"], "us_graph": tm["us_graph"], "us": d * 1e6, "tflops": flops / d / 1e12, "alg_GBps": byts32 / d / 1e9,
                                     "frac_of_hbm_peak": byts32 / d / 1e9 / HBM_PEAK_GBS,
                                     "algorithmic_bytes": byts32,
                                     "roofline": side_roofline("hbm", byts32 / d / 1e9, "rgms_f32_ell3d_config5"),
                                     "ell_rows": int(sum(r.size for r in rows))}
    # the form that holds nothing derived from the index arrays: one atomic per (ELL row, output)
    f32a = ops.build_rgms_f32(n, n, R, fin, fout, rb32, buckets, [c.shape[0] for c in cols], deterministic=False)
    tm_a = time_small(lambda: f32a(w32, x32, y, *triples, *mids), 20, 2, torch)
    da = tm_a["us_back_to_back"] / 1e6
    out["rgms_f32_ell3d_config5"]["atomic_form_us"] = da * 1e6
    del f32a
    # every ELL row adds feat_out floats to Y with one atomic each: that form's bound.  Beside
    # it, what the same number of row additions to hashed rows of Y takes with nothing else going on
    er = out["rgms_f32_ell3d_config5"]["ell_rows"]
    out["rgms_f32_ell3d_config5"]["atomic_adds"] = er * fout
    out["rgms_f32_ell3d_config5"]["atomic_adds_G_per_s"] = er * fout / da / 1e9
    if fout == 32:
        P = load_probes()
        yp = ctypes.c_void_p(y.data_ptr())

        def scatter_only():  # on the stream that is current when it is called (a capture has its own)
            if P.bench_probe_atomic_rows(yp, n, er, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) != 0:
                raise RuntimeError("atomic probe failed")
        tp = time_small(scatter_only, 20, 2, torch)
        out["rgms_f32_ell3d_config5"]["probe_atomic_rows_us"] = tp["us_back_to_back"]
        out["rgms_f32_ell3d_config5"]["probe_atomic_adds_G_per_s"] = er * fout / tp["us_back_to_back"] / 1e3
    csf = [t(cfg[k]) for k in ("indptr0", "indices0", "indptr1", "indices1")]
    ones = torch.ones(E, device=dev)
    fc = ops.build_rgms_csf(n, n, R, fin, fout, len(cfg["indices0"]), E)
    fc(ones, w32, x32, y, *csf)  # builds its edge index
    tm = time_small(lambda: fc(ones, w32, x32, y, *csf), 20, 2, torch)
    d = tm["us_back_to_back"] / 1e6
    out["rgms_f32_csf_config5"] = {"us_per_call": tm["us_per_call"], "us_graph": tm["us_graph"], "us": d * 1e6, "tflops": flops / d / 1e12, "alg_GBps": byts32 / d / 1e9,
                                   "frac_of_hbm_peak": byts32 / d / 1e9 / HBM_PEAK_GBS,
                                   "algorithmic_bytes": byts32,
                                   "roofline": side_roofline("hbm", byts32 / d / 1e9, "rgms_f32_csf_config5"),
                                   "stored_rows": int(len(cfg["indices0"]))}
    fca = ops.build_rgms_csf(n, n, R, fin, fout, len(cfg["indices0"]), E, deterministic=False)  # stateless, atomics
    tm_a = time_small(lambda: fca(ones, w32, x32, y, *csf), 20, 2, torch)
    out["rgms_f32_csf_config5"]["atomic_form_us"] = tm_a["us_back_to_back"]
    del fca
    return out


def hyb_workload(args, columns, torch, dev, st, datasets, ops):
    """Graph, device format pass and operators of config 3 with the given column distribution."""
    t0 = time.time()
    g = datasets.config3(columns=columns, scale=args.scale)
    m, n = g["m"], g["n"]
    indptr, indices = g["indptr"], g["indices"]
    nnz = int(indices.shape[0])
    parts = args.parts if args.parts is not None else g["num_col_parts"]
    buckets = [int(b) for b in args.buckets.split(",")] if args.buckets else g["buckets"]
    log(f"[bench] graph ({columns} columns): {m} nodes, {nnz} edges, max degree {int(np.diff(indptr).max())} "
        f"({time.time() - t0:.1f}s); hyb: {parts} column partitions, widths {buckets}")
    d_indptr = torch.from_numpy(indptr).to(dev)
    d_indices = torch.from_numpy(indices).to(dev)
    torch.cuda.synchronize()
    t0 = time.time()
    rows, cols, mask = st.column_part_hyb(m, n, d_indptr, d_indices, parts, buckets)
    torch.cuda.synchronize()
    fmt_first_s = time.time() - t0   # includes the first allocations of the process
    del rows, cols, mask
    t0 = time.time()
    rows, cols, mask = st.column_part_hyb(m, n, d_indptr, d_indices, parts, buckets)
    torch.cuda.synchronize()
    fmt_s = time.time() - t0
    triples, nrows, slots = [], [], 0
    for p in range(parts):
        for b in range(len(buckets)):
            triples += [mask[p][b].reshape(-1).float(), rows[p][b], cols[p][b].reshape(-1)]
            nrows.append(int(rows[p][b].shape[0]))
            slots += int(cols[p][b].numel())
    del mask
    log(f"[bench] device column_part_hyb: {fmt_s * 1e3:.1f} ms, {sum(nrows)} ELL rows, "
        f"{slots} slots ({slots / nnz:.3f} per edge)")
    feat = args.feat
    gen = torch.Generator(device=dev)
    gen.manual_seed(2)
    x = torch.randn(n * feat, generator=gen, device=dev, dtype=torch.float32)
    c = torch.zeros(m * feat, device=dev, dtype=torch.float32)
    hyb = ops.build_hyb_csrmm(m, n, feat, parts, buckets, nrows)
    csr = ops.build_csrmm(m, n, feat, nnz)
    sig = f"{columns}/p{parts}/b{'-'.join(map(str, buckets))}/f{feat}/s{args.scale}"
    return dict(m=m, n=n, nnz=nnz, indptr=indptr, indices=indices, d_indptr=d_indptr, d_indices=d_indices,
                parts=parts, buckets=buckets, triples=triples, nrows=nrows, slots=slots, fmt_s=fmt_s,
                fmt_first_s=fmt_first_s, x=x, c=c, hyb=hyb, csr=csr, gen=gen, sig=sig, feat=feat)


def check_first_call(wl, torch, dev):
    """hyb against the CSR kernel on every element of the first call's output."""
    m, feat, nnz = wl["m"], wl["feat"], wl["nnz"]
    wl["c"].zero_()
    wl["hyb"](wl["x"], wl["c"], *wl["triples"])
    ones = torch.ones(nnz, device=dev, dtype=torch.float32)
    c_csr = torch.empty(m * feat, device=dev, dtype=torch.float32)
    wl["csr"](ones, wl["x"], c_csr, wl["d_indptr"], wl["d_indices"])
    torch.cuda.synchronize()
    deg = torch.from_numpy(np.diff(wl["indptr"]).astype(np.float32)).to(dev)
    # |x| <~ 6 for N(0,1): bound the summed magnitude by deg * 6
    tol = 1e-5 * (deg.clamp(min=1.0) * 6.0).repeat_interleave(feat)
    diff = (wl["c"] - c_csr).abs()
    ok = bool((diff <= tol).all().item())
    worst = float(diff.max().item())
    log(f"[bench] hyb vs csr kernel: max |diff| {worst:.3e}, within tolerance: {ok}")
    return ok, worst, ones, c_csr


def roofline_block(wl, dev_mean, dev_min, probes=None):
    m, n, nnz, feat, slots = wl["m"], wl["n"], wl["nnz"], wl["feat"], wl["slots"]
    alg_bytes = 8.0 * nnz + 4.0 * (m + 1) + 4.0 * n * feat + 4.0 * m * feat
    achieved = alg_bytes / dev_mean / 1e9
    traffic, note = measured_traffic(wl["sig"])
    blk = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": note,
           "kernel": "hyb_spmm_kernel<32,1>" if feat == 128 else "hyb_spmm_kernel",
           "kernel_ms_mean": dev_mean * 1e3, "kernel_ms_min": dev_min * 1e3,
           "algorithmic_bytes": alg_bytes,
           "traffic_GBps": traffic / dev_mean / 1e9 if traffic else None,
           "uncached_gather_bytes": 4.0 * slots * feat + 8.0 * slots + 4.0 * m * feat}
    if probes is not None:
        blk["probes"] = probes
    return blk, alg_bytes


def main():
    global PROFILE_RUN
    args = parse()
    PROFILE_RUN = args.profile
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported: this build has no "
              "multi-GPU path (the kernel runs on one GPU's share at its real shape).", file=sys.stderr)
        sys.exit(2)
    import torch
    import sparsetir_amd as st
    from sparsetir_amd import datasets, ops

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    feat = args.feat
    if args.lds_probes:
        out = torch.zeros(512, dtype=torch.int32, device=dev)
        rc = load_probes().bench_probe_bsr_lds(2000, ctypes.c_void_p(out.data_ptr()),
                                               ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        print(json.dumps({"lds_probes": "launched" if rc == 0 else "failed"}))
        sys.exit(0 if rc == 0 else 1)

    wl = hyb_workload(args, args.columns, torch, dev, st, datasets, ops)
    m, n, nnz = wl["m"], wl["n"], wl["nnz"]
    indptr, indices = wl["indptr"], wl["indices"]
    x, c, hyb, csr, triples = wl["x"], wl["c"], wl["hyb"], wl["csr"], wl["triples"]
    d_indptr, d_indices = wl["d_indptr"], wl["d_indices"]

    # ---- correctness of the first call: against the CSR kernel everywhere, and against the
    # CPU oracle on a row sample
    hyb_vs_csr_ok, max_diff, ones, c_csr = check_first_call(wl, torch, dev)
    check = {"hyb_vs_csr_max_abs_diff": max_diff, "hyb_vs_csr_ok": hyb_vs_csr_ok}
    cpu = None
    if not args.no_cpu:
        import oracle  # checker and cpu_baseline only
        r_hi = min(m, args.cpu_rows)
        sub_ptr = indptr[: r_hi + 1].copy()
        sub_idx = indices[: sub_ptr[-1]]
        xh = x.cpu().numpy()
        vals = np.ones(sub_idx.shape[0], np.float32)
        t0 = time.perf_counter()
        ref = oracle.csrmm(vals, xh, sub_ptr, sub_idx, feat)
        cpu_s = time.perf_counter() - t0
        got = c[: r_hi * feat].cpu().numpy().reshape(r_hi, feat)
        nz = np.diff(sub_ptr) > 0
        bound = 1e-5 * (np.maximum(np.diff(sub_ptr), 1) * 6.0)[:, None]
        oracle_ok = bool(np.all(np.abs(got[nz] - ref[nz]) <= bound[nz]))
        check.update({"oracle_rows": int(r_hi), "oracle_ok": oracle_ok,
                      "oracle_max_abs_diff": float(np.abs(got[nz] - ref[nz]).max())})
        cpu_flops = 2.0 * sub_idx.shape[0] * feat
        cpu = {"value": cpu_flops / cpu_s / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
               "sample": f"rows [0, {r_hi}) of the same graph ({sub_idx.shape[0]} edges, feat {feat}): "
                         f"serial CSR loop nest of the reference's unscheduled llvm build, {cpu_s:.2f} s; "
                         f"host has {os.cpu_count()} logical CPUs"}
        log(f"[bench] cpu baseline: {cpu['value']:.2f} GFLOP/s on 1 core ({cpu_s:.2f}s); oracle check {oracle_ok}")
        del xh, ref, got

    # Probes: a plain copy of known size (n*feat*4 bytes read and written; also the kernel the
    # FETCH_SIZE / WRITE_SIZE counters are scaled by under rocprofv3 --pmc) and nnz gathers of
    # feat*4-byte rows at pseudo-random indices (what the access pattern allows at best).
    P = load_probes()
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    st0 = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    nbytes = (n * feat * 4) // 16 * 16

    def probe(rc):
        if rc != 0:
            raise RuntimeError("bandwidth probe failed")

    _, copy_s, _ = time_steps(lambda: probe(P.bench_probe_copy(vp(x), vp(c_csr), nbytes, st0)), 3, 1, torch)
    probes = {"copy_GBps": 2.0 * nbytes / copy_s / 1e9}
    if feat in (32, 64, 128, 256):
        _, gat_s, _ = time_steps(lambda: probe(P.bench_probe_gather(vp(x), n, feat, nnz, vp(c_csr), st0)),
                                 3, 1, torch)
        probes["random_row_gather_GBps"] = nnz * feat * 4.0 / gat_s / 1e9
    # ... and the rate at which the matrix cores take v_mfma_f32_32x32x16_f16 from registers (four
    # wavefronts per SIMD, four independent accumulators each, 2.4 ms): what the 2.5 PFLOP/s that
    # the BSR / TC-SpMM / RGMS lines are priced against amounts to at the clock this GPU sustains
    mfma_flop = ctypes.c_double(0.0)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    _, mfma_s, _ = time_steps(lambda: probe(P.bench_probe_mfma_f16(cus, 4, 8192, vp(c_csr), ctypes.byref(mfma_flop),
                                                                   st0)), 3, 1, torch)
    probes["mfma_f16_32x32x16_TFLOPs"] = mfma_flop.value / mfma_s / 1e12
    log(f"[bench] probes: {probes}")

    # ---- timed region
    wall, dev_mean, dev_min = time_steps(lambda: hyb(x, c, *triples), args.steps, args.warmup, torch)
    flops = 2.0 * nnz * feat
    roof, alg_bytes = roofline_block(wl, dev_mean, dev_min, probes)
    result = {
        "metric": "hyb SpMM GFLOP/s (fp32, feat %d, power-law graph %d nodes / %d edges)" % (feat, m, nnz),
        "value": flops / wall / 1e9,
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "config 3: hyb SpMM fp32, 2.45M-node / 61.9M-edge power-law graph, feat 128",
                   "nodes": m, "edges": nnz, "feat": feat, "columns": args.columns,
                   "num_col_parts": wl["parts"], "buckets": wl["buckets"], "ell_slots": wl["slots"],
                   "format_pass_ms": wl["fmt_s"] * 1e3, "format_pass_first_call_ms": wl["fmt_first_s"] * 1e3,
                   "format_pass_alg_GBps": (4.0 * (m + 1) + 4.0 * nnz + 4.0 * (sum(wl["nrows"]) + 2 * wl["slots"]))
                   / wl["fmt_s"] / 1e9},
        "roofline": roof,
        "cpu_baseline": cpu,
        "check": check,
    }

    if not args.no_extra:
        extra = {}
        steps = max(3, min(args.steps, 10))
        w2, d2, _ = time_steps(lambda: csr(ones, x, c_csr, d_indptr, d_indices), steps, 1, torch)
        extra["csr_spmm"] = {"gflops": flops / w2 / 1e9, "ms": d2 * 1e3, "alg_GBps": alg_bytes / d2 / 1e9,
                             "roofline": side_roofline("hbm", alg_bytes / d2 / 1e9,
                                                       f"csr/{args.columns}/f{feat}/s{args.scale}")}
        del c_csr, ones
        f2 = 64
        gen = wl["gen"]
        a2 = torch.randn(m * f2, generator=gen, device=dev, dtype=torch.float32)
        b2 = torch.randn(n * f2, generator=gen, device=dev, dtype=torch.float32)
        out = torch.empty(nnz, device=dev, dtype=torch.float32)
        mid = torch.empty(nnz, device=dev, dtype=torch.int32)
        pre = ops.build_sddmm_preproc(m, n, f2, nnz)
        sd = ops.build_sddmm_scaled(m, n, f2, nnz)
        edge = torch.rand(nnz, generator=gen, device=dev, dtype=torch.float32)
        sargs = (a2, b2, out, d_indptr, d_indices, mid)
        w3, d3, _ = time_steps(lambda: pre(*sargs), 3, 1, torch)
        w4, d4, _ = time_steps(lambda: sd(*sargs, edge), steps, 1, torch)
        # out_e = A_e * <X[row], Y[col]>: index + edge value + result per nonzero, X and Y once
        sd_bytes = nnz * 12.0 + 4.0 * (m + 1) + 4.0 * (m + n) * f2
        extra["sddmm_feat64_scaled"] = {"gflops": (2.0 * f2 + 1.0) * nnz / w4 / 1e9, "ms": d4 * 1e3,
                                        "alg_GBps": sd_bytes / d4 / 1e9,
                                        "frac_of_hbm_peak": sd_bytes / d4 / 1e9 / HBM_PEAK_GBS,
                                        "algorithmic_bytes": sd_bytes,
                                        "roofline": side_roofline("hbm", sd_bytes / d4 / 1e9,
                                                                  f"sddmm/{args.columns}/f{f2}/s{args.scale}"),
                                        "preproc_ms": d3 * 1e3}
        del edge, a2, b2, out, mid, sargs
        if args.parts is None and args.buckets is None and not getattr(args, "profile", False):
            # the reference's own decomposition for a graph of this size: 16 column partitions, widths
            # 1..32 (examples/spmm/bench_spmm.py:233-253); the bench line above uses 1 x 1..512
            rparts, rbuckets = 16, [1, 2, 4, 8, 16, 32]
            rr, rc, rm = st.column_part_hyb(m, n, d_indptr, d_indices, rparts, rbuckets)
            rtriples, rnrows = [], []
            for p in range(rparts):
                for b in range(len(rbuckets)):
                    rtriples += [rm[p][b].reshape(-1).float(), rr[p][b], rc[p][b].reshape(-1)]
                    rnrows.append(int(rr[p][b].shape[0]))
            del rr, rc, rm
            rhyb = ops.build_hyb_csrmm(m, n, feat, rparts, rbuckets, rnrows)
            c.zero_()
            hyb(x, c, *triples)
            c_ref = torch.zeros_like(c)
            rhyb(x, c_ref, *rtriples)
            torch.cuda.synchronize()
            rdiff = float((c_ref - c).abs().max().item())
            deg_max = float(np.diff(indptr).max())
            check["reference_decomposition_vs_bench_decomposition_ok"] = bool(rdiff <= 1e-5 * 6.0 * max(deg_max, 1.0))

            def rstep():
                c_ref.zero_()  # the operator adds to C
                rhyb(x, c_ref, *rtriples)

            wr, dr, _ = time_steps(rstep, steps, 1, torch)
            wz, dz, _ = time_steps(lambda: c_ref.zero_(), steps, 1, torch)
            extra["hyb_spmm_reference_decomposition"] = {"num_col_parts": rparts, "buckets": rbuckets,
                                                         "ell_rows": int(sum(rnrows)),
                                                         "ms_per_step_with_clearing_C": wr * 1e3,
                                                         "clearing_C_ms": wz * 1e3, "ms": (wr - wz) * 1e3,
                                                         "gflops": flops / (wr - wz) / 1e9,
                                                         "max_abs_diff_to_bench_decomposition": rdiff}
            del rtriples, rhyb, c_ref
            torch.cuda.empty_cache()
        # the main workload's arrays are released before the next graph is built
        del x, c, hyb, csr, triples, d_indptr, d_indices, indptr, indices
        wl.clear()
        torch.cuda.empty_cache()
        if args.scale == 1.0 or args.columns == "uniform":
            # the same kernel on the same-sized graph whose columns follow the power law as well
            # (an undirected graph: hub rows are hub columns), where L2 and the memory-side cache
            # hold the hot rows of X
            other = "symmetric" if args.columns == "uniform" else "uniform"
            w2l = hyb_workload(args, other, torch, dev, st, datasets, ops)
            ok2, worst2, ones2, ccsr2 = check_first_call(w2l, torch, dev)
            check[f"{other}_hyb_vs_csr_ok"] = ok2
            ws, ds, dmin = time_steps(lambda: w2l["hyb"](w2l["x"], w2l["c"], *w2l["triples"]), steps, 2, torch)
            wc, dc, _ = time_steps(lambda: w2l["csr"](ones2, w2l["x"], ccsr2, w2l["d_indptr"], w2l["d_indices"]),
                                   steps, 1, torch)
            roof2, _ = roofline_block(w2l, ds, dmin)
            fl2 = 2.0 * w2l["nnz"] * feat
            extra[f"hyb_spmm_{other}_columns"] = {"nodes": w2l["m"], "edges": w2l["nnz"], "gflops": fl2 / ws / 1e9,
                                                  "ms_per_step": ws * 1e3, "csr_ms": dc * 1e3,
                                                  "hyb_vs_csr_max_abs_diff": worst2, "roofline": roof2}
            del ones2, ccsr2
            w2l.clear()
            torch.cuda.empty_cache()
        extra.update(side_kernels(torch, dev, ops, st, datasets, time_steps))
        extra["config2_hyb_vs_csr"] = config2_sweep(torch, dev, ops, st, datasets, time_steps)
        result["extra"] = extra

    print(json.dumps(result), flush=True)
    failed = [k for k, v in check.items() if k.endswith("_ok") and not v]
    if failed:
        log(f"[bench] FAILED checks: {failed}")
        sys.exit(3)


if __name__ == "__main__":
    main()
