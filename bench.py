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
row sample of the same graph.  `extra` carries the CSR row-split comparator and SDDMM.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE; scaled by a
# plain copy of known size), keyed by workload signature.  None when not measured.
MEASURED_TRAFFIC = {
    # profiles/hyb_spmm_config3_uniform.md: FETCH_SIZE 15,737,890 KiB x 2.0 + WRITE_SIZE 1,266,963 KiB x 1.0
    "uniform/p1/b1-2-4-8-16-32-64-128-256-512/f128/s1.0": 33.53e9,
}


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


MFMA_F16_PEAK_TFLOPS = 2500.0


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
    ones = torch.ones(nnz, device=dev)
    out = {"nodes": m, "edges": nnz, "num_col_parts": parts}
    for feat in (32, 64, 128, 256):
        x = torch.randn(n * feat, device=dev)
        c = torch.zeros(m * feat, device=dev)
        hyb = ops.build_hyb_csrmm(m, n, feat, parts, buckets, nrows)
        csr = ops.build_csrmm(m, n, feat, nnz)
        _, dh, _ = time_steps(lambda: hyb(x, c, *triples), 50, 5, torch)
        _, dc, _ = time_steps(lambda: csr(ones, x, c, d_ptr, d_idx), 50, 5, torch)
        byts = 8.0 * nnz + 4.0 * (m + 1) + 4.0 * n * feat + 4.0 * m * feat
        out[f"feat{feat}"] = {"hyb_us": dh * 1e6, "csr_us": dc * 1e6, "hyb_gflops": 2.0 * nnz * feat / dh / 1e9,
                              "hyb_alg_GBps": byts / dh / 1e9}
    return out


def side_kernels(torch, dev, ops, st, datasets, time_steps):
    """BSR SpMM (config 4 and a scaled-up shape) and RGMS (config 5): time, flop rate against the
    dense fp16 MFMA peak, algorithmic bytes against the HBM peak."""
    out = {}

    def bsr(tag, mb, nb, blk, density, feat, dtype):
        cfg = datasets.config4(seed=3, mb=mb, nb=nb, blk=blk, density=density, feat=32)
        nnzb = len(cfg["indices"])
        a = torch.from_numpy(cfg["data"]).to(dev).to(dtype).reshape(-1)
        x = torch.randn(nb * blk * feat, device=dev).to(dtype)
        y = torch.zeros(mb * blk * feat, device=dev, dtype=dtype)
        ip, ix = torch.from_numpy(cfg["indptr"]).to(dev), torch.from_numpy(cfg["indices"]).to(dev)
        f = ops.build_bsrmm(mb, nb, nnzb, blk, feat, dtype)
        _, d, _ = time_steps(lambda: f(a, x, y, ip, ix), 100, 5, torch)
        flops = 2.0 * nnzb * blk * blk * feat
        byts = 2.0 * nnzb * blk * blk + 4 * nnzb + 4 * (mb + 1) + 2.0 * nb * blk * feat + 2.0 * mb * blk * feat
        out[tag] = {"us": d * 1e6, "tflops": flops / d / 1e12, "frac_of_mfma_peak": flops / d / 1e12 / MFMA_F16_PEAK_TFLOPS,
                    "alg_GBps": byts / d / 1e9, "frac_of_hbm_peak": byts / d / 1e9 / HBM_PEAK_GBS,
                    "nnzb": nnzb, "shape": [mb * blk, nb * blk, feat], "blk": blk, "dtype": str(dtype).split(".")[-1]}

    bsr("bsr_config4_f16", 128, 128, 32, 0.10, 512, torch.float16)
    bsr("bsr_config4_bf16", 128, 128, 32, 0.10, 512, torch.bfloat16)
    bsr("bsr_16384x16384_f4096_f16", 512, 512, 32, 0.10, 4096, torch.float16)

    cfg = datasets.config5()
    R, n, fin, fout = cfg["num_rels"], cfg["n"], cfg["feat_in"], cfg["feat_out"]
    buckets, group = cfg["buckets"], 256
    rb = [group // b for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"],
                                            rb, buckets)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    triples, mids = [], []
    for k in range(len(buckets)):
        triples += [t(mask[k].astype(np.float16).ravel()), t(rows[k].ravel()), t(cols[k].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[k]))))
    f = ops.build_rgms(n, n, R, fin, fout, rb, buckets, [c.shape[0] for c in cols])
    w = t(cfg["w"].astype(np.float16).ravel())
    x = t(cfg["x"].astype(np.float16).ravel())
    y = torch.zeros(n * fout, device=dev)
    _, d, _ = time_steps(lambda: f(w, x, y, *triples, *mids), 10, 1, torch)
    E = len(cfg["indices1"])
    flops = 2.0 * E * fin * fout + 2.0 * E * fout
    byts = 8.0 * E + 2.0 * n * fin + 2.0 * R * fin * fout + 4.0 * n * fout
    out["rgms_config5"] = {"us": d * 1e6, "tflops": flops / d / 1e12, "alg_GBps": byts / d / 1e9,
                           "frac_of_hbm_peak": byts / d / 1e9 / HBM_PEAK_GBS, "edges": E,
                           "ell_rows": int(sum(r.size for r in rows)),
                           "accumulation": "32-row output tiles, written once (no atomics)"}

    # SpMM over the condensed format (t = 32, g = 16) on the config-2 graph, fp16 in, fp32 out
    g2 = datasets.config2()
    gptr, tiles, cmask = st.condense(g2["indptr"], g2["indices"], 32, 16)
    mb2, nnzb2, f2 = len(gptr) - 1, tiles.shape[0], 128
    tc = ops.build_tcspmm(mb2, nnzb2, f2, 32, 16, g2["n"], torch.float32)
    a2, b2 = t(cmask.astype(np.float16).ravel()), torch.randn(g2["n"] * f2, device=dev).half()
    c2 = torch.zeros(mb2 * 32 * f2, device=dev)
    gp, ti = t(gptr), t(tiles.ravel())
    _, d, _ = time_steps(lambda: tc(a2, b2, c2, gp, ti), 50, 5, torch)
    nnz2 = len(g2["indices"])
    out["tcspmm_config2_feat128"] = {"us": d * 1e6, "useful_gflops": 2.0 * nnz2 * f2 / d / 1e9,
                                     "mfma_tflops": 2.0 * nnzb2 * 32 * 16 * f2 / d / 1e12, "groups": int(nnzb2),
                                     "mask_density": float(nnz2) / (nnzb2 * 32 * 16)}

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
    f32 = ops.build_rgms_f32(n, n, R, fin, fout, rb32, buckets, [c.shape[0] for c in cols])
    _, d, _ = time_steps(lambda: f32(w32, x32, y, *triples, *mids), 10, 1, torch)
    out["rgms_f32_ell3d_config5"] = {"us": d * 1e6, "tflops": flops / d / 1e12, "alg_GBps": byts32 / d / 1e9,
                                     "frac_of_hbm_peak": byts32 / d / 1e9 / HBM_PEAK_GBS,
                                     "ell_rows": int(sum(r.size for r in rows))}
    csf = [t(cfg[k]) for k in ("indptr0", "indices0", "indptr1", "indices1")]
    ones = torch.ones(E, device=dev)
    fc = ops.build_rgms_csf(n, n, R, fin, fout, len(cfg["indices0"]), E)
    _, d, _ = time_steps(lambda: fc(ones, w32, x32, y, *csf), 10, 1, torch)
    out["rgms_f32_csf_config5"] = {"us": d * 1e6, "tflops": flops / d / 1e12, "alg_GBps": byts32 / d / 1e9,
                                   "frac_of_hbm_peak": byts32 / d / 1e9 / HBM_PEAK_GBS,
                                   "stored_rows": int(len(cfg["indices0"]))}
    return out


def main():
    args = parse()
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

    t0 = time.time()
    g = datasets.config3(columns=args.columns, scale=args.scale)
    m, n = g["m"], g["n"]
    indptr, indices = g["indptr"], g["indices"]
    nnz = int(indices.shape[0])
    parts = args.parts if args.parts is not None else g["num_col_parts"]
    buckets = [int(b) for b in args.buckets.split(",")] if args.buckets else g["buckets"]
    log(f"[bench] graph: {m} nodes, {nnz} edges, max degree {int(np.diff(indptr).max())} "
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

    gen = torch.Generator(device=dev)
    gen.manual_seed(2)
    x = torch.randn(n * feat, generator=gen, device=dev, dtype=torch.float32)
    c = torch.zeros(m * feat, device=dev, dtype=torch.float32)
    hyb = ops.build_hyb_csrmm(m, n, feat, parts, buckets, nrows)

    # ---- correctness of the first call: against the CSR kernel everywhere, and against the
    # CPU oracle on a row sample
    hyb(x, c, *triples)
    ones = torch.ones(nnz, device=dev, dtype=torch.float32)
    c_csr = torch.empty(m * feat, device=dev, dtype=torch.float32)
    csr = ops.build_csrmm(m, n, feat, nnz)
    csr(ones, x, c_csr, d_indptr, d_indices)
    torch.cuda.synchronize()
    deg = torch.from_numpy(np.diff(indptr).astype(np.float32)).to(dev)
    # |x| <~ 6 for N(0,1): bound the summed magnitude by deg * 6
    tol = 1e-5 * (deg.clamp(min=1.0) * 6.0).repeat_interleave(feat)
    diff = (c - c_csr).abs()
    hyb_vs_csr_ok = bool((diff <= tol).all().item())
    max_diff = float(diff.max().item())
    log(f"[bench] hyb vs csr kernel: max |diff| {max_diff:.3e}, within tolerance: {hyb_vs_csr_ok}")

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
    import ctypes
    from sparsetir_amd import _lib
    L = _lib.lib()
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    st0 = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    nbytes = (n * feat * 4) // 16 * 16
    _, copy_s, _ = time_steps(lambda: _lib.check(L.stir_probe_copy(vp(x), vp(c_csr), nbytes, st0)), 3, 1, torch)
    probes = {"copy_GBps": 2.0 * nbytes / copy_s / 1e9}
    if feat in (32, 64, 128, 256):
        _, gat_s, _ = time_steps(lambda: _lib.check(L.stir_probe_gather(vp(x), n, feat, nnz, vp(c_csr), st0)),
                                 3, 1, torch)
        probes["random_row_gather_GBps"] = nnz * feat * 4.0 / gat_s / 1e9
    log(f"[bench] probes: {probes}")

    # ---- timed region
    wall, dev_mean, dev_min = time_steps(lambda: hyb(x, c, *triples), args.steps, args.warmup, torch)
    flops = 2.0 * nnz * feat
    alg_bytes = 8.0 * nnz + 4.0 * (m + 1) + 4.0 * n * feat + 4.0 * m * feat
    achieved = alg_bytes / dev_mean / 1e9
    sig = f"{args.columns}/p{parts}/b{'-'.join(map(str, buckets))}/f{feat}/s{args.scale}"
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
                   "num_col_parts": parts, "buckets": buckets, "ell_slots": slots,
                   "format_pass_ms": fmt_s * 1e3, "format_pass_first_call_ms": fmt_first_s * 1e3,
                   "format_pass_alg_GBps": (4.0 * (m + 1) + 4.0 * nnz + 4.0 * (sum(nrows) + 2 * slots)) / fmt_s / 1e9},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC.get(sig),
                     "kernel": "hyb_spmm_kernel<32,1>" if feat == 128 else "hyb_spmm_kernel",
                     "kernel_ms_mean": dev_mean * 1e3, "kernel_ms_min": dev_min * 1e3,
                     "algorithmic_bytes": alg_bytes, "probes": probes,
                     "traffic_GBps": (MEASURED_TRAFFIC.get(sig) or 0) / dev_mean / 1e9 or None,
                     "uncached_gather_bytes": 4.0 * slots * feat + 8.0 * slots + 4.0 * m * feat},
        "cpu_baseline": cpu,
        "check": check,
    }

    if not args.no_extra:
        extra = {}
        steps = max(3, min(args.steps, 10))
        w2, d2, _ = time_steps(lambda: csr(ones, x, c_csr, d_indptr, d_indices), steps, 1, torch)
        extra["csr_spmm"] = {"gflops": flops / w2 / 1e9, "ms": d2 * 1e3, "alg_GBps": alg_bytes / d2 / 1e9}
        del c_csr, ones
        f2 = 64
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
                                        "preproc_ms": d3 * 1e3}
        del edge
        del a2, b2, out, mid
        extra.update(side_kernels(torch, dev, ops, st, datasets, time_steps))
        extra["config2_hyb_vs_csr"] = config2_sweep(torch, dev, ops, st, datasets, time_steps)
        result["extra"] = extra

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
