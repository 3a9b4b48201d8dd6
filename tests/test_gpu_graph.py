"""The launches allocate nothing and synchronise nothing once their plans exist, so a caller can
record them into a HIP graph.  Each graph is replayed several times with eager work and
synchronisations in between; every replay is checked against the eager result."""
import numpy as np
import pytest
import torch

import sparsetir_amd as st
from sparsetir_amd import datasets, ops

pytestmark = pytest.mark.gpu


def _replays(dev, graph, out, want, refill):
    for k in range(3):
        refill()
        # unrelated eager work between replays
        junk = torch.randn(1 << 16, device=dev).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {k}"
        del junk


def test_graph_bsr_config4(dev):
    cfg = datasets.config4()
    mb, nb, blk, feat = cfg["mb"], cfg["nb"], cfg["blk"], cfg["feat"]
    a = torch.from_numpy(cfg["data"]).to(dev).half().reshape(-1)
    x = torch.from_numpy(cfg["x"]).to(dev).half().reshape(-1)
    ip, ix = torch.from_numpy(cfg["indptr"]).to(dev), torch.from_numpy(cfg["indices"]).to(dev)
    f = ops.build_bsrmm(mb, nb, len(cfg["indices"]), blk, feat, torch.float16)
    want = torch.empty(mb * blk * feat, dtype=torch.float16, device=dev)
    f(a, x, want, ip, ix)
    torch.cuda.synchronize()
    y = torch.zeros_like(want)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        f(a, x, y, ip, ix)  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        f(a, x, y, ip, ix)
    _replays(dev, g, y, want, lambda: y.fill_(1.0))


def test_graph_hyb_and_rgms_tiles(dev):
    """hyb SpMM (plan made before capture) and the destination-tiled RGMS (edge index made by an
    eager first launch): two kernels of different operators in one graph."""
    gcfg = datasets.config2()
    m, n, feat, parts, buckets = gcfg["m"], gcfg["n"], 32, 2, [1, 2, 4, 8, 16, 32]
    t = lambda v: torch.from_numpy(np.ascontiguousarray(v)).to(dev)
    rows, cols, mask = st.column_part_hyb(m, n, t(gcfg["indptr"]), t(gcfg["indices"]), parts, buckets)
    triples = [a for p in range(parts) for b in range(len(buckets))
               for a in (mask[p][b].reshape(-1).float(), rows[p][b], cols[p][b].reshape(-1))]
    hyb = ops.build_hyb_csrmm(m, n, feat, parts, buckets, [int(r.shape[0]) for p in rows for r in p])
    x = torch.randn(n * feat, device=dev)
    c_want = torch.zeros(m * feat, device=dev)
    hyb(x, c_want, *triples)

    cfg = datasets.config5(n=20000, num_rels=9, num_edges=200000, seed=7)
    R, rn, fin, fout, rb_buckets = cfg["num_rels"], cfg["n"], cfg["feat_in"], cfg["feat_out"], cfg["buckets"]
    rb = [256 // b for b in rb_buckets]
    ptr, rrows, rcols, rmask = st.csf_to_ell3d(cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"],
                                               rb, rb_buckets)
    rtrip, mids = [], []
    for k in range(len(rb_buckets)):
        rtrip += [t(rmask[k].astype(np.float16).ravel()), t(rrows[k].ravel()), t(rcols[k].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[k]))))
    rg = ops.build_rgms(rn, rn, R, fin, fout, rb, rb_buckets, [c.shape[0] for c in rcols])
    w, rx = t(cfg["w"].astype(np.float16).ravel()), t(cfg["x"].astype(np.float16).ravel())
    y_want = torch.zeros(rn * fout, device=dev)
    rg(w, rx, y_want, *rtrip, *mids)  # builds the edge index
    torch.cuda.synchronize()

    # rows of the last bucket are added with atomics in any order: |a| = 1, |x| below ~6
    deg = t(np.diff(gcfg["indptr"]).astype(np.float32))
    tol = (1e-5 * 6.0 * deg.clamp(min=1.0)).repeat_interleave(feat)
    c, y = torch.zeros_like(c_want), torch.zeros_like(y_want)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        c.zero_()
        y.zero_()
        hyb(x, c, *triples)
        rg(w, rx, y, *rtrip, *mids)
    for k in range(3):
        c.fill_(5.0)
        y.fill_(5.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert bool(((c - c_want).abs() <= tol).all()), f"hyb replay {k}: {(c - c_want).abs().max().item():.3e}"
        # bit-equal except in the few tiles that are cut into units and meet in atomics
        assert torch.allclose(y, y_want, rtol=1e-6, atol=1e-6), f"rgms replay {k}"
        assert float((y != y_want).float().mean()) < 0.01


def test_graph_tcspmm_with_plan(dev):
    """TC-SpMM with fp16 output: the plan and its memory for partial tiles exist after the eager
    first call, so the three launches of a later call can be recorded."""
    g = datasets.config2()
    gptr, tiles, mask = st.condense(g["indptr"], g["indices"], 32, 16)
    mb, nnzb, feat = len(gptr) - 1, tiles.shape[0], 64
    t = lambda v: torch.from_numpy(np.ascontiguousarray(v)).to(dev)
    a, b = t(mask.astype(np.float16).ravel()), torch.randn(g["n"] * feat, device=dev).half()
    gp, ti = t(gptr), t(tiles.ravel())
    f = ops.build_tcspmm(mb, nnzb, feat, 32, 16, g["n"], torch.float16)
    want = torch.empty(mb * 32 * feat, dtype=torch.float16, device=dev)
    f(a, b, want, gp, ti)  # makes the plan
    torch.cuda.synchronize()
    c = torch.zeros_like(want)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        f(a, b, c, gp, ti)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        f(a, b, c, gp, ti)
    _replays(dev, graph, c, want, lambda: c.fill_(1.0))
