"""The entry point that allocates nothing (stir_hyb_spmm_f32_noalloc) against the plan-based pair
it is a variant of (stir_hyb_plan_create + stir_hyb_spmm_f32), both called through the C ABI, and
against the oracle's CSR product of the matrix the format was made from.

Two calls in a row on one GPU, the second with a smaller input, so that descriptors left in the
library's fixed device array by the first call would show.  Buckets that store (one partition,
all but the last bucket) must agree bit for bit; buckets that add with atomics agree within the
fp32 bar, |difference| <= 1e-5 * sum |a||x| (the order of the atomic adds differs between runs).
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
import sparsetir_amd as st
from sparsetir_amd import _lib
from helpers import random_csr

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def _decompose(dev, m, n, nnz, parts, buckets, seed):
    indptr, indices = random_csr(m, n, nnz, seed, skew=1.2)
    t = lambda a: torch.from_numpy(a).to(dev)
    vals = torch.rand(len(indices), device=dev, generator=torch.Generator(device=dev).manual_seed(seed)) + 0.5
    rows, cols, mask, avals = st.column_part_hyb(m, n, t(indptr), t(indices), parts, buckets, values=vals)
    A, R, C, nrows = [], [], [], []
    for p in range(parts):
        for b in range(len(buckets)):
            A.append(avals[p][b].reshape(-1).contiguous())
            R.append(rows[p][b].contiguous())
            C.append(cols[p][b].reshape(-1).contiguous())
            nrows.append(int(rows[p][b].shape[0]))
    return indptr, indices, vals, A, R, C, nrows


def _both_ways(dev, m, n, feat, parts, buckets, A, R, C, nrows, x):
    L = _lib.lib()
    nb = len(buckets)
    widths = (ctypes.c_int32 * nb)(*buckets)
    counts = (ctypes.c_int64 * len(nrows))(*nrows)
    tab = lambda ts: _lib.ptr_table([t.data_ptr() if t.numel() else 0 for t in ts])
    ta, tr, tc = tab(A), tab(R), tab(C)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    # the existing pair
    plan = ctypes.c_void_p()
    _lib.check(L.stir_hyb_plan_create(ctypes.byref(plan), m, n, parts, nb, widths, counts, ta, tr, tc))
    want = torch.zeros(m * feat, device=dev)
    _lib.check(L.stir_hyb_spmm_f32(plan, feat, vp(x), vp(want), stream))
    torch.cuda.synchronize()
    _lib.check(L.stir_hyb_plan_destroy(plan))
    # the entry point under test
    got = torch.zeros(m * feat, device=dev)
    _lib.check(L.stir_hyb_spmm_f32_noalloc(m, n, parts, nb, widths, counts, ta, tr, tc, feat, vp(x), vp(got), stream))
    torch.cuda.synchronize()
    return got, want


def _compare(dev, got, want, m, feat, indptr, vals, x, R, nrows, parts, nb, what):
    # magnitude of the summed terms per output element: sum_e |a_e| |x[col_e, f]| <= deg * 1.5 * max|x|
    deg = torch.from_numpy(np.diff(indptr).astype(np.float32)).to(dev)
    tol = (RTOL * 1.5 * float(x.abs().max()) * deg.clamp(min=1.0)).repeat_interleave(feat)
    assert bool(((got - want).abs() <= tol).all()), f"{what}: worst {float((got - want).abs().max()):.3e}"
    if parts == 1:
        # rows written by storing buckets only (not fed by the last bucket) are identical
        fed_by_last = torch.zeros(m, dtype=torch.bool, device=dev)
        if nrows[nb - 1]:
            fed_by_last[R[nb - 1].long()] = True
        keep = (~fed_by_last).repeat_interleave(feat)
        assert torch.equal(got[keep], want[keep]), what


@pytest.mark.parametrize("parts,buckets,feat", [
    (1, [1, 2, 4, 8, 16, 32], 128),            # storing buckets + an adding last bucket
    (2, [1, 2, 4, 8, 16, 32, 64, 128, 256, 512], 64),
    (16, [1, 2, 4, 8, 16, 32], 32),            # 96 buckets: three descriptor launches
    (3, [2, 3, 7], 20),                        # row mode and the kernel for any feature width
])
def test_noalloc_matches_plan_based_entry_point_twice(dev, parts, buckets, feat):
    big = (6000, 5000, 150000)
    small = (700, 900, 6000)   # the second call is smaller: fewer rows, fewer non-empty buckets
    for call, (m, n, nnz) in enumerate((big, small)):
        indptr, indices, vals, A, R, C, nrows = _decompose(dev, m, n, nnz, parts, buckets, seed=31 + call)
        x = torch.randn(n * feat, device=dev, generator=torch.Generator(device=dev).manual_seed(call))
        got, want = _both_ways(dev, m, n, feat, parts, buckets, A, R, C, nrows, x)
        _compare(dev, got, want, m, feat, indptr, vals, x, R, nrows, parts, len(buckets), f"call {call}")
        # and the oracle: C = A @ X from the CSR arrays the decomposition was made from
        ref = torch.from_numpy(oracle.csrmm(vals.cpu().numpy(), x.cpu().numpy(), indptr, indices, feat)).to(dev)
        _compare(dev, got, ref.reshape(-1), m, feat, indptr, vals, x, R, nrows, 0, len(buckets), f"call {call} vs oracle")


def test_noalloc_rejects_more_buckets_than_the_fixed_array_holds(dev):
    L = _lib.lib()
    parts, nb = 1025, 1
    k = parts * nb
    one = torch.ones(1, device=dev)
    idx = torch.zeros(1, dtype=torch.int32, device=dev)
    widths = (ctypes.c_int32 * nb)(1)
    counts = (ctypes.c_int64 * k)(*([1] * k))
    tab = lambda t: _lib.ptr_table([t.data_ptr()] * k)
    x = torch.zeros(4 * k, device=dev)
    y = torch.zeros(4, device=dev)
    rc = L.stir_hyb_spmm_f32_noalloc(1, k, parts, nb, widths, counts, tab(one), tab(idx), tab(idx), 4,
                                     ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(y.data_ptr()), None)
    assert rc == -1
    assert b"at most 1024" in L.stir_last_error()
    assert bool((y == 0).all())


def test_noalloc_inside_a_captured_graph(dev):
    """What the entry point is for: a call recorded into a HIP graph (after one eager call on the
    device, which looks up the fixed array's address -- that first call must happen outside a
    capture).  The graph is replayed twice; between the replays an eager call with another, smaller
    operator overwrites the descriptors in the fixed array, so the second replay only gives the
    right sums if the recorded fill kernels write them again.  Every replay is compared with the
    plan-based pair."""
    L = _lib.lib()
    feat, parts, buckets = 64, 2, [1, 2, 4, 8, 16, 32]
    nb = len(buckets)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    tab = lambda ts: _lib.ptr_table([t.data_ptr() if t.numel() else 0 for t in ts])
    widths = (ctypes.c_int32 * nb)(*buckets)

    def operator(m, n, nnz, seed):
        indptr, indices, vals, A, R, C, nrows = _decompose(dev, m, n, nnz, parts, buckets, seed=seed)
        x = torch.randn(n * feat, device=dev, generator=torch.Generator(device=dev).manual_seed(seed))
        counts = (ctypes.c_int64 * len(nrows))(*nrows)
        return dict(m=m, n=n, indptr=indptr, vals=vals, A=A, R=R, C=C, nrows=nrows, x=x, counts=counts,
                    tabs=(tab(A), tab(R), tab(C)))

    def launch(op, out):
        ta, tr, tc = op["tabs"]
        _lib.check(L.stir_hyb_spmm_f32_noalloc(op["m"], op["n"], parts, nb, widths, op["counts"], ta, tr, tc, feat,
                                               vp(op["x"]), vp(out),
                                               ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))

    def expected(op):
        ta, tr, tc = op["tabs"]
        plan = ctypes.c_void_p()
        _lib.check(L.stir_hyb_plan_create(ctypes.byref(plan), op["m"], op["n"], parts, nb, widths, op["counts"], ta, tr, tc))
        want = torch.zeros(op["m"] * feat, device=dev)
        _lib.check(L.stir_hyb_spmm_f32(plan, feat, vp(op["x"]), vp(want),
                                       ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        _lib.check(L.stir_hyb_plan_destroy(plan))
        return want

    big, small = operator(5000, 4000, 120000, 51), operator(600, 800, 5000, 52)
    want_big, want_small = expected(big), expected(small)
    out_big = torch.zeros(big["m"] * feat, device=dev)
    out_small = torch.zeros(small["m"] * feat, device=dev)
    launch(big, out_big)  # eager: the first call on this device
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch(big, out_big)
    for replay in range(2):
        out_big.zero_()
        graph.replay()
        torch.cuda.synchronize()
        _compare(dev, out_big, want_big, big["m"], feat, big["indptr"], big["vals"], big["x"], big["R"], big["nrows"],
                 parts, nb, f"replay {replay}")
        # another operator's descriptors go into the fixed array
        out_small.zero_()
        launch(small, out_small)
        torch.cuda.synchronize()
        _compare(dev, out_small, want_small, small["m"], feat, small["indptr"], small["vals"], small["x"], small["R"],
                 small["nrows"], parts, nb, f"eager call after replay {replay}")
