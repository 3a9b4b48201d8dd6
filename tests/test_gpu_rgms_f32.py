"""GPU parity of the fp32 RGMS kernels (ELL3D buckets and CSF traversal, W[r, fo, fi]) against
the oracle and the float64 closed form.  Tolerance: rtol 1e-5 on the result plus 1e-5 of the sum
of term magnitudes (the kernel sums a row's X rows before multiplying by W, and adds rows into Y
with atomics, so the order of the fp32 additions differs from the oracle's)."""
import numpy as np
import pytest
import torch

import oracle
import sparsetir_amd as st
from sparsetir_amd import datasets, ops
from helpers import random_csf, rgms_f64

pytestmark = pytest.mark.gpu


def _t(dev, a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _check(got, want64, scale64, ref, what):
    err = np.abs(got - want64)
    assert np.all(err <= 1e-5 * np.abs(want64) + 1e-5 * scale64 + 1e-30), f"{what}: worst {err.max():.3e}"
    assert np.all(np.abs(got - ref) <= 1e-5 * np.abs(ref) + 2e-5 * scale64 + 1e-30), f"{what}: vs oracle"


def _closed_forms(csf, a, x, w, m):
    wt = np.ascontiguousarray(w.transpose(0, 2, 1))
    return rgms_f64(*csf, a, x, wt, m), rgms_f64(*csf, np.abs(a), np.abs(x), np.abs(wt), m)


@pytest.mark.parametrize("fin,fout", [(32, 32), (8, 12), (4, 4), (20, 40), (64, 96), (128, 32), (16, 70)])
def test_rgms_csf_f32(dev, fin, fout):
    R, n = 6, 300
    csf = random_csf(R, n, 1500, seed=fin + fout)
    rng = np.random.default_rng(fin)
    x = rng.standard_normal((n, fin), dtype=np.float32)
    w = rng.standard_normal((R, fout, fin), dtype=np.float32) * 0.1
    a = (0.5 + rng.random(len(csf[3]), dtype=np.float32))
    a[::7] = 0.0  # zero-weight edges add nothing
    f = ops.build_rgms_csf(n, n, R, fin, fout, len(csf[1]), len(csf[3]))
    y = torch.zeros(n * fout, dtype=torch.float32, device=dev)
    f(_t(dev, a), _t(dev, w.ravel()), _t(dev, x.ravel()), y, *[_t(dev, c) for c in csf])
    torch.cuda.synchronize()
    want, scale = _closed_forms(csf, a, x, w, n)
    _check(y.cpu().numpy().reshape(n, fout), want, scale, oracle.rgms_csf_f32(a, w, x, *csf, n), f"csf {fin}x{fout}")


@pytest.mark.parametrize("deterministic", [False, True])
def test_rgms_csf_f32_long_row_and_empty_relations(dev, deterministic):
    """One stored row with thousands of edges (several 64-edge passes of one tile), relations
    without rows, a single stored row in the last relation.  (3005 edges: both settings run the
    atomic kernel; the deterministic one through a plan.)"""
    n, fin, fout, R = 5000, 32, 32, 5
    rng = np.random.default_rng(3)
    long_cols = np.sort(rng.choice(n, 3000, replace=False)).astype(np.int32)
    p0 = np.asarray([0, 0, 3, 3, 3, 4], np.int32)
    i0 = np.asarray([7, 9, 4000, 9], np.int32)
    p1 = np.asarray([0, 2, 3002, 3003, 3005], np.int32)
    i1 = np.concatenate([[1, 2], long_cols, [0], [4999, 17]]).astype(np.int32)
    csf = (p0, i0, p1, i1)
    x = rng.standard_normal((n, fin), dtype=np.float32)
    w = rng.standard_normal((R, fout, fin), dtype=np.float32) * 0.1
    a = rng.standard_normal(len(i1)).astype(np.float32)
    f = ops.build_rgms_csf(n, n, R, fin, fout, len(i0), len(i1), deterministic=deterministic)
    y = torch.zeros(n * fout, dtype=torch.float32, device=dev)
    f(_t(dev, a), _t(dev, w.ravel()), _t(dev, x.ravel()), y, *[_t(dev, c) for c in csf])
    torch.cuda.synchronize()
    want, scale = _closed_forms(csf, a, x, w, n)
    _check(y.cpu().numpy().reshape(n, fout), want, scale, oracle.rgms_csf_f32(a, w, x, *csf, n), "long row")


def test_rgms_csf_f32_empty(dev):
    f = ops.build_rgms_csf(10, 10, 3, 8, 8, 0, 0)
    z = lambda dt, k=0: torch.zeros(k, dtype=dt, device=dev)
    y = torch.full((80,), 3.0, dtype=torch.float32, device=dev)
    f(z(torch.float32), z(torch.float32, 3 * 64), z(torch.float32, 80), y, z(torch.int32, 4), z(torch.int32),
      z(torch.int32, 1), z(torch.int32))
    torch.cuda.synchronize()
    assert torch.all(y == 3.0)


def _run_ell3d(dev, csf, n, x, w, group, buckets, weighted, seed=0, deterministic=True):
    R, fout, fin = w.shape
    rows_bkt = [max(1, group // b) for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rows_bkt, buckets)
    rng = np.random.default_rng(seed)
    triples, mids, bk = [], [], []
    for b in range(len(buckets)):
        a = mask[b].astype(np.float32)
        if weighted:
            a = a * (0.5 + rng.random(a.shape, dtype=np.float32))
        mid = np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[b]))
        bk.append((a, rows[b], cols[b], mid))
        triples += [_t(dev, a.ravel()), _t(dev, rows[b].ravel()), _t(dev, cols[b].ravel())]
        mids.append(_t(dev, mid))
    f = ops.build_rgms_f32(n, n, R, fin, fout, rows_bkt, buckets, [c.shape[0] for c in cols],
                           deterministic=deterministic)
    y = torch.zeros(n * fout, dtype=torch.float32, device=dev)
    f(_t(dev, w.ravel()), _t(dev, x.ravel()), y, *triples, *mids)
    torch.cuda.synchronize()
    return y.cpu().numpy().reshape(n, fout), bk


@pytest.mark.parametrize("group,buckets,fin,fout,weighted", [
    (32, [1, 2, 4, 8, 16], 32, 32, False),     # the reference's composable configuration
    (256, [1, 2, 4, 8, 16], 32, 32, True),     # rb > 32: several tiles per group
    (16, [1, 2, 4], 16, 40, True),
    (12, [1, 3, 6], 48, 32, True),             # rb does not divide 32, cb not a power of two
    (64, [2, 64], 64, 96, False),
    (8, [1, 2], 4, 4, True),
])
def test_rgms_ell3d_f32(dev, group, buckets, fin, fout, weighted):
    R, n = 5, 300
    csf = random_csf(R, n, 900, seed=group)
    rng = np.random.default_rng(group)
    x = rng.standard_normal((n, fin), dtype=np.float32)
    w = rng.standard_normal((R, fout, fin), dtype=np.float32) * 0.1
    got, bk = _run_ell3d(dev, csf, n, x, w, group, buckets, weighted)
    ref = oracle.rgms_ell3d_f32(w, x, bk, n)
    if not weighted:
        ones = np.ones(len(csf[3]), np.float32)
        want, scale = _closed_forms(csf, ones, x, w, n)
        _check(got, want, scale, ref, f"ell3d group={group}")
    else:
        scale = oracle.rgms_ell3d_f32(np.abs(w), np.abs(x), [(np.abs(a), r, c, m) for a, r, c, m in bk], n)
        assert np.all(np.abs(got - ref) <= 1e-5 * np.abs(ref) + 2e-5 * scale + 1e-30)


@pytest.mark.parametrize("deterministic", [False, True])
def test_rgms_f32_config5_reduced_both_forms_agree(dev, deterministic):
    cfg = datasets.config5(n=4000, num_rels=65, num_edges=40000)
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    n = cfg["n"]
    w = np.ascontiguousarray(cfg["w"].transpose(0, 2, 1))
    got, bk = _run_ell3d(dev, csf, n, cfg["x"], w, 32, cfg["buckets"], False, deterministic=deterministic)
    ones = np.ones(len(csf[3]), np.float32)
    want, scale = _closed_forms(csf, ones, cfg["x"], w, n)
    _check(got, want, scale, oracle.rgms_ell3d_f32(w, cfg["x"], bk, n), "config5 ell3d")
    f = ops.build_rgms_csf(n, n, 65, 32, 32, len(csf[1]), len(csf[3]), deterministic=deterministic)
    y = torch.zeros(n * 32, dtype=torch.float32, device=dev)
    f(_t(dev, ones), _t(dev, w.ravel()), _t(dev, cfg["x"].ravel()), y, *[_t(dev, c) for c in csf])
    torch.cuda.synchronize()
    _check(y.cpu().numpy().reshape(n, 32), want, scale, oracle.rgms_csf_f32(ones, w, cfg["x"], *csf, n), "config5 csf")



# ---- deterministic=True, from 8192 slots on: the destination-tiled kernel (an edge index by 64-row
# tile of Y, the (relation, row) pairs multiplied 16 at a time on the 16x16x4 fp32 instruction, no
# atomics: the same bits on every run)

@pytest.mark.parametrize("fin,fout,R,n", [
    (32, 32, 7, 1000),    # the RGCN layer's sizes; the last tile has 40 rows
    (20, 40, 3, 777),     # inputs and outputs that fill neither a k group nor an output tile
    (64, 64, 5, 640),     # two input halves per lane, four output tiles
    (48, 16, 40, 500),    # more relations than pairs in a product: most products hold one to three pairs
    (4, 4, 2, 129),
])
def test_rgms_f32_tiled_both_front_ends(dev, fin, fout, R, n):
    edges = 12000
    csf = random_csf(R, n, edges, seed=fin * 100 + fout)
    rng = np.random.default_rng(fin + R)
    x = rng.standard_normal((n, fin), dtype=np.float32)
    w = rng.standard_normal((R, fout, fin), dtype=np.float32) * 0.1
    a = (0.5 + rng.random(len(csf[3]), dtype=np.float32))
    a[::5] = 0.0
    assert len(csf[3]) >= 8192
    want, scale = _closed_forms(csf, a, x, w, n)
    # CSF front end, twice: the second call adds to Y, and both calls give the same bits
    f = ops.build_rgms_csf(n, n, R, fin, fout, len(csf[1]), len(csf[3]), deterministic=True)
    d = [_t(dev, a), _t(dev, w.ravel()), _t(dev, x.ravel())]
    d_csf = [_t(dev, c) for c in csf]
    y = torch.zeros(n * fout, dtype=torch.float32, device=dev)
    f(d[0], d[1], d[2], y, *d_csf)
    torch.cuda.synchronize()
    first = y.clone()
    _check(first.cpu().numpy().reshape(n, fout), want, scale, oracle.rgms_csf_f32(a, w, x, *csf, n), "tiled csf")
    y2 = torch.zeros_like(y)
    f(d[0], d[1], d[2], y2, *d_csf)
    f(d[0], d[1], d[2], y, *d_csf)
    torch.cuda.synchronize()
    assert torch.equal(y2, first)  # no atomics: the same sums in the same order
    assert np.all(np.abs(y.cpu().numpy().reshape(n, fout) - 2 * want) <= 2e-5 * np.abs(want) + 2e-5 * scale + 1e-30)
    assert f.plan_builds == 1
    # edge values rewritten in place are read by the next call (the plan holds their addresses)
    d[0].mul_(2.0)
    y3 = torch.zeros_like(y)
    f(d[0], d[1], d[2], y3, *d_csf)
    torch.cuda.synchronize()
    assert np.all(np.abs(y3.cpu().numpy().reshape(n, fout) - 2 * want) <= 2e-5 * np.abs(want) + 2e-5 * scale + 1e-30)
    # ELL3D front end on the same graph (weights 1)
    ones = np.ones(len(csf[3]), np.float32)
    want1, scale1 = _closed_forms(csf, ones, x, w, n)
    got, bk = _run_ell3d(dev, csf, n, x, w, 32, [1, 2, 4, 8, 16], False, deterministic=True)
    assert sum(b[0].size for b in bk) >= 8192
    _check(got, want1, scale1, oracle.rgms_ell3d_f32(w, x, bk, n), "tiled ell3d")
    again, _ = _run_ell3d(dev, csf, n, x, w, 32, [1, 2, 4, 8, 16], False, deterministic=True)
    assert np.array_equal(got, again)


def test_rgms_f32_tiled_hub_row_and_empty_relations(dev):
    """A destination row with 9000 edges of one relation (one pair whose edges a lane group walks
    four at a time), relations without rows, a tile of Y without edges, m != n."""
    m, n, fin, fout, R = 700, 9500, 32, 32, 6
    rng = np.random.default_rng(5)
    rows_per_rel = [np.asarray([3, 650], np.int32), np.zeros(0, np.int32), np.asarray([3, 4, 5, 699], np.int32),
                    np.zeros(0, np.int32), np.zeros(0, np.int32), np.asarray([650], np.int32)]
    counts = {(0, 3): 9000, (0, 650): 40, (2, 3): 5, (2, 4): 1, (2, 5): 70, (2, 699): 17, (5, 650): 300}
    p0, i0, p1, i1 = [0], [], [0], []
    for r in range(R):
        for row in rows_per_rel[r]:
            i0.append(int(row))
            cols = np.sort(rng.choice(n, counts[(r, int(row))], replace=False))
            i1.extend(cols.tolist())
            p1.append(len(i1))
        p0.append(len(i0))
    csf = tuple(np.asarray(v, np.int32) for v in (p0, i0, p1, i1))
    assert len(csf[3]) >= 8192
    x = rng.standard_normal((n, fin), dtype=np.float32)
    w = rng.standard_normal((R, fout, fin), dtype=np.float32) * 0.1
    a = rng.standard_normal(len(csf[3])).astype(np.float32)
    f = ops.build_rgms_csf(m, n, R, fin, fout, len(csf[1]), len(csf[3]), deterministic=True)
    y = torch.zeros(m * fout, dtype=torch.float32, device=dev)
    f(_t(dev, a), _t(dev, w.ravel()), _t(dev, x.ravel()), y, *[_t(dev, c) for c in csf])
    torch.cuda.synchronize()
    want, scale = _closed_forms(csf, a, x, w, m)
    got = y.cpu().numpy().reshape(m, fout)
    _check(got, want, scale, oracle.rgms_csf_f32(a, w, x, *csf, m), "hub row")
    untouched = np.setdiff1d(np.arange(m), [3, 4, 5, 650, 699])
    assert np.all(got[untouched] == 0)


def test_rgms_f32_tiled_rejects_bad_ids(dev):
    """Row, column and relation ids are checked when the index of the deterministic form is built."""
    from sparsetir_amd._lib import SparseTIRError
    R, n, fin, fout = 3, 500, 32, 32
    csf = list(random_csf(R, n, 30000, seed=77))
    assert len(csf[3]) >= 8192  # below that the kernel with atomics runs, which reads no index ahead
    x = torch.zeros(n * fin, device=dev)
    w = torch.zeros(R * fout * fin, device=dev)
    a = torch.ones(len(csf[3]), device=dev)
    bad_cols = csf[3].copy()
    bad_cols[123] = n
    f = ops.build_rgms_csf(n, n, R, fin, fout, len(csf[1]), len(csf[3]), deterministic=True)
    with pytest.raises(SparseTIRError, match="column id"):
        f(a, w, x, torch.zeros(n * fout, device=dev), _t(dev, csf[0]), _t(dev, csf[1]), _t(dev, csf[2]), _t(dev, bad_cols))
    bad_rows = csf[1].copy()
    bad_rows[7] = n + 5
    with pytest.raises(SparseTIRError, match="row id"):
        f(a, w, x, torch.zeros(n * fout, device=dev), _t(dev, csf[0]), _t(dev, bad_rows), _t(dev, csf[2]), _t(dev, csf[3]))


def test_packed_rgms_f32_static_structure_sums_in_tiles(dev):
    """Under "sparsetir.static_structure"(1) the PackedFuncs sparsetir.rgms_f32 and
    sparsetir.rgms_csf keep an edge index per set of arrays and sum every tile of Y on chip: the
    closed form within tolerance, the same bits on every call, one plan per function for any
    number of calls; edge values rewritten in place are read by the next call; without the promise
    the same calls build no index."""
    from sparsetir_amd import packed
    promise = packed.get_global_func("sparsetir.static_structure")
    inval = packed.get_global_func("sparsetir.invalidate_plans")
    R, n, fin, fout, group, buckets = 7, 3000, 32, 32, 32, [1, 2, 4, 8, 16]
    csf = random_csf(R, n, 40000, seed=77)
    rng = np.random.default_rng(77)
    x = rng.standard_normal((n, fin), dtype=np.float32)
    w = rng.standard_normal((R, fout, fin), dtype=np.float32) * 0.1
    a = 0.5 + rng.random(len(csf[3]), dtype=np.float32)
    want, scale = _closed_forms(csf, a, x, w, n)
    ones = np.ones(len(csf[3]), np.float32)
    want1, scale1 = _closed_forms(csf, ones, x, w, n)
    rb = [group // b for b in buckets]
    iptr, rows, cols, mask = st.csf_to_ell3d(*csf, rb, buckets)
    triples, mids = [], []
    for k in range(len(buckets)):
        triples += [_t(dev, mask[k].astype(np.float32).ravel()), _t(dev, rows[k].ravel()), _t(dev, cols[k].ravel())]
        mids.append(_t(dev, np.repeat(np.arange(R, dtype=np.int32), np.diff(iptr[k]))))
    assert sum(c.size for c in cols) >= 8192
    dw, dx, da = _t(dev, w.ravel()), _t(dev, x.ravel()), _t(dev, a)
    d_csf = [_t(dev, c) for c in csf]
    f_ell, f_csf = packed.get_global_func("sparsetir.rgms_f32"), packed.get_global_func("sparsetir.rgms_csf")

    def run_ell():
        y = torch.zeros(n * fout, device=dev)
        f_ell(dw, dx, y, *triples, *mids, fin, fout)
        torch.cuda.synchronize()
        return y

    def run_csf():
        y = torch.zeros(n * fout, device=dev)
        f_csf(da, dw, dx, y, *d_csf, fin, fout)
        torch.cuda.synchronize()
        return y

    inval()
    promise(1)
    try:
        before = packed.plan_builds()
        e0, e1, c0, c1 = run_ell(), run_ell(), run_csf(), run_csf()
        assert packed.plan_builds() == before + 2
        assert torch.equal(e0, e1) and torch.equal(c0, c1)
        _check(e0.cpu().numpy().reshape(n, fout), want1, scale1, oracle.rgms_csf_f32(ones, w, x, *csf, n), "packed ell3d")
        _check(c0.cpu().numpy().reshape(n, fout), want, scale, oracle.rgms_csf_f32(a, w, x, *csf, n), "packed csf")
        da.mul_(2.0)
        c2 = run_csf()
        assert np.all(np.abs(c2.cpu().numpy().reshape(n, fout) - 2 * want) <= 2e-5 * np.abs(want) + 2e-5 * scale + 1e-30)
        assert packed.plan_builds() == before + 2
        da.mul_(0.5)
        promise(0)  # the plans made under the promise go away
        before = packed.plan_builds()
        c3 = run_csf()
        assert packed.plan_builds() == before  # stateless again
        _check(c3.cpu().numpy().reshape(n, fout), want, scale, oracle.rgms_csf_f32(a, w, x, *csf, n), "packed csf, atomics")
    finally:
        promise(0)
        inval()
