"""GPU parity of CSR row-split SpMM and hyb SpMM (through the C ABI) against the CPU oracle.

Tolerance: fp32, |got - want| <= 1e-5 * (|A| @ |X|) elementwise, i.e. relative 1e-5 measured
against the magnitude of the terms that are summed (an rtol-only check against the result is
meaningless where the terms cancel); the float64 closed form is the reference value.
"""
import numpy as np
import pytest
import torch

import oracle
import sparsetir_amd as st
from sparsetir_amd import datasets, ops
from sparsetir_amd._lib import SparseTIRError
from helpers import random_csr, spmm_f64

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def _check(got, indptr, indices, vals, x, what):
    want = spmm_f64(indptr, indices, vals, x)
    scale = spmm_f64(indptr, indices, np.abs(vals), np.abs(x))
    err = np.abs(got.astype(np.float64) - want)
    bad = err > RTOL * scale + 1e-30
    assert not bad.any(), f"{what}: {bad.sum()} elements off, worst {err.max():.3e}"


def _run_csr(dev, indptr, indices, vals, x, feat, fill=None):
    m, n = len(indptr) - 1, x.shape[0]
    f = ops.build_csrmm(m, n, feat, len(indices))
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    c = torch.full((m * feat,), float("nan") if fill is None else fill, dtype=torch.float32, device=dev)
    f(t(vals), t(x.ravel()), c, t(indptr), t(indices))
    torch.cuda.synchronize()
    return c.cpu().numpy().reshape(m, feat)


def test_csr_spmm_config1(dev):
    g = datasets.config1()
    got = _run_csr(dev, g["indptr"], g["indices"], g["values"], g["x"], g["feat"])
    _check(got, g["indptr"], g["indices"], g["values"], g["x"], "config1")
    # and against the C restatement of the reference's serial loop nest
    ref = oracle.csrmm(g["values"], g["x"], g["indptr"], g["indices"], g["feat"])
    scale = spmm_f64(g["indptr"], g["indices"], g["values"], np.abs(g["x"]))
    assert np.all(np.abs(got - ref) <= 2 * RTOL * scale)


@pytest.mark.parametrize("feat", [32, 64, 128, 256, 512, 48, 20, 1, 4, 16, 96, 384, 260, 516])
def test_csr_spmm_feature_widths(dev, feat):
    m, n = 1003, 777
    indptr, indices = random_csr(m, n, 30000, feat, skew=1.2)
    rng = np.random.default_rng(feat)
    vals = rng.random(len(indices), dtype=np.float32)
    x = rng.standard_normal((n, feat), dtype=np.float32)
    got = _run_csr(dev, indptr, indices, vals, x, feat)
    assert np.all(got[np.diff(indptr) == 0] == 0.0)  # rows without nonzeros are zeroed
    _check(got, indptr, indices, vals, x, f"feat={feat}")


def test_csr_spmm_edge_shapes(dev):
    for m, n, nnz in [(1, 1, 1), (5, 3, 0), (0, 4, 0), (130, 2, 200)]:
        indptr, indices = random_csr(m, n, nnz, 3)
        rng = np.random.default_rng(0)
        vals = rng.random(len(indices), dtype=np.float32)
        x = rng.standard_normal((n, 64), dtype=np.float32)
        got = _run_csr(dev, indptr, indices, vals, x, 64)
        if m:
            _check(got, indptr, indices, vals, x, f"shape {(m, n, nnz)}")


def test_csr_spmm_long_row(dev):
    # one row holding every column (the power-law tail)
    m, n, feat = 9, 5000, 128
    indptr = np.asarray([0, 3, n + 3] + [n + 3] * (m - 2), np.int32)
    indices = np.concatenate([[1, 5, 9], np.arange(n)]).astype(np.int32)
    rng = np.random.default_rng(5)
    vals = rng.random(len(indices), dtype=np.float32)
    x = rng.standard_normal((n, feat), dtype=np.float32)
    got = _run_csr(dev, indptr, indices, vals, x, feat)
    _check(got, indptr, indices, vals, x, "long row")


@pytest.mark.parametrize("feat", [32, 128, 512, 96])
def test_csr_spmm_hub_rows_are_split(dev, feat):
    """Enough nonzeros for the second launch that adds up rows longer than 64 entries in
    256-entry pieces: hub rows of different lengths (piece boundaries inside, at the start and at
    the end of rows), rows just below and above the limit, the output pre-filled with NaN."""
    m, n = 4500, 40000
    rng = np.random.default_rng(feat)
    deg = rng.integers(0, 120, m)
    for row, d in [(0, 257), (1, 256), (2, 2049), (3, 64), (4, 65), (5, 63), (7, 30000), (8, 2560), (1500, 12345),
                   (m - 1, 5000)]:
        deg[row] = d
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    assert indptr[-1] >= 1 << 18
    indices = np.concatenate([np.sort(rng.choice(n, d, replace=False)) for d in deg]).astype(np.int32)
    vals = (rng.random(len(indices), dtype=np.float32) - 0.3)
    x = rng.standard_normal((n, feat), dtype=np.float32)
    got = _run_csr(dev, indptr, indices, vals, x, feat)
    _check(got, indptr, indices, vals, x, f"hub rows feat={feat}")


@pytest.mark.parametrize("feat", [4, 8, 12, 32, 40, 64, 128])
@pytest.mark.parametrize("split", [False, True])
def test_csr_spmm_lane_group_per_row(dev, feat, split):
    """Feature rows narrower than a wavefront: a wavefront owns several rows, one per lane group.
    Row lengths around every limit of that kernel -- 0, 1, the group width G, 2G (the longest row a
    group takes alone), 2G + 1 (left to the whole wavefront), 64, 65, 256, 257 and a hub row --
    next to each other in one wavefront's rows, a row count that is no multiple of the rows per
    wavefront, and (split) enough nonzeros for the second launch that adds up rows above 64."""
    G = next(g for g in (4, 8, 16, 32) if 4 * g >= feat)
    rng = np.random.default_rng(100 * feat + split)
    special = [0, 1, G - 1, G, G + 1, 2 * G, 2 * G + 1, 3 * G, 63, 64, 65, 255, 256, 257, 0, 1500]
    # 128 features take this kernel below 16 nonzeros per row on average
    m, n = (64 * 300 + 5 if feat == 128 and split else 64 * 37 + 5), 9000
    deg = rng.integers(0, 12, m)
    for k, d in enumerate(special):
        deg[k] = d                              # all in the first wavefronts, side by side
        deg[(k * 97 + 300) % m] = d             # and scattered
    deg[m - 1] = 2 * G + 1
    if split:
        deg[m // 2] = 6000
        deg[m // 3] = n
        big = np.nonzero(deg <= 12)[0]
        while deg.sum() < (1 << 18) + 1000:     # rows of 250 .. 400 until the second launch is on
            deg[rng.choice(big)] = rng.integers(250, 400)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    assert (indptr[-1] >= 1 << 18) == split
    assert feat != 128 or indptr[-1] < 16 * m
    indices = np.concatenate([np.sort(rng.choice(n, d, replace=False)) for d in deg]).astype(np.int32)
    vals = rng.random(len(indices), dtype=np.float32) - 0.4
    x = rng.standard_normal((n, feat), dtype=np.float32)
    got = _run_csr(dev, indptr, indices, vals, x, feat)
    assert np.all(got[deg == 0] == 0.0)
    _check(got, indptr, indices, vals, x, f"lane group per row, feat={feat}, split={split}")


def test_csr_spmm_argument_checks(dev):
    f = ops.build_csrmm(4, 4, 32, 3)
    z = lambda k, dt=torch.float32: torch.zeros(k, dtype=dt, device=dev)
    good = [z(3), z(128), z(128), z(5, torch.int32), z(3, torch.int32)]
    f(*good)
    with pytest.raises(SparseTIRError, match="num_args"):
        f(*good[:4])
    with pytest.raises(SparseTIRError, match="dtype"):
        f(good[0], good[1], good[2], z(5, torch.int64), good[4])
    with pytest.raises(SparseTIRError, match="shape"):
        f(good[0], z(127), good[2], good[3], good[4])
    with pytest.raises(SparseTIRError, match="ndim"):
        f(good[0], z(128).reshape(4, 32), good[2], good[3], good[4])
    with pytest.raises(SparseTIRError, match="device"):
        f(good[0].cpu(), good[1], good[2], good[3], good[4])


# ------------------------------------------------------------------------------- hyb

def _hyb_setup(dev, indptr, indices, m, n, parts, buckets, weighted, seed, device_format=False):
    if device_format:
        ti = lambda a: torch.from_numpy(a).to(dev)
        rows, cols, mask = st.column_part_hyb(m, n, ti(indptr), ti(indices), parts, buckets)
        tonp = lambda a: a.cpu().numpy()
        rows = [[tonp(a) for a in p] for p in rows]
        cols = [[tonp(a) for a in p] for p in cols]
        mask = [[tonp(a) for a in p] for p in mask]
    else:
        rows, cols, mask = st.column_part_hyb(m, n, indptr, indices, parts, buckets)
    rng = np.random.default_rng(seed)
    triples_np = []
    for p in range(parts):
        for b in range(len(buckets)):
            a = mask[p][b].astype(np.float32)
            if weighted:
                a = a * rng.random(a.shape, dtype=np.float32)
            triples_np.append((a, rows[p][b], cols[p][b]))
    return triples_np


def _run_hyb(dev, m, n, feat, parts, buckets, triples_np, x):
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    f = ops.build_hyb_csrmm(m, n, feat, parts, buckets, [len(r) for _, r, _ in triples_np])
    args = []
    for a, r, c in triples_np:
        args += [t(a.ravel()), t(r), t(c.ravel())]
    cdev = torch.zeros(m * feat, dtype=torch.float32, device=dev)
    f(t(x.ravel()), cdev, *args)
    torch.cuda.synchronize()
    return cdev.cpu().numpy().reshape(m, feat), (f, args)


def _hyb_as_coo(triples_np):
    """(row, col, value) of every slot with a nonzero weight, as a CSR for the float64 form."""
    rr, cc, vv = [], [], []
    for a, r, c in triples_np:
        if len(r) == 0:
            continue
        sel = a != 0
        rr.append(np.repeat(r[:, None], c.shape[1], 1)[sel])
        cc.append(c[sel])
        vv.append(a[sel])
    return np.concatenate(rr), np.concatenate(cc), np.concatenate(vv)


@pytest.mark.parametrize("feat", [32, 64, 128, 256, 512, 96, 7, 4, 16, 40, 384])
@pytest.mark.parametrize("parts,buckets", [(1, [1, 2, 4, 8, 16, 32]), (2, [1, 2, 4, 8, 16, 32, 64, 128, 256, 512]),
                                           (4, [2, 3, 7]), (3, [1]),
                                           # more than four partitions: every bucket of the single launch adds
                                           # with atomics; 16 x [1..32] is the reference's own setting for its
                                           # largest graph (examples/spmm/bench_spmm.py:233-253)
                                           (8, [1, 2, 4, 8, 16, 32, 64]), (16, [1, 2, 4, 8, 16, 32]),
                                           (5, [2, 5, 300])])
def test_hyb_spmm_matches_oracle(dev, feat, parts, buckets):
    m = n = 3001
    indptr, indices = random_csr(m, n, 60000, 17, skew=1.3)
    triples = _hyb_setup(dev, indptr, indices, m, n, parts, buckets, weighted=True, seed=feat)
    x = np.random.default_rng(feat).standard_normal((n, feat), dtype=np.float32)
    got, _ = _run_hyb(dev, m, n, feat, parts, buckets, triples, x)
    want = oracle.hyb_spmm(m, feat, x, triples, parts)
    import scipy.sparse as sp
    r, c, v = _hyb_as_coo(triples)
    scale = sp.csr_matrix((np.abs(v).astype(np.float64), (r, c)), shape=(m, n)) @ np.abs(x).astype(np.float64)
    exact = sp.csr_matrix((v.astype(np.float64), (r, c)), shape=(m, n)) @ x.astype(np.float64)
    assert np.all(np.abs(got - exact) <= RTOL * scale + 1e-30)
    assert np.all(np.abs(got - want) <= 2 * RTOL * scale + 1e-30)


def test_hyb_spmm_store_semantics_of_non_atomic_buckets(dev):
    """With one column partition every bucket but the last stores (overwrites) its rows and
    the last one accumulates (examples/spmm/bench_spmm.py:170-177): calling the operator
    twice on the same C doubles only the rows of the last bucket."""
    m = n = 500
    feat, buckets = 64, [1, 2, 4]
    indptr, indices = random_csr(m, n, 4000, 3, skew=1.0)
    triples = _hyb_setup(dev, indptr, indices, m, n, 1, buckets, weighted=False, seed=0)
    x = np.random.default_rng(0).standard_normal((n, feat), dtype=np.float32)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    f = ops.build_hyb_csrmm(m, n, feat, 1, buckets, [len(r) for _, r, _ in triples])
    args = []
    for a, r, c in triples:
        args += [t(a.ravel()), t(r), t(c.ravel())]
    cdev = torch.zeros(m * feat, dtype=torch.float32, device=dev)
    f(t(x.ravel()), cdev, *args)
    once = cdev.cpu().numpy().reshape(m, feat).copy()
    f(t(x.ravel()), cdev, *args)
    twice = cdev.cpu().numpy().reshape(m, feat)
    last_rows = np.unique(triples[-1][1])
    other = np.setdiff1d(np.arange(m), last_rows)
    assert np.array_equal(twice[other], once[other])
    assert np.allclose(twice[last_rows], 2 * once[last_rows], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("feat", [32, 64, 128, 256])
def test_hyb_spmm_config2_against_csr_kernel_and_oracle(dev, feat):
    g = datasets.config2()
    m, n, parts, buckets = g["m"], g["n"], g["num_col_parts"], g["buckets"]
    triples = _hyb_setup(dev, g["indptr"], g["indices"], m, n, parts, buckets, weighted=False, seed=0,
                         device_format=True)
    x = datasets.features(n, feat, seed=7)
    got, _ = _run_hyb(dev, m, n, feat, parts, buckets, triples, x)
    ones = np.ones(len(g["indices"]), np.float32)
    _check(got, g["indptr"], g["indices"], ones, x, "config2 hyb")
    csr = _run_csr(dev, g["indptr"], g["indices"], ones, x, feat)
    scale = spmm_f64(g["indptr"], g["indices"], ones, np.abs(x))
    assert np.all(np.abs(got - csr) <= 2 * RTOL * scale + 1e-30)
    want = oracle.hyb_spmm(m, feat, x, triples, parts)
    assert np.all(np.abs(got - want) <= 2 * RTOL * scale + 1e-30)


@pytest.mark.parametrize("where", ["same_bucket", "two_buckets", "with_last_bucket"])
def test_hyb_spmm_caller_built_arrays_sharing_output_rows(dev, where):
    """Arrays that ColumnPartHyb would not produce: inside one column partition an output row is
    fed by several ELL rows of buckets other than the last.  The reference adds every bucket
    atomically when there are several partitions (examples/spmm/bench_spmm.py:170-177), so the
    sums must still be complete (with 2-4 partitions the library may only drop the atomics when
    every such row has a single writer, which it checks when the plan is made)."""
    m, n, feat, parts, buckets = 64, 512, 128, 2, [2, 4, 8]
    rng = np.random.default_rng(3)
    nrows = 4096  # many ELL rows onto few output rows: lost updates would be certain without atomics
    def ell(width, count, row_ids):
        cols = rng.integers(0, n // 2, (count, width)).astype(np.int32)
        a = rng.random((count, width), dtype=np.float32) + 0.5
        return a, np.asarray(row_ids, np.int32), cols
    empty = lambda w: (np.zeros((0, w), np.float32), np.zeros(0, np.int32), np.zeros((0, w), np.int32))
    part0 = [empty(2), empty(4), empty(8)]
    if where == "same_bucket":
        part0[0] = ell(2, nrows, rng.integers(0, 8, nrows))
    elif where == "two_buckets":
        part0[0] = ell(2, nrows, np.arange(nrows) % m)
        part0[1] = ell(4, nrows, (np.arange(nrows) * 7) % m)
    else:
        part0[1] = ell(4, m, np.arange(m))
        part0[2] = ell(8, nrows, np.sort(rng.integers(0, m, nrows)))
    part1 = [ell(2, m, np.arange(m)), empty(4), ell(8, 10, np.arange(10))]
    part1 = [(a, r, c + n // 2) for a, r, c in part1]
    triples = part0 + part1
    x = rng.standard_normal((n, feat), dtype=np.float32)
    got, _ = _run_hyb(dev, m, n, feat, parts, buckets, triples, x)
    import scipy.sparse as sp
    r, c, v = _hyb_as_coo(triples)
    exact = sp.coo_matrix((v.astype(np.float64), (r, c)), shape=(m, n)).tocsr() @ x.astype(np.float64)
    scale = sp.coo_matrix((np.abs(v).astype(np.float64), (r, c)), shape=(m, n)).tocsr() @ np.abs(x).astype(np.float64)
    assert np.all(np.abs(got - exact) <= RTOL * scale + 1e-30)
    want = oracle.hyb_spmm(m, feat, x, triples, parts)
    assert np.all(np.abs(got - want) <= 2 * RTOL * scale + 1e-30)


def test_fused_launch_of_two_row_sums(dev):
    """The reference's one numeric unit test (tests/python/sparsetir/test_horizontal_fuse.py:177-215):
    two row-sum kernels, over a 128 x 128 and a 64 x 128 matrix, fused into one launch and compared
    with numpy at rtol = atol = 1e-5.  Here the two "kernels" are two ELL buckets of one fused hyb
    launch: the matrices' entries are the slot weights, every slot gathers a row of ones, and the
    buckets write disjoint output rows (the second one, as the last bucket, by adding)."""
    rng = np.random.default_rng(0)
    x_np = rng.random((128, 128), dtype=np.float32)
    y_np = rng.random((64, 128), dtype=np.float32)
    feat, n = 4, 256
    cols0 = np.tile(np.arange(128, dtype=np.int32), (128, 1))
    y_pad = np.concatenate([y_np, np.zeros((64, 128), np.float32)], axis=1)  # width 256, half of it padding
    cols1 = np.concatenate([np.tile(np.arange(128, 256, dtype=np.int32), (64, 1)), np.zeros((64, 128), np.int32)], axis=1)
    triples = [(x_np, np.arange(128, dtype=np.int32), cols0), (y_pad, np.arange(128, 192, dtype=np.int32), cols1)]
    ones = np.ones((n, feat), np.float32)
    got, _ = _run_hyb(dev, 192, n, feat, 1, [128, 256], triples, ones)
    for k in range(feat):
        np.testing.assert_allclose(got[:128, k], x_np.sum(axis=-1), rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(got[128:, k], y_np.sum(axis=-1), rtol=1e-5, atol=1e-5)


def test_hyb_plan_rejects_row_ids_out_of_range(dev):
    m, n, feat, parts, buckets = 16, 32, 32, 2, [1, 2]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    f = ops.build_hyb_csrmm(m, n, feat, parts, buckets, [1, 0, 0, 0])
    z = lambda k, dt: torch.zeros(k, dtype=dt, device=dev)
    args = [t(np.ones(1, np.float32)), t(np.asarray([m], np.int32)), z(1, torch.int32)]
    for _ in range(3):
        args += [z(0, torch.float32), z(0, torch.int32), z(0, torch.int32)]
    with pytest.raises(SparseTIRError, match="row index"):
        f(z(n * feat, torch.float32), z(m * feat, torch.float32), *args)


def test_hyb_spmm_empty_and_degenerate(dev):
    # no nonzeros at all: every bucket empty, C stays zero
    m = n = 10
    indptr = np.zeros(m + 1, np.int32)
    indices = np.zeros(0, np.int32)
    triples = _hyb_setup(dev, indptr, indices, m, n, 2, [1, 2], weighted=False, seed=0)
    x = np.ones((n, 32), np.float32)
    got, _ = _run_hyb(dev, m, n, 32, 2, [1, 2], triples, x)
    assert np.all(got == 0)


def test_time_evaluator_protocol(dev):
    """One discarded call, then the mean of `number` launches between device events
    (the reference's f.time_evaluator(f.entry_name, dev, number=N), src/runtime/profiling.cc:742-797)."""
    g = datasets.config1()
    m, n, feat, nnz = g["m"], g["n"], g["feat"], len(g["indices"])
    f = ops.build_csrmm(m, n, feat, nnz)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    c = torch.zeros(m * feat, device=dev)
    secs = f.time_evaluator(number=20)(t(g["values"]), t(g["x"].ravel()), c, t(g["indptr"]), t(g["indices"]))
    assert 0 < secs < 1e-2
    assert f.entry_name == "main"
    _check(c.cpu().numpy().reshape(m, feat), g["indptr"], g["indices"], g["values"], g["x"], "after timing")


@pytest.mark.parametrize("parts,buckets", [(8, [1, 2, 4, 8]), (16, [1, 2, 4, 8, 16, 32]), (6, [3, 300])])
def test_hyb_spmm_many_partitions_add_and_follow_the_weights(dev, parts, buckets):
    """More than four column partitions: the plan lists the slots of every output row once and its
    launches go over that list.  The operator still adds to C (the reference's buckets add with
    atomics when there are several partitions, examples/spmm/bench_spmm.py:170-177), also for a
    row of thousands of entries, and still reads the weights at every call."""
    m, n, feat = 2000, 2500, 64
    indptr, indices = random_csr(m, n, 50000, parts, skew=1.2)
    # one row with entries in every partition, far beyond one wavefront's share
    hub = np.sort(np.random.default_rng(parts).choice(n, 2200, replace=False)).astype(np.int32)
    deg = np.diff(indptr)
    indices = np.concatenate([indices[:indptr[7]], hub, indices[indptr[8]:]]).astype(np.int32)
    deg[7] = len(hub)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    triples = _hyb_setup(dev, indptr, indices, m, n, parts, buckets, weighted=True, seed=parts)
    x = np.random.default_rng(1).standard_normal((n, feat), dtype=np.float32)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    f = ops.build_hyb_csrmm(m, n, feat, parts, buckets, [len(r) for _, r, _ in triples])
    args = []
    for a, r, c in triples:
        args += [t(a.ravel()), t(r), t(c.ravel())]
    import scipy.sparse as sp
    r, c, v = _hyb_as_coo(triples)
    exact = sp.csr_matrix((v.astype(np.float64), (r, c)), shape=(m, n)) @ x.astype(np.float64)
    scale = sp.csr_matrix((np.abs(v).astype(np.float64), (r, c)), shape=(m, n)) @ np.abs(x).astype(np.float64)
    start = np.random.default_rng(2).standard_normal((m, feat), dtype=np.float32)
    cdev = t(start.ravel().copy())
    f(t(x.ravel()), cdev, *args)
    got = cdev.cpu().numpy().reshape(m, feat)
    assert np.all(np.abs(got - (start + exact)) <= RTOL * (scale + np.abs(start)) + 1e-30)
    # the weights doubled in place: the same plan gives twice the product
    for k in range(0, len(args), 3):
        args[k].mul_(2)
    cdev.zero_()
    f(t(x.ravel()), cdev, *args)
    got2 = cdev.cpu().numpy().reshape(m, feat)
    assert np.all(np.abs(got2 - 2 * exact) <= 2 * RTOL * scale + 1e-30)


def test_hyb_spmm_many_partitions_invalidate_after_rewriting_columns(dev):
    """A plan with more than four partitions holds a copy of the column ids: a caller that rewrites
    the column arrays in place tells the operator (invalidate) and then gets the result for the
    new columns, the one a fresh operator computes."""
    m, n, feat, parts, buckets = 1500, 1800, 32, 6, [1, 2, 4, 8]
    indptr, indices = random_csr(m, n, 30000, 5, skew=1.1)
    triples = _hyb_setup(dev, indptr, indices, m, n, parts, buckets, weighted=True, seed=3)
    x = np.random.default_rng(3).standard_normal((n, feat), dtype=np.float32)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    args = []
    for a, r, c in triples:
        args += [t(a.ravel()), t(r), t(c.ravel())]
    nrows = [len(r) for _, r, _ in triples]
    xd = t(x.ravel())

    def run(op):
        cdev = torch.zeros(m * feat, dtype=torch.float32, device=dev)
        op(xd, cdev, *args)
        torch.cuda.synchronize()
        return cdev

    f = ops.build_hyb_csrmm(m, n, feat, parts, buckets, nrows)
    before = run(f)
    for k in range(2, len(args), 3):
        args[k].copy_((args[k] + 7) % n)   # other columns at the same addresses
    fresh = run(ops.build_hyb_csrmm(m, n, feat, parts, buckets, nrows))
    assert not torch.allclose(fresh, before, rtol=1e-3, atol=1e-3)
    f.invalidate()
    assert torch.allclose(run(f), fresh, rtol=1e-5, atol=1e-5)
