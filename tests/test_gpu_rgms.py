"""GPU parity of RGMS (gather -> MFMA -> scatter-add, fp16 in, fp32 out) against the oracle.
Tolerance: rtol 2e-2 (fp16 inputs, fp32 accumulation) with the term magnitudes as atol scale."""
import numpy as np
import pytest
import torch

import oracle
import sparsetir_amd as st
from sparsetir_amd import datasets, ops
from helpers import random_csf, rgms_f64

pytestmark = pytest.mark.gpu


def _run(dev, csf, m, n, x, w, group, buckets, weighted, seed=0, static=False, dtype=torch.float16):
    p0, i0, p1, i1 = csf
    R, fin, fout = w.shape
    rows_bkt = [max(1, group // b) for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(p0, i0, p1, i1, rows_bkt, buckets)
    rng = np.random.default_rng(seed)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    triples, mids, avals = [], [], []
    for b in range(len(buckets)):
        a = mask[b].astype(np.float32)
        if weighted:
            a = a * (0.5 + rng.random(a.shape, dtype=np.float32))
        a16 = a.astype(np.float16)
        avals.append(a16)
        triples += [t(a16.ravel()), t(rows[b].ravel()), t(cols[b].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[b]))))
    f = ops.build_rgms(m, n, R, fin, fout, rows_bkt, buckets, [c.shape[0] for c in cols], static_weights=static)
    y = torch.zeros(m * fout, dtype=torch.float32, device=dev)
    x16, w16 = x.astype(np.float16), w.astype(np.float16)
    f(t(w16.ravel()), t(x16.ravel()), y, *triples, *mids)
    torch.cuda.synchronize()
    if static:  # a second call reuses the index that holds the weights
        y2 = torch.zeros_like(y)
        f(t(w16.ravel()), t(x16.ravel()), y2, *triples, *mids)
        torch.cuda.synchronize()
        assert torch.allclose(y, y2, rtol=1e-6, atol=1e-6)
    # edge weights in CSF order for the closed form: decode them from the ELL3D arrays
    coo = {}
    for b in range(len(buckets)):
        rel = np.repeat(np.arange(R), np.diff(ptr[b]))
        G, rb, cb = cols[b].shape
        for g in range(G):
            for ii in range(rb):
                for s in range(cb):
                    if mask[b][g, ii, s]:
                        coo[(rel[g], rows[b][g, ii], cols[b][g, ii, s])] = float(avals[b][g, ii, s])
    av = np.zeros(len(i1), np.float32)
    for r in range(R):
        for i in range(p0[r], p0[r + 1]):
            for j in range(p1[i], p1[i + 1]):
                av[j] = coo[(r, i0[i], i1[j])]
    return y.cpu().numpy().reshape(m, fout), x16.astype(np.float32), w16.astype(np.float32), av


def _check(got, csf, av, x32, w32, m, what):
    want = rgms_f64(*csf, av, x32, w32, m)
    scale = rgms_f64(*csf, np.abs(av), np.abs(x32), np.abs(w32), m)
    err = np.abs(got - want)
    assert np.all(err <= 2e-2 * np.abs(want) + 1e-5 * scale + 1e-30), f"{what}: worst {err.max():.3e}"
    ref = oracle.rgms(w32, x32, av, *csf, m)
    assert np.all(np.abs(got - ref) <= 2e-2 * np.abs(ref) + 2e-5 * scale + 1e-30)


@pytest.mark.parametrize("group,buckets,fin,fout,weighted", [
    (256, [1, 2, 4, 8, 16], 32, 32, False),
    (32, [1, 2, 4, 8, 16, 32], 32, 64, True),
    (16, [1, 2, 4], 16, 32, True),
    (12, [1, 3, 6], 48, 32, True),
    (64, [2, 64], 64, 96, False),
])
def test_rgms_small(dev, group, buckets, fin, fout, weighted):
    R, n = 5, 300
    csf = random_csf(R, n, 900, seed=group)
    rng = np.random.default_rng(group)
    x = rng.standard_normal((n, fin), dtype=np.float32)
    w = rng.standard_normal((R, fin, fout), dtype=np.float32) * 0.1
    got, x32, w32, av = _run(dev, csf, n, n, x, w, group, buckets, weighted)
    _check(got, csf, av, x32, w32, n, f"group={group} buckets={buckets}")


def test_rgms_config5_reduced(dev):
    cfg = datasets.config5(n=4000, num_rels=65, num_edges=40000)
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    got, x32, w32, av = _run(dev, csf, cfg["m"], cfg["n"], cfg["x"], cfg["w"], 256, cfg["buckets"], False)
    _check(got, csf, av, x32, w32, cfg["m"], "config5 reduced")


@pytest.mark.parametrize("group,buckets", [(256, [1, 2, 4, 8, 16]), (32, [1, 2, 4, 8, 16, 32]), (48, [1, 3, 4, 16])])
def test_rgms_tiled_accumulation(dev, group, buckets):
    """Enough slots for the destination-tiled kernel (edges re-indexed by 32-row output tile, no
    atomics), bucket widths that are not powers of two included."""
    cfg = datasets.config5(n=20000, num_rels=9, num_edges=200000, seed=7)
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    got, x32, w32, av = _run(dev, csf, cfg["m"], cfg["n"], cfg["x"], cfg["w"], group, buckets, True)
    _check(got, csf, av, x32, w32, cfg["m"], f"tiled group={group}")


@pytest.mark.parametrize("group,buckets,weighted", [(256, [1, 2, 4, 8, 16], False), (32, [1, 2, 4, 8, 16, 32], True),
                                                    (48, [1, 3, 4, 16], True)])
def test_rgms_tiled_static_weights(dev, group, buckets, weighted):
    """The plan that was promised unchanging slot weights: zero-weight (padding) slots are left out
    of the edge index and the weights travel inside 8-byte records.  Same result as the oracle."""
    cfg = datasets.config5(n=20000, num_rels=9, num_edges=200000, seed=11)
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    got, x32, w32, av = _run(dev, csf, cfg["m"], cfg["n"], cfg["x"], cfg["w"], group, buckets, weighted, static=True)
    _check(got, csf, av, x32, w32, cfg["m"], f"static group={group}")


def test_rgms_static_weights_edge_cases(dev):
    """Every slot weight zero: nothing is launched and Y keeps its content.  The promise cannot be
    changed after the first launch.  bf16 weights take the same path."""
    from sparsetir_amd._lib import SparseTIRError, lib, check
    import ctypes
    cfg = datasets.config5(n=6000, num_rels=4, num_edges=40000, seed=12)
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    R, fin, fout, buckets, group = 4, 32, 32, [1, 2, 4, 8], 64
    rb = [group // b for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rb, buckets)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    zero_triples, triples, mids = [], [], []
    for b in range(len(buckets)):
        zero_triples += [torch.zeros(mask[b].size, dtype=torch.bfloat16, device=dev), t(rows[b].ravel()), t(cols[b].ravel())]
        triples += [t(mask[b].astype(np.float32).ravel()).bfloat16(), t(rows[b].ravel()), t(cols[b].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[b]))))
    groups = [c.shape[0] for c in cols]
    w = t(cfg["w"].ravel()).bfloat16()
    x = t(cfg["x"].ravel()).bfloat16()
    y = torch.full((cfg["m"] * fout,), 3.0, device=dev)
    ops.build_rgms(cfg["m"], cfg["n"], R, fin, fout, rb, buckets, groups, torch.bfloat16, static_weights=True)(
        w, x, y, *zero_triples, *mids)
    torch.cuda.synchronize()
    assert bool((y == 3.0).all())
    # bf16 with the 0/1 mask: equals the plan without the promise
    ya, yb = torch.zeros(cfg["m"] * fout, device=dev), torch.zeros(cfg["m"] * fout, device=dev)
    fa = ops.build_rgms(cfg["m"], cfg["n"], R, fin, fout, rb, buckets, groups, torch.bfloat16, static_weights=True)
    fb = ops.build_rgms(cfg["m"], cfg["n"], R, fin, fout, rb, buckets, groups, torch.bfloat16)
    fa(w, x, ya, *triples, *mids)
    fb(w, x, yb, *triples, *mids)
    torch.cuda.synchronize()
    assert ya.abs().sum() > 0 and torch.allclose(ya, yb, rtol=1e-5, atol=1e-5)
    with pytest.raises(SparseTIRError, match="launched already"):
        check(lib().stir_rgms_plan_set_static_weights(next(iter(fa._plans._plans.values()))[0], 0))


def test_rgms_tiled_repeat_calls_accumulate(dev):
    cfg = datasets.config5(n=20000, num_rels=5, num_edges=150000, seed=8)
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    R, fin, fout, buckets, group = 5, 32, 32, [1, 2, 4, 8], 64
    rows_bkt = [group // b for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rows_bkt, buckets)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    triples, mids = [], []
    for b in range(len(buckets)):
        triples += [t(mask[b].astype(np.float16).ravel()), t(rows[b].ravel()), t(cols[b].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[b]))))
    f = ops.build_rgms(cfg["m"], cfg["n"], R, fin, fout, rows_bkt, buckets, [c.shape[0] for c in cols])
    w, x = t(cfg["w"].astype(np.float16).ravel()), t(cfg["x"].astype(np.float16).ravel())
    y = torch.zeros(cfg["m"] * fout, dtype=torch.float32, device=dev)
    f(w, x, y, *triples, *mids)
    once = y.clone()
    f(w, x, y, *triples, *mids)   # Y is accumulated into, as with the atomic kernel; the index is reused
    torch.cuda.synchronize()
    assert once.abs().sum() > 0
    assert torch.allclose(y, 2 * once, rtol=1e-6, atol=1e-6)
    y2 = torch.zeros_like(y)
    f(w, x, y2, *triples, *mids)
    torch.cuda.synchronize()
    # a tile is summed in a fixed order by one workgroup; only the few tiles cut into several
    # units (those holding the repeated row ids of the ELL3D padding) meet in atomics
    assert torch.allclose(y2, once, rtol=1e-6, atol=1e-6)
    assert float((y2 != once).float().mean()) < 0.01


def test_rgms_bf16(dev):
    """bf16 W, X and slot weights through the same kernel (bf16 MFMA), fp32 accumulate and output."""
    R, n, fin, fout, group, buckets = 5, 300, 32, 64, 32, [1, 2, 4, 8]
    csf = random_csf(R, n, 900, seed=31)
    rng = np.random.default_rng(31)
    rows_bkt = [group // b for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rows_bkt, buckets)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    x = torch.from_numpy(rng.standard_normal((n, fin), dtype=np.float32)).to(dev).bfloat16()
    w = torch.from_numpy(rng.standard_normal((R, fin, fout), dtype=np.float32) * 0.1).to(dev).bfloat16()
    triples, mids = [], []
    for b in range(len(buckets)):
        triples += [t(mask[b].astype(np.float32).ravel()).bfloat16(), t(rows[b].ravel()), t(cols[b].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[b]))))
    f = ops.build_rgms(n, n, R, fin, fout, rows_bkt, buckets, [c.shape[0] for c in cols], dtype=torch.bfloat16)
    y = torch.zeros(n * fout, dtype=torch.float32, device=dev)
    f(w.reshape(-1), x.reshape(-1), y, *triples, *mids)
    y2 = torch.zeros_like(y)
    from sparsetir_amd import packed
    packed.get_global_func("sparsetir.rgms")(w.reshape(-1), x.reshape(-1), y2, *triples, *mids, fin, fout)
    torch.cuda.synchronize()
    av = np.ones(len(csf[3]), np.float32)
    _check(y.cpu().numpy().reshape(n, fout), csf, av, x.float().cpu().numpy(), w.float().cpu().numpy(), n, "bf16")
    assert torch.allclose(y, y2, rtol=1e-5, atol=1e-5)


def _csf_from_pairs(pairs, n):
    """CSF from one (dst, src) array pair per relation (duplicates removed, sorted)."""
    indptr0, indices0, indptr1, indices1, nnz = [0], [], [0], [], 0
    for dst, src in pairs:
        key = np.unique(dst.astype(np.int64) * n + src)
        dst, src = key // n, key % n
        rows, counts = np.unique(dst, return_counts=True)
        indptr0.append(indptr0[-1] + len(rows))
        indices0.append(rows)
        indptr1.append(nnz + np.cumsum(counts))
        indices1.append(src)
        nnz += len(src)
    i32 = lambda parts: np.concatenate([np.atleast_1d(p) for p in parts]).astype(np.int32)
    return i32(indptr0), i32(indices0), i32(indptr1), i32(indices1)


@pytest.mark.parametrize("fin,fout,group,buckets,bf16", [
    (32, 32, 256, [1, 2, 4, 8, 16], False),
    (16, 64, 64, [1, 2, 4, 64], False),
    (48, 32, 48, [1, 3, 4, 16], False),
    (128, 32, 32, [2, 8, 32], False),
    (32, 64, 64, [1, 4, 16], True),
])
def test_rgms_tiled_hub_rows(dev, fin, fout, group, buckets, bf16):
    """Destination-tiled path: output rows not a multiple of 32, one row that
    receives thousands of edges in three relations (its tile is cut into several units that meet
    in atomics), relations without edges, widths that are not powers of two."""
    n, R = 5001, 7
    rng = np.random.default_rng(fin + fout)
    pairs = []
    for r in range(R):
        e = 0 if r == 3 else 20000
        dst, src = rng.integers(0, n, e), rng.integers(0, n, e)
        if r in (0, 1, 5):
            hub = rng.choice(n, 3000, replace=False)
            dst = np.concatenate([dst, np.full(3000, 77)])
            src = np.concatenate([src, hub])
        pairs.append((dst, src))
    csf = _csf_from_pairs(pairs, n)
    rows_bkt = [max(1, group // b) for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rows_bkt, buckets)
    assert sum(mk.size for mk in mask) >= 8192
    tdt = torch.bfloat16 if bf16 else torch.float16
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    x = t(rng.standard_normal((n, fin), dtype=np.float32)).to(tdt)
    w = t(rng.standard_normal((R, fin, fout), dtype=np.float32) * 0.1).to(tdt)
    triples, mids, wts = [], [], []
    for b in range(len(buckets)):
        a = t(mask[b].astype(np.float32) * (0.5 + rng.random(mask[b].shape, dtype=np.float32))).to(tdt)
        wts.append(a.float().cpu().numpy())
        triples += [a.reshape(-1), t(rows[b].ravel()), t(cols[b].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[b]))))
    f = ops.build_rgms(n, n, R, fin, fout, rows_bkt, buckets, [c.shape[0] for c in cols], dtype=tdt)
    y = torch.zeros(n * fout, dtype=torch.float32, device=dev)
    f(w.reshape(-1), x.reshape(-1), y, *triples, *mids)
    torch.cuda.synchronize()
    # closed form in float64 straight from the ELL3D arrays: Y[row] += a * X[col] @ W[rel]
    x64, w64 = x.double().cpu().numpy(), w.double().cpu().numpy()
    want, scale = np.zeros((n, fout)), np.zeros((n, fout))
    for b in range(len(buckets)):
        G, rb, cb = cols[b].shape
        rel = np.repeat(np.arange(R), np.diff(ptr[b]))
        for r in range(R):
            g = np.nonzero(rel == r)[0]
            if len(g) == 0:
                continue
            a = wts[b][g].reshape(-1, cb).astype(np.float64)
            c = cols[b][g].reshape(-1, cb)
            agg = np.einsum("es,esk->ek", a, x64[c])
            agg_abs = np.einsum("es,esk->ek", a, np.abs(x64[c]))
            dest = rows[b][g].reshape(-1)
            np.add.at(want, dest, agg @ w64[r])
            np.add.at(scale, dest, agg_abs @ np.abs(w64[r]))
    got = y.cpu().numpy().reshape(n, fout).astype(np.float64)
    err = np.abs(got - want)
    assert np.all(err <= 2e-2 * np.abs(want) + 1e-5 * scale + 1e-30), f"worst {err.max():.3e}"
    assert np.abs(want[77]).max() > 0


def _tiled_case(dev, pairs, m, n, R, fin, fout, group, buckets, seed):
    """Runs the fp16 operator on CSF built from (dst, src) pairs; returns (got, want, scale)."""
    csf = _csf_from_pairs(pairs, n)
    rows_bkt = [max(1, group // b) for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rows_bkt, buckets)
    rng = np.random.default_rng(seed)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    x = t(rng.standard_normal((n, fin), dtype=np.float32)).half()
    w = t(rng.standard_normal((R, fin, fout), dtype=np.float32) * 0.1).half()
    triples, mids = [], []
    for b in range(len(buckets)):
        triples += [t(mask[b].astype(np.float16).ravel()), t(rows[b].ravel()), t(cols[b].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[b]))))
    f = ops.build_rgms(m, n, R, fin, fout, rows_bkt, buckets, [c.shape[0] for c in cols])
    y = torch.zeros(m * fout, dtype=torch.float32, device=dev)
    f(w.reshape(-1), x.reshape(-1), y, *triples, *mids)
    torch.cuda.synchronize()
    ones = np.ones(len(csf[3]), np.float32)
    x32, w32 = x.float().cpu().numpy(), w.float().cpu().numpy()
    want = rgms_f64(*csf, ones, x32, w32, m)
    scale = rgms_f64(*csf, ones, np.abs(x32), np.abs(w32), m)
    return y.cpu().numpy().reshape(m, fout), want, scale, (f, w, x, triples, mids, slots_of(mask))


def slots_of(mask):
    return sum(mk.size for mk in mask)


def test_rgms_tiled_few_output_rows(dev):
    """Five output rows, 12000 edges from 4000 sources: one tile of 32 rows cut into many units
    that meet in atomics; m != n."""
    m, n, R = 5, 4000, 3
    rng = np.random.default_rng(5)
    pairs = [(rng.integers(0, m, 6000), rng.integers(0, n, 6000)) for _ in range(R)]
    got, want, scale, info = _tiled_case(dev, pairs, m, n, R, 32, 32, 32, [8, 32], 5)
    assert info[-1] >= 8192
    assert np.all(np.abs(got - want) <= 2e-2 * np.abs(want) + 1e-5 * scale + 1e-30)


def test_rgms_tiled_sparse_rows_and_empty_tiles(dev):
    """Edges end in two narrow bands of a large row range: most tiles have no edge and get no
    unit; the rows in between stay untouched (checked with a non-zero Y)."""
    m, n, R = 100_000, 3000, 4
    rng = np.random.default_rng(6)
    pairs = []
    for r in range(R):
        dst = np.concatenate([rng.integers(40, 140, 2500), rng.integers(99_900, m, 2500)])
        pairs.append((dst, rng.integers(0, n, 5000)))
    got, want, scale, info = _tiled_case(dev, pairs, m, n, R, 32, 32, 64, [1, 2, 4, 8, 16, 64], 6)
    assert info[-1] >= 8192
    assert np.all(np.abs(got - want) <= 2e-2 * np.abs(want) + 1e-5 * scale + 1e-30)
    f, w, x, triples, mids, _ = info
    y = torch.full((m * 32,), 3.0, dtype=torch.float32, device=dev)
    f(w.reshape(-1), x.reshape(-1), y, *triples, *mids)
    torch.cuda.synchronize()
    y = y.cpu().numpy().reshape(m, 32)
    assert np.all(y[200:99_000] == 3.0)
    assert np.all(np.abs(y - 3.0 - want) <= 2e-2 * np.abs(want) + 1e-5 * (scale + 3.0) + 1e-30)


def test_rgms_tiled_rejects_ids_out_of_range(dev):
    """The index is built by the first launch: a row id >= m or a column id >= n fails it."""
    m = n = 3000
    rng = np.random.default_rng(7)
    pairs = [(rng.integers(0, m, 6000), rng.integers(0, n, 6000)) for _ in range(2)]
    csf = _csf_from_pairs(pairs, n)
    buckets, rows_bkt = [1, 4, 16], [16, 4, 1]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rows_bkt, buckets)
    assert slots_of(mask) >= 8192
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    for what in ("row", "col"):
        triples, mids = [], []
        for b in range(len(buckets)):
            r, c = rows[b].copy(), cols[b].copy()
            if b == 1 and what == "row":
                r.ravel()[3] = m
            if b == 1 and what == "col":
                c.ravel()[3] = n + 7
            triples += [t(mask[b].astype(np.float16).ravel()), t(r.ravel()), t(c.ravel())]
            mids.append(t(np.repeat(np.arange(2, dtype=np.int32), np.diff(ptr[b]))))
        f = ops.build_rgms(m, n, 2, 32, 32, rows_bkt, buckets, [c.shape[0] for c in cols])
        x = torch.zeros(n * 32, dtype=torch.float16, device=dev)
        w = torch.zeros(2 * 32 * 32, dtype=torch.float16, device=dev)
        y = torch.zeros(m * 32, dtype=torch.float32, device=dev)
        with pytest.raises(Exception, match="outside"):
            f(w, x, y, *triples, *mids)


@pytest.mark.parametrize("seed", range(10))
def test_rgms_tiled_random_shapes(dev, seed):
    """Random relation counts, row/column ranges, bucket lists and feature sizes, all large enough
    for the destination-tiled kernel."""
    rng = np.random.default_rng(100 + seed)
    R = int(rng.integers(1, 13))
    m, n = int(rng.integers(33, 3000)), int(rng.integers(40, 3000))
    per_rel = int(rng.integers(9000, 30000)) // R + 1
    pairs = [(rng.integers(0, m, per_rel), rng.integers(0, n, per_rel)) for _ in range(R)]
    group = int(rng.choice([16, 32, 64, 256]))
    widths = sorted(set(int(w) for w in rng.choice([1, 2, 3, 4, 8, 16], size=int(rng.integers(1, 5)))))
    widths = [w for w in widths if w <= group]
    fin, fout = int(rng.choice([16, 32, 64])), int(rng.choice([32, 64]))
    got, want, scale, info = _tiled_case(dev, pairs, m, n, R, fin, fout, group, widths, seed)
    assert info[-1] >= 8192, "shape too small for the tiled kernel"
    err = np.abs(got - want)
    assert np.all(err <= 2e-2 * np.abs(want) + 1e-5 * scale + 1e-30), (
        f"R={R} m={m} n={n} group={group} widths={widths} fin={fin} fout={fout}: worst {err.max():.3e}")


@pytest.mark.parametrize("R,skew", [
    (100, 1.0),   # two ranges of 50 relations, each with W in the LDS
    (150, 1.2),   # three ranges, a long tail of small relations
    (200, 0.0),   # too many ranges: one launch that reads W from memory
    (1000, 1.5),  # relations without edges among them
])
def test_rgms_tiled_more_relations_than_fit_the_lds(dev, R, skew):
    """More relations than the LDS of a compute unit holds (the reference's AIFB, BGS and AM
    graphs, examples/rgms/rgcn/bench_rgcn_tensorcore.py:917, have about 90 to 270 with their
    inverses): the plan indexes a few ranges of relations apart and launches them in turn, or reads
    W from memory.  Relation sizes follow a power law and are shuffled, so a range mixes large
    and small relations; against the float64 closed form, added to a Y that is not zero."""
    rng = np.random.default_rng(77 + R)
    m, n, fin, fout = 2100, 1900, 32, 32
    size = 1.0 / np.arange(1, R + 1) ** skew
    size = rng.permutation(np.floor(size / size.sum() * 50000).astype(np.int64))
    assert (size == 0).any() == (R == 1000)
    pairs = [(rng.integers(0, m, k), rng.integers(0, n, k)) for k in size]
    csf = _csf_from_pairs(pairs, n)
    group, buckets = 64, [1, 2, 4, 8]
    rows_bkt = [group // b for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rows_bkt, buckets)
    assert slots_of(mask) >= 8192
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    x = t(rng.standard_normal((n, fin), dtype=np.float32)).half()
    w = t(rng.standard_normal((R, fin, fout), dtype=np.float32) * 0.1).half()
    triples, mids = [], []
    for b in range(len(buckets)):
        triples += [t(mask[b].astype(np.float16).ravel()), t(rows[b].ravel()), t(cols[b].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[b]))))
    ones = np.ones(len(csf[3]), np.float32)
    x32, w32 = x.float().cpu().numpy(), w.float().cpu().numpy()
    want = rgms_f64(*csf, ones, x32, w32, m)
    scale = rgms_f64(*csf, ones, np.abs(x32), np.abs(w32), m)
    for static in (False, True):
        f = ops.build_rgms(m, n, R, fin, fout, rows_bkt, buckets, [c.shape[0] for c in cols], static_weights=static)
        y = torch.full((m * fout,), 0.5, dtype=torch.float32, device=dev)
        f(w.reshape(-1), x.reshape(-1), y, *triples, *mids)
        torch.cuda.synchronize()
        err = np.abs(y.cpu().numpy().reshape(m, fout) - 0.5 - want)
        assert np.all(err <= 2e-2 * np.abs(want) + 1e-5 * scale + 1e-6), f"static={static}: worst {err.max():.3e}"


@pytest.mark.parametrize("R,fin,fout,static", [
    (60, 32, 32, True),    # W of 120 KB: resident kernel, 12 wavefronts per compute unit
    (65, 32, 32, False),   # 130 KB: the most that leaves room for 12
    (68, 32, 32, True),    # 136 KB: 8 wavefronts
    (80, 32, 32, False),   # 160 KB: two ranges of 40 relations, a launch each
    (20, 64, 64, True),    # two feature tiles out, four operand blocks in
    (33, 48, 32, False),   # feat_in that is not a power of two
])
def test_rgms_tiled_sizes_of_w(dev, R, fin, fout, static):
    """The destination-tiled operator picks its kernel by the size of W (num_rels x feat_in x
    feat_out): all regimes against the float64 closed form, and W at an address that is not a
    multiple of 16 bytes (served by the kernel that reads W from memory)."""
    rng = np.random.default_rng(1000 + R)
    m, n = 3001, 2500
    per_rel = 60000 // R
    pairs = [(rng.integers(0, m, per_rel), rng.integers(0, n, per_rel)) for _ in range(R)]
    csf = _csf_from_pairs(pairs, n)
    group, buckets = 64, [1, 2, 4, 8]
    rows_bkt = [group // b for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rows_bkt, buckets)
    assert slots_of(mask) >= 8192
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    x = t(rng.standard_normal((n, fin), dtype=np.float32)).half()
    w_store = torch.zeros(R * fin * fout + 8, dtype=torch.float16, device=dev)
    w_vals = t(rng.standard_normal((R, fin, fout), dtype=np.float32) * 0.1).half()
    triples, mids = [], []
    for b in range(len(buckets)):
        triples += [t(mask[b].astype(np.float16).ravel()), t(rows[b].ravel()), t(cols[b].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[b]))))
    ones = np.ones(len(csf[3]), np.float32)
    x32, w32 = x.float().cpu().numpy(), w_vals.float().cpu().numpy()
    want = rgms_f64(*csf, ones, x32, w32, m)
    scale = rgms_f64(*csf, ones, np.abs(x32), np.abs(w32), m)
    for shift in (0, 1):  # 0: aligned, 1: two bytes off
        w = w_store[shift:shift + R * fin * fout]
        w.copy_(w_vals.reshape(-1))
        f = ops.build_rgms(m, n, R, fin, fout, rows_bkt, buckets, [c.shape[0] for c in cols], static_weights=static)
        y = torch.zeros(m * fout, dtype=torch.float32, device=dev)
        f(w, x.reshape(-1), y, *triples, *mids)
        f(w, x.reshape(-1), y, *triples, *mids)  # the operator accumulates: twice the sum
        torch.cuda.synchronize()
        got = y.cpu().numpy().reshape(m, fout) / 2
        err = np.abs(got - want)
        assert np.all(err <= 2e-2 * np.abs(want) + 1e-5 * scale + 1e-30), f"shift={shift}: worst {err.max():.3e}"
