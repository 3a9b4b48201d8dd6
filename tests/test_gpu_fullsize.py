"""Parity at the full sizes of the headline configurations (config 3: 2.45M nodes / 61.9M edges;
config 5: 100k nodes / 65 relations / 2M edges): bit-exact index arrays against the oracle, and
size-independent properties for the numeric kernels (hyb equals CSR row-split on the same matrix,
linearity, oracle agreement on row / edge samples)."""
import numpy as np
import pytest
import torch

import oracle
import sparsetir_amd as st
from sparsetir_amd import datasets, ops
from helpers import rgms_f64, spmm_f64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cfg3():
    return datasets.config3()


@pytest.mark.parametrize("parts,buckets", [
    (2, [1, 2, 4, 8, 16, 32]),
    (1, [1, 2, 4, 8, 16, 32, 64, 128, 256, 512]),   # the decomposition bench.py times
    (16, [1, 2, 4, 8, 16, 32]),                     # examples/spmm/bench_spmm.py:233-253 for a graph of this size
])
def test_config3_device_format_bit_exact(dev, cfg3, parts, buckets):
    g = cfg3
    m, n = g["m"], g["n"]
    t = lambda a: torch.from_numpy(a).to(dev)
    rows, cols, mask = st.column_part_hyb(m, n, t(g["indptr"]), t(g["indices"]), parts, buckets)
    want = oracle.column_part_hyb(m, n, g["indptr"], g["indices"], parts, buckets)
    total = 0
    for p in range(parts):
        for b in range(len(buckets)):
            assert np.array_equal(rows[p][b].cpu().numpy(), want[0][p][b])
            assert np.array_equal(cols[p][b].cpu().numpy(), want[1][p][b])
            assert np.array_equal(mask[p][b].cpu().numpy(), want[2][p][b])
            total += int(want[2][p][b].sum())
    assert total == len(g["indices"])  # every nonzero placed exactly once


@pytest.mark.parametrize("setting", ["bench", "reference"])
def test_config3_hyb_equals_csr_and_oracle_sample(dev, cfg3, setting):
    g = cfg3
    m, n, feat = g["m"], g["n"], 128
    # "bench": the decomposition bench.py times; "reference": 16 partitions x widths 1..32, what
    # examples/spmm/bench_spmm.py:233-253 picks for a graph of this size (every bucket adds with atomics)
    parts, buckets = (g["num_col_parts"], g["buckets"]) if setting == "bench" else (16, [1, 2, 4, 8, 16, 32])
    indptr, indices = g["indptr"], g["indices"]
    nnz = len(indices)
    t = lambda a: torch.from_numpy(a).to(dev)
    d_ptr, d_idx = t(indptr), t(indices)
    vals = torch.rand(nnz, device=dev, generator=torch.Generator(device=dev).manual_seed(5)) + 0.5
    rows, cols, mask, avals = st.column_part_hyb(m, n, d_ptr, d_idx, parts, buckets, values=vals)
    triples, nrows = [], []
    for p in range(parts):
        for b in range(len(buckets)):
            triples += [avals[p][b].reshape(-1), rows[p][b], cols[p][b].reshape(-1)]
            nrows.append(int(rows[p][b].shape[0]))
    del mask
    x = torch.randn(n * feat, device=dev, generator=torch.Generator(device=dev).manual_seed(6))
    hyb = ops.build_hyb_csrmm(m, n, feat, parts, buckets, nrows)
    csr = ops.build_csrmm(m, n, feat, nnz)
    c_h = torch.zeros(m * feat, device=dev)
    c_c = torch.empty(m * feat, device=dev)
    hyb(x, c_h, *triples)
    csr(vals, x, c_c, d_ptr, d_idx)
    torch.cuda.synchronize()
    deg = t(np.diff(indptr).astype(np.float32))
    # |a| <= 1.5, |x| below ~6: summed magnitude per element is at most 9 * degree
    tol = (1e-5 * 9.0 * deg.clamp(min=1.0)).repeat_interleave(feat)
    assert bool(((c_h - c_c).abs() <= tol).all())
    # linearity: hyb(2x) == 2 hyb(x) up to accumulation order
    c2 = torch.zeros(m * feat, device=dev)
    hyb(2 * x, c2, *triples)
    assert bool(((c2 - 2 * c_h).abs() <= 2 * tol).all())
    # oracle (serial CPU loop nest) on the first 20000 rows
    r = 20000
    sub_ptr, sub_idx = indptr[:r + 1], indices[:indptr[r]]
    vh, xh = vals[:indptr[r]].cpu().numpy(), x.cpu().numpy().reshape(n, feat)
    ref = oracle.csrmm(vh, xh, sub_ptr, sub_idx, feat)
    scale = spmm_f64(sub_ptr, sub_idx, vh, np.abs(xh))
    got = c_h[:r * feat].cpu().numpy().reshape(r, feat)
    assert np.all(np.abs(got - ref) <= 2e-5 * scale + 1e-30)


def test_config3_sddmm_edge_sample(dev, cfg3):
    g = cfg3
    m, n, feat = g["m"], g["n"], 64
    indptr, indices = g["indptr"], g["indices"]
    nnz = len(indices)
    t = lambda a: torch.from_numpy(a).to(dev)
    a = torch.randn(m * feat, device=dev, generator=torch.Generator(device=dev).manual_seed(7))
    b = torch.randn(n * feat, device=dev, generator=torch.Generator(device=dev).manual_seed(8))
    out = torch.empty(nnz, device=dev)
    mid = torch.empty(nnz, dtype=torch.int32, device=dev)
    args = (a, b, out, t(indptr), t(indices), mid)
    ops.build_sddmm_preproc(m, n, feat, nnz)(*args)
    ops.build_sddmm(m, n, feat, nnz)(*args)
    torch.cuda.synchronize()
    rows = np.repeat(np.arange(m, dtype=np.int32), np.diff(indptr))
    assert np.array_equal(mid.cpu().numpy(), rows)  # mid is the row of every nonzero
    sel = np.random.default_rng(0).choice(nnz, 200000, replace=False)
    ah = a.cpu().numpy().reshape(m, feat)[rows[sel]].astype(np.float64)
    bh = b.cpu().numpy().reshape(n, feat)[indices[sel]].astype(np.float64)
    want = np.einsum("ek,ek->e", ah, bh)
    scale = np.einsum("ek,ek->e", np.abs(ah), np.abs(bh))
    assert np.all(np.abs(out.cpu().numpy()[sel] - want) <= 1e-5 * scale)
    # the edge-scaled form out_e = A_e <X[row], Y[col]> on the same inputs, A_e from U(0,1)
    ev = torch.rand(nnz, device=dev, generator=torch.Generator(device=dev).manual_seed(9))
    out2 = torch.full((nnz,), float("nan"), device=dev)
    ops.build_sddmm_scaled(m, n, feat, nnz)(a, b, out2, args[3], args[4], mid, ev)
    torch.cuda.synchronize()
    evh = ev.cpu().numpy()[sel].astype(np.float64)
    assert np.all(np.abs(out2.cpu().numpy()[sel] - want * evh) <= 2e-5 * scale * evh + 1e-30)
    # and everywhere: scaled result == edge value * unscaled result up to one rounding
    assert bool(((out2 - ev * out).abs() <= 1e-6 * (ev * out).abs() + 1e-30).all())


@pytest.mark.parametrize("deterministic", [True, False])
def test_config5_rgms_f32_full(dev, deterministic):
    """Config 5 in fp32, both front ends, against the float64 closed form (|err| <= 1e-5 of the
    summed magnitudes).  The tile form at this size runs 1563 units, of which the few beyond whole
    rounds of resident workgroups are cut into pieces whose partial tiles the last piece adds up:
    eight calls back to back give the same bits."""
    cfg = datasets.config5()
    R, n, fin, fout = cfg["num_rels"], cfg["n"], cfg["feat_in"], cfg["feat_out"]
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    rng = np.random.default_rng(11)
    a = (0.5 + rng.random(len(csf[3]))).astype(np.float32)
    w = np.ascontiguousarray(cfg["w"].transpose(0, 2, 1))  # [R, fout, fin]
    want = rgms_f64(*csf, a, cfg["x"], cfg["w"], n)
    scale = rgms_f64(*csf, np.abs(a), np.abs(cfg["x"]), np.abs(cfg["w"]), n)
    f = ops.build_rgms_csf(n, n, R, fin, fout, len(csf[1]), len(csf[3]), deterministic=deterministic)
    d = [t(a), t(w.ravel()), t(cfg["x"].ravel())] + [t(c) for c in csf]
    ys = [torch.zeros(n * fout, device=dev) for _ in range(8)]
    for y in ys:
        f(d[0], d[1], d[2], y, *d[3:])
    torch.cuda.synchronize()
    got = ys[0].cpu().numpy().reshape(n, fout)
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-5 * scale + 1e-30)
    if deterministic:
        assert all(torch.equal(ys[0], y) for y in ys[1:])
    # ELL3D buckets of the same graph (weights 1)
    buckets, group = cfg["buckets"], 32
    rb = [max(1, group // b) for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rb, buckets)
    triples, mids = [], []
    for k in range(len(buckets)):
        triples += [t(mask[k].astype(np.float32).ravel()), t(rows[k].ravel()), t(cols[k].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[k]))))
    ones = np.ones(len(csf[3]), np.float32)
    want1 = rgms_f64(*csf, ones, cfg["x"], cfg["w"], n)
    scale1 = rgms_f64(*csf, ones, np.abs(cfg["x"]), np.abs(cfg["w"]), n)
    g = ops.build_rgms_f32(n, n, R, fin, fout, rb, buckets, [c.shape[0] for c in cols], deterministic=deterministic)
    ys = [torch.zeros(n * fout, device=dev) for _ in range(8)]
    for y in ys:
        g(d[1], d[2], y, *triples, *mids)
    torch.cuda.synchronize()
    got = ys[0].cpu().numpy().reshape(n, fout)
    assert np.all(np.abs(got - want1) <= 1e-5 * np.abs(want1) + 1e-5 * scale1 + 1e-30)
    if deterministic:
        assert all(torch.equal(ys[0], y) for y in ys[1:])


def test_config5_rgms_full(dev):
    cfg = datasets.config5()
    R, n, fin, fout = cfg["num_rels"], cfg["n"], cfg["feat_in"], cfg["feat_out"]
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    buckets, group = cfg["buckets"], 256
    rb = [group // b for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rb, buckets)
    want_fmt = oracle.csf_to_ell3d(*csf, rb, buckets)
    for q, arrs in enumerate((ptr, rows, cols, mask)):
        for k in range(len(buckets)):
            assert np.array_equal(arrs[k], want_fmt[q][k])
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    triples, mids = [], []
    for k in range(len(buckets)):
        triples += [t(mask[k].astype(np.float16).ravel()), t(rows[k].ravel()), t(cols[k].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[k]))))
    x16, w16 = cfg["x"].astype(np.float16), cfg["w"].astype(np.float16)
    y = torch.zeros(n * fout, device=dev)
    ops.build_rgms(n, n, R, fin, fout, rb, buckets, [c.shape[0] for c in cols])(
        t(w16.ravel()), t(x16.ravel()), y, *triples, *mids)
    torch.cuda.synchronize()
    ones = np.ones(len(cfg["indices1"]), np.float32)
    x32, w32 = x16.astype(np.float32), w16.astype(np.float32)
    want = rgms_f64(*csf, ones, x32, w32, n)
    scale = rgms_f64(*csf, ones, np.abs(x32), np.abs(w32), n)
    got = y.cpu().numpy().reshape(n, fout)
    assert np.all(np.abs(got - want) <= 2e-2 * np.abs(want) + 1e-5 * scale + 1e-30)
    ref = oracle.rgms(w32, x32, ones, *csf, n)
    assert np.all(np.abs(got - ref) <= 2e-2 * np.abs(ref) + 2e-5 * scale + 1e-30)


def test_offsets_beyond_2_to_31_elements(dev):
    """X with 2.3e9 floats (9.2 GB): rows of X that start beyond the 2^31-th element must be
    reached with 64-bit offsets by the CSR, hyb and SDDMM kernels.  Checked against torch's own
    gathers on the device."""
    n, feat, m = 18_000_000, 128, 2048
    assert n * feat > 2**31
    gen = torch.Generator(device=dev).manual_seed(11)
    x = torch.randn(n * feat, device=dev, generator=gen)
    rng = np.random.default_rng(11)
    deg = rng.integers(1, 40, m)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    # most columns near the end of X, a few near the start
    cols = [np.sort(rng.choice(np.concatenate([np.arange(n - 200000, n), np.arange(0, 1000)]), d, replace=False))
            for d in deg]
    indices = np.concatenate(cols).astype(np.int32)
    nnz = len(indices)
    t = lambda a: torch.from_numpy(a).to(dev)
    d_ptr, d_idx = t(indptr), t(indices)
    vals = torch.rand(nnz, device=dev, generator=gen) + 0.5
    rowid = torch.repeat_interleave(torch.arange(m, device=dev), t(deg.astype(np.int64)))
    want = torch.zeros(m, feat, device=dev, dtype=torch.float64)
    want.index_add_(0, rowid, (x.view(n, feat)[d_idx.long()] * vals[:, None]).double())
    scale = torch.zeros(m, feat, device=dev, dtype=torch.float64)
    scale.index_add_(0, rowid, (x.view(n, feat)[d_idx.long()] * vals[:, None]).abs().double())

    c = torch.empty(m * feat, device=dev)
    ops.build_csrmm(m, n, feat, nnz)(vals, x, c, d_ptr, d_idx)
    assert torch.all((c.view(m, feat).double() - want).abs() <= 1e-5 * scale + 1e-30)

    buckets = [1, 2, 4, 8, 16, 32, 64]
    rows, cols_k, mask, avals = st.column_part_hyb(m, n, d_ptr, d_idx, 1, buckets, values=vals)
    triples = [a for b in range(len(buckets)) for a in (avals[0][b].reshape(-1), rows[0][b], cols_k[0][b].reshape(-1))]
    c2 = torch.zeros(m * feat, device=dev)
    ops.build_hyb_csrmm(m, n, feat, 1, buckets, [int(r.shape[0]) for r in rows[0]])(x, c2, *triples)
    assert torch.all((c2.view(m, feat).double() - want).abs() <= 1e-5 * scale + 1e-30)

    a = torch.randn(m * feat, device=dev, generator=gen)
    out = torch.empty(nnz, device=dev)
    mid = torch.empty(nnz, dtype=torch.int32, device=dev)
    args = (a, x, out, d_ptr, d_idx, mid)
    ops.build_sddmm_preproc(m, n, feat, nnz)(*args)
    ops.build_sddmm(m, n, feat, nnz)(*args)
    torch.cuda.synchronize()
    ref = (a.view(m, feat)[rowid].double() * x.view(n, feat)[d_idx.long()].double()).sum(1)
    mag = (a.view(m, feat)[rowid].double() * x.view(n, feat)[d_idx.long()].double()).abs().sum(1)
    assert torch.all((out.double() - ref).abs() <= 1e-5 * mag + 1e-30)


def _far_ids(rng, count, total, replace=False):
    """Ids out of [0, total): most of them near the end, a few near the start."""
    tail = min(200_000, total // 2)
    pool = np.concatenate([np.arange(total - tail, total), np.arange(0, min(1000, total - tail))])
    return np.sort(rng.choice(pool, count, replace=replace))


@pytest.mark.parametrize("out32", [False, True])
def test_bsr_offsets_beyond_2_to_31_elements(dev, out32):
    """X and Y with 2.6e9 elements each: the blocks of X and the block rows of Y that start beyond
    the 2^31-th element (and the 2^32-th byte) must be reached with 64-bit offsets.  Non-empty
    block rows against fp32 products by torch, every other block row must be zero."""
    mb = nb = 40_000
    blk, feat = 32, 2048
    assert nb * blk * feat > 2**31 and mb * blk * feat > 2**31
    rng = np.random.default_rng(21)
    live = _far_ids(rng, 160, mb)
    counts = np.zeros(mb, np.int64)
    counts[live] = rng.integers(1, 7, len(live))
    indptr = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    indices = np.concatenate([_far_ids(rng, counts[i], nb) for i in live]).astype(np.int32)
    nnzb = len(indices)
    gen = torch.Generator(device=dev).manual_seed(21)
    a = (torch.randn(nnzb * blk * blk, device=dev, generator=gen) * 0.05).half()
    x = torch.randn(nb * blk * feat, device=dev, generator=gen, dtype=torch.float16)
    odt = torch.float32 if out32 else torch.float16
    y = torch.ones(mb * blk * feat, device=dev, dtype=odt)
    t = lambda v: torch.from_numpy(v).to(dev)
    ops.build_bsrmm(mb, nb, nnzb, blk, feat, torch.float16, odt)(a, x, y, t(indptr), t(indices))
    torch.cuda.synchronize()
    yv, xv = y.view(mb, blk, feat), x.view(nb, blk, feat)
    for i in live:
        want = torch.zeros(blk, feat, device=dev)
        scale = torch.zeros(blk, feat, device=dev)
        for p in range(indptr[i], indptr[i + 1]):
            blk_a = a[p * blk * blk:(p + 1) * blk * blk].view(blk, blk).float()
            want += blk_a @ xv[indices[p]].float()
            scale += blk_a.abs() @ xv[indices[p]].float().abs()
        tol = (1e-5 if out32 else 2e-2) * want.abs() + 1e-5 * scale + 1e-30
        assert bool(((yv[i].float() - want).abs() <= tol).all()), int(i)
    # all the rest is zero: the non-zero entries of Y are those of the live block rows
    assert int(torch.count_nonzero(y)) == int(torch.count_nonzero(yv[t(live)]))


@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_tcspmm_offsets_beyond_2_to_31_elements(dev, out_dtype):
    """B and C with 2.3e9 / 2.5e9 elements: tiles at the far end of C, among them one long enough
    for the launch of the long tiles, gather rows at the far end of B."""
    n, feat, mb = 18_000_000, 128, 600_000
    m = mb * 32
    assert n * feat > 2**31 and m * feat > 2**31
    rng = np.random.default_rng(22)
    deg = np.zeros(m, np.int64)
    live_tiles = _far_ids(rng, 24, mb)
    for k, tile in enumerate(live_tiles):
        rows = np.arange(tile * 32, tile * 32 + 32)
        deg[rows] = rng.integers(0, 6, 32) if k != len(live_tiles) - 2 else 40  # one tile of 1280 columns
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    live_rows = np.nonzero(deg)[0]
    indices = np.concatenate([_far_ids(rng, deg[r], n) for r in live_rows]).astype(np.int32)
    gptr, tiles, mask = st.condense(indptr, indices, 32, 16)
    nnzb = tiles.shape[0]
    assert int(np.diff(gptr).max()) * 16 > 16 * 32  # more than 16 steps of 32 columns in one tile
    t = lambda v: torch.from_numpy(np.ascontiguousarray(v)).to(dev)
    gen = torch.Generator(device=dev).manual_seed(22)
    b = torch.randn(n * feat, device=dev, generator=gen, dtype=torch.float16)
    c = torch.ones(m * feat, device=dev, dtype=out_dtype)
    ops.build_tcspmm(mb, nnzb, feat, 32, 16, n, out_dtype)(
        t(mask.astype(np.float16).ravel()), b, c, t(gptr), t(tiles.ravel()))
    torch.cuda.synchronize()
    d_rows, d_idx = t(live_rows), t(indices)
    rowid = torch.repeat_interleave(torch.arange(len(live_rows), device=dev), t(deg[live_rows]))
    gathered = b.view(n, feat)[d_idx.long()].double()
    want = torch.zeros(len(live_rows), feat, device=dev, dtype=torch.float64).index_add_(0, rowid, gathered)
    scale = torch.zeros(len(live_rows), feat, device=dev, dtype=torch.float64).index_add_(0, rowid, gathered.abs())
    got = c.view(m, feat)[d_rows].double()
    rtol = 2e-2 if out_dtype == torch.float16 else 1e-5
    assert bool(((got - want).abs() <= rtol * want.abs() + 1e-5 * scale + 1e-30).all())
    assert int(torch.count_nonzero(c)) == int(torch.count_nonzero(c.view(m, feat)[d_rows]))


def test_rgms_x_beyond_2_to_32_bytes(dev):
    """70 M nodes: X has 4.5 GB and Y 9 GB, so source rows beyond the 2^32-th byte and destination
    tiles beyond the 2^31-th float are used.  Expected values from per-edge fp64 products by
    torch; everything outside the destination rows stays zero."""
    n = m = 70_000_000
    R, fin, fout = 8, 32, 32
    assert n * fin * 2 > 2**32 and m * fout > 2**31
    rng = np.random.default_rng(23)
    p0, i0, p1, i1 = [0], [], [0], []
    for r in range(R):
        rows = np.unique(_far_ids(rng, 800, m))
        for i in rows:
            cols = np.unique(_far_ids(rng, rng.integers(1, 17), n, replace=True))
            i1.append(cols)
            p1.append(p1[-1] + len(cols))
        i0.append(rows)
        p0.append(p0[-1] + len(rows))
    csf = (np.array(p0, np.int32), np.concatenate(i0).astype(np.int32), np.array(p1, np.int32),
           np.concatenate(i1).astype(np.int32))
    buckets = [1, 2, 4, 8, 16]
    rb = [32 // b for b in buckets]
    ptr, rows, cols, mask = st.csf_to_ell3d(*csf, rb, buckets)
    assert sum(c.size for c in cols) >= 8192  # the destination-tile path
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    triples, mids = [], []
    for k in range(len(buckets)):
        triples += [t(mask[k].astype(np.float16).ravel()), t(rows[k].ravel()), t(cols[k].ravel())]
        mids.append(t(np.repeat(np.arange(R, dtype=np.int32), np.diff(ptr[k]))))
    gen = torch.Generator(device=dev).manual_seed(23)
    x = torch.randn(n * fin, device=dev, generator=gen, dtype=torch.float16)
    w = (torch.randn(R * fin * fout, device=dev, generator=gen) * 0.1).half()
    y = torch.zeros(m * fout, device=dev)
    ops.build_rgms(m, n, R, fin, fout, rb, buckets, [c.shape[0] for c in cols])(w, x, y, *triples, *mids)
    torch.cuda.synchronize()
    # per edge: X[col] @ W[rel], summed per destination row
    rel = np.repeat(np.arange(R), np.diff(csf[0]))           # relation of every stored row
    e_rel = t(np.repeat(rel, np.diff(csf[2])).astype(np.int64))
    e_row = np.repeat(csf[1], np.diff(csf[2]))
    dst, inv = np.unique(e_row, return_inverse=True)
    xe = x.view(n, fin)[t(csf[3]).long()].double()
    we = w.view(R, fin, fout).double()[e_rel]
    prod = torch.bmm(xe[:, None, :], we)[:, 0, :]
    mag = torch.bmm(xe.abs()[:, None, :], we.abs())[:, 0, :]
    want = torch.zeros(len(dst), fout, device=dev, dtype=torch.float64).index_add_(0, t(inv.astype(np.int64)), prod)
    scale = torch.zeros(len(dst), fout, device=dev, dtype=torch.float64).index_add_(0, t(inv.astype(np.int64)), mag)
    d_dst = t(dst.astype(np.int64))
    got = y.view(m, fout)[d_dst].double()
    assert bool(((got - want).abs() <= 2e-2 * want.abs() + 1e-5 * scale + 1e-30).all())
    assert int(torch.count_nonzero(y)) == int(torch.count_nonzero(y.view(m, fout)[d_dst]))

    # the fp32 forms on the same graph (X has 9 GB there): W is laid out [relation, out, in]
    x32 = x.float()
    w32 = w.view(R, fin, fout).float().transpose(1, 2).contiguous().view(-1)
    triples32 = [a.float() if a.dtype == torch.float16 else a for a in triples]
    for form in ("ell3d", "csf"):
        y.zero_()
        if form == "ell3d":
            ops.build_rgms_f32(m, n, R, fin, fout, rb, buckets, [c.shape[0] for c in cols])(
                w32, x32, y, *triples32, *mids)
        else:
            ones = torch.ones(len(csf[3]), device=dev)
            ops.build_rgms_csf(m, n, R, fin, fout, len(csf[1]), len(csf[3]))(
                ones, w32, x32, y, t(csf[0]), t(csf[1]), t(csf[2]), t(csf[3]))
        torch.cuda.synchronize()
        got = y.view(m, fout)[d_dst].double()
        assert bool(((got - want).abs() <= 1e-5 * scale + 1e-30).all()), form
        assert int(torch.count_nonzero(y)) == int(torch.count_nonzero(y.view(m, fout)[d_dst])), form
