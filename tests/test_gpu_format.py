"""Device-side format passes (ColumnPartHyb, CSFToELL3D, CSR to BSR): index arrays bit-exact with
the oracle."""
import numpy as np
import pytest
import torch

import oracle
import sparsetir_amd as st
from sparsetir_amd import datasets
from sparsetir_amd._lib import SparseTIRError
from helpers import coo_pairs, decode_hyb, random_csf, random_csr

pytestmark = pytest.mark.gpu


def _device_hyb(dev, m, n, indptr, indices, parts, buckets):
    r, c, k = st.column_part_hyb(m, n, torch.from_numpy(indptr).to(dev), torch.from_numpy(indices).to(dev),
                                 parts, buckets)
    tonp = lambda nest: [[a.cpu().numpy() for a in p] for p in nest]
    return tonp(r), tonp(c), tonp(k)


@pytest.mark.parametrize("m,n,nnz,parts,buckets,seed", [
    (1000, 1000, 10000, 4, [1, 2, 4], 0),
    (2000, 1500, 60000, 2, [1, 2, 4, 8, 16, 32, 64, 128, 256, 512], 1),
    (513, 77, 9000, 16, [1, 2, 4, 8, 16, 32], 2),
    (100, 100, 0, 3, [1, 2], 3),
    (64, 4096, 20000, 5, [3, 5, 9], 5),
    (300, 300, 5000, 1, [1], 6),
    (50, 7, 300, 7, [1, 2, 4], 7),
    (63, 63, 900, 2, [1, 2, 4, 8], 8),
    (65, 200, 5000, 3, [1, 2], 9),
    # one partition, tiles with few rows next to tiles with hundreds (both placement paths in
    # one workgroup)
    (20000, 500, 30000, 1, [1, 2, 4, 8], 10),
    (50000, 500, 70000, 1, [1, 2, 4, 8], 11),
    (2000, 2000, 150000, 1, [1, 2, 4, 8, 16, 32], 12),
])
def test_device_column_part_hyb_bit_exact(dev, m, n, nnz, parts, buckets, seed):
    indptr, indices = random_csr(m, n, nnz, seed, skew=1.1)
    got = _device_hyb(dev, m, n, indptr, indices, parts, buckets)
    want = oracle.column_part_hyb(m, n, indptr, indices, parts, buckets)
    for name, g, w in zip(["rows", "cols", "mask"], got, want):
        for p in range(parts):
            for b in range(len(buckets)):
                assert g[p][b].shape == w[p][b].shape, (name, p, b)
                assert np.array_equal(g[p][b], w[p][b]), (name, p, b)


def test_device_column_part_hyb_config2(dev):
    g = datasets.config2()
    got = _device_hyb(dev, g["m"], g["n"], g["indptr"], g["indices"], g["num_col_parts"], g["buckets"])
    want = oracle.column_part_hyb(g["m"], g["n"], g["indptr"], g["indices"], g["num_col_parts"], g["buckets"])
    for gq, wq in zip(got, want):
        for gp, wp in zip(gq, wq):
            for a, b in zip(gp, wp):
                assert np.array_equal(a, b)
    assert np.array_equal(decode_hyb(*got), coo_pairs(g["indptr"], g["indices"]))


def test_device_column_part_hyb_one_partition_takes_unsorted_rows(dev):
    """With one partition a (row, partition) run is the whole row, so the column order inside
    rows does not matter: same arrays as the sequential routine."""
    for m, n, nnz, buckets, seed in [(50, 40, 600, [1, 2, 4], 3), (3000, 900, 90000, [1, 2, 4, 8, 16, 32], 4)]:
        indptr, indices = random_csr(m, n, nnz, seed, sort=False, skew=1.0)
        got = _device_hyb(dev, m, n, indptr, indices, 1, buckets)
        want = oracle.column_part_hyb(m, n, indptr, indices, 1, buckets)
        for gq, wq in zip(got, want):
            for a, b in zip(gq[0], wq[0]):
                assert np.array_equal(a, b)


def _assert_same(got, want):
    for gq, wq in zip(got, want):
        for gp, wp in zip(gq, wq):
            for a, b in zip(gp, wp):
                assert a.shape == b.shape and np.array_equal(a, b)


@pytest.mark.parametrize("m,n,nnz,parts,buckets,seed", [
    (50, 40, 600, 2, [1, 2, 4], 3),
    (3000, 900, 90000, 4, [1, 2, 4, 8, 16, 32], 4),
    (700, 5000, 40000, 16, [1, 2, 4, 8], 5),
    (20000, 300, 30000, 3, [1, 2], 6),
])
def test_device_column_part_hyb_unsorted_rows_with_partitions(dev, m, n, nnz, parts, buckets, seed):
    """Rows in arbitrary column order and several partitions: the device pass regroups the
    nonzeros by (row, partition) with a stable sort and must give the sequential routine's arrays
    (every run keeps the CSR order of its entries)."""
    indptr, indices = random_csr(m, n, nnz, seed, sort=False, skew=1.0)
    got = _device_hyb(dev, m, n, indptr, indices, parts, buckets)
    _assert_same(got, oracle.column_part_hyb(m, n, indptr, indices, parts, buckets))


def test_device_column_part_hyb_partition_ordered_rows(dev):
    """Columns shuffled inside every (row, partition) run but the runs in partition order: the
    fast path applies (its row searches only compare partitions) and must stay bit-exact."""
    m, n, parts, buckets = 800, 640, 4, [1, 2, 4, 8, 16]
    indptr, indices = random_csr(m, n, 30000, 21, sort=False, skew=1.0)
    psize = (n + parts - 1) // parts
    for i in range(m):
        seg = indices[indptr[i]:indptr[i + 1]]
        seg[:] = seg[np.argsort(seg // psize, kind="stable")]
    got = _device_hyb(dev, m, n, indptr, indices, parts, buckets)
    _assert_same(got, oracle.column_part_hyb(m, n, indptr, indices, parts, buckets))


def test_device_column_part_hyb_one_swapped_pair(dev):
    """One swapped pair inside one row, across a partition boundary (every other row ascending):
    the regrouping path must be taken -- found through the descent counts -- and be bit-exact."""
    m, n, parts, buckets = 400, 300, 2, [1, 2, 4]
    indptr, indices = random_csr(m, n, 6000, 11, skew=1.0)
    psize = (n + parts - 1) // parts
    for row in range(m):
        seg = indices[indptr[row]:indptr[row + 1]]
        cut = np.searchsorted(seg, psize)
        if 0 < cut < len(seg):
            e = indptr[row] + cut
            break
    swapped = indices.copy()
    swapped[e - 1], swapped[e] = indices[e], indices[e - 1]
    got = _device_hyb(dev, m, n, indptr, swapped, parts, buckets)
    want = oracle.column_part_hyb(m, n, indptr, swapped, parts, buckets)
    _assert_same(got, want)


def test_device_column_part_hyb_unsorted_value_rewrite(dev):
    m, n, parts, buckets = 600, 500, 3, [1, 2, 4, 8]
    indptr, indices = random_csr(m, n, 12000, 14, sort=False, skew=1.0)
    vals = np.random.default_rng(14).random(len(indices), dtype=np.float32) + 0.5
    t = lambda a: torch.from_numpy(a).to(dev)
    rows, cols, mask, avals = st.column_part_hyb(m, n, t(indptr), t(indices), parts, buckets, values=t(vals))
    import scipy.sparse as sp
    dense = sp.csr_matrix((vals, indices, indptr), shape=(m, n)).toarray()
    for p in range(parts):
        for b in range(len(buckets)):
            r, c = rows[p][b].cpu().numpy(), cols[p][b].cpu().numpy()
            k, a = mask[p][b].cpu().numpy(), avals[p][b].cpu().numpy()
            if len(r):
                assert np.array_equal(a, (dense[np.repeat(r[:, None], c.shape[1], 1), c] * k).astype(np.float32))


def test_device_column_part_hyb_rejects_bad_input(dev):
    bad = np.asarray([0, 50], np.int32)
    with pytest.raises(SparseTIRError, match="outside"):
        _device_hyb(dev, 2, 40, np.asarray([0, 1, 2], np.int32), bad, 2, [1, 2])
    indptr, indices = random_csr(400, 300, 6000, 11, skew=1.0)
    with pytest.raises(SparseTIRError, match="row pointer"):
        ptr = indptr.copy()
        ptr[10] = ptr[11] + 1
        _device_hyb(dev, 400, 300, ptr, indices, 2, [1, 2, 4])


def test_device_column_part_hyb_mostly_empty_rows_and_offset_row_pointer(dev):
    m, n = 6000, 500
    indptr, indices = random_csr(m, n, 400, 12, skew=2.0)
    got = _device_hyb(dev, m, n, indptr, indices, 3, [1, 2, 4])
    want = oracle.column_part_hyb(m, n, indptr, indices, 3, [1, 2, 4])
    for gq, wq in zip(got, want):
        for gp, wp in zip(gq, wq):
            for a, b in zip(gp, wp):
                assert np.array_equal(a, b)
    # a row pointer that does not start at zero: rows 100.. of a larger matrix, same indices array
    big_ptr, big_idx = random_csr(900, 300, 20000, 13, skew=1.0)
    sub = big_ptr[100:].copy()
    got = _device_hyb(dev, 800, 300, sub, big_idx, 2, [1, 2, 4, 8])
    want = oracle.column_part_hyb(800, 300, sub - sub[0], big_idx[sub[0]:], 2, [1, 2, 4, 8])
    for gq, wq in zip(got, want):
        for gp, wp in zip(gq, wq):
            for a, b in zip(gp, wp):
                assert np.array_equal(a, b)


def test_device_hyb_value_rewrite(dev):
    """A_k gathered on the device equals the values placed by the decomposition's own index
    arrays: A_k[r, s] = value of nonzero (rows_k[r], cols_k[r, s]) where mask is 1, else 0."""
    import scipy.sparse as sp

    m = n = 700
    parts, buckets = 3, [1, 2, 4, 8]
    indptr, indices = random_csr(m, n, 12000, 4, skew=1.1)
    vals = np.random.default_rng(4).random(len(indices), dtype=np.float32) + 0.5
    t = lambda a: torch.from_numpy(a).to(dev)
    rows, cols, mask, avals = st.column_part_hyb(m, n, t(indptr), t(indices), parts, buckets, values=t(vals))
    dense = sp.csr_matrix((vals, indices, indptr), shape=(m, n)).toarray()
    for p in range(parts):
        for b in range(len(buckets)):
            r, c = rows[p][b].cpu().numpy(), cols[p][b].cpu().numpy()
            k, a = mask[p][b].cpu().numpy(), avals[p][b].cpu().numpy()
            if len(r) == 0:
                continue
            want = dense[np.repeat(r[:, None], c.shape[1], 1), c] * k
            assert np.array_equal(a, want.astype(np.float32))


@pytest.mark.parametrize("m,n,blk,nnz,seed", [(256, 256, 32, 3000, 0), (4096, 4096, 32, 200000, 1),
                                             (128, 512, 16, 900, 2), (64, 64, 64, 50, 3), (96, 160, 32, 0, 4),
                                             (2048, 8192, 64, 100000, 5)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_device_csr_to_bsr_matches_scipy(dev, m, n, blk, nnz, seed, dtype):
    import scipy.sparse as sp

    indptr, indices = random_csr(m, n, nnz, seed, sort=(seed % 2 == 0), skew=0.5)
    vals = np.random.default_rng(seed).standard_normal(len(indices)).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev)
    bptr, bidx, bdata = st.csr_to_bsr(t(indptr), t(indices), t(vals), (m, n), blk, dtype)
    ref = sp.csr_matrix((vals, indices, indptr), shape=(m, n)).tobsr((blk, blk))
    ref.sort_indices()
    assert np.array_equal(bptr.cpu().numpy(), ref.indptr.astype(np.int32))
    assert np.array_equal(bidx.cpu().numpy(), ref.indices.astype(np.int32))
    want = torch.from_numpy(ref.data.astype(np.float32)).to(dtype)
    assert torch.equal(bdata.cpu(), want.reshape(bdata.shape))


def test_device_csr_to_bsr_feeds_the_bsr_operator(dev):
    from sparsetir_amd import ops
    import scipy.sparse as sp

    m = n = 1024
    blk, feat = 32, 64
    indptr, indices = random_csr(m, n, 30000, 9)
    vals = (np.random.default_rng(9).standard_normal(len(indices)) * 0.1).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev)
    bptr, bidx, bdata = st.csr_to_bsr(t(indptr), t(indices), t(vals), (m, n), blk, torch.float16)
    x = torch.randn(n * feat, device=dev).half()
    y = torch.zeros(m * feat, device=dev, dtype=torch.float32)
    ops.build_bsrmm(m // blk, n // blk, bidx.numel(), blk, feat, torch.float16, torch.float32)(
        bdata.reshape(-1), x, y, bptr, bidx)
    torch.cuda.synchronize()
    a16 = sp.csr_matrix((vals.astype(np.float16).astype(np.float64), indices, indptr), shape=(m, n))
    want = a16 @ x.float().cpu().numpy().astype(np.float64).reshape(n, feat)
    assert np.allclose(y.cpu().numpy().reshape(m, feat), want, rtol=2e-2, atol=1e-3)


def test_device_csr_to_bsr_errors(dev):
    z = lambda k, dt: torch.zeros(k, dtype=dt, device=dev)
    with pytest.raises(SparseTIRError, match="multiple"):
        st.csr_to_bsr(z(101, torch.int32), z(0, torch.int32), z(0, torch.float32), (100, 64), 32)
    with pytest.raises(SparseTIRError, match="outside"):
        st.csr_to_bsr(torch.tensor([0, 1] + [1] * 31, dtype=torch.int32, device=dev),
                      torch.tensor([99], dtype=torch.int32, device=dev), z(1, torch.float32), (32, 64), 32)


def test_on_disk_cache_of_a_device_decomposition_feeds_the_hyb_operator(dev, tmp_path):
    """A decomposition computed on the GPU is stored as host arrays; a later call (another
    process in practice) gets device arrays back that equal the oracle's bit for bit and that the
    hyb operator takes as they are."""
    from sparsetir_amd import ops
    from sparsetir_amd.cache import cached_column_part_hyb
    from helpers import spmm_f64

    m = n = 2500
    parts, buckets, feat = 2, [1, 2, 4, 8], 64
    indptr, indices = random_csr(m, n, 40000, 9, skew=1.1)
    t = lambda a: torch.from_numpy(a).to(dev)
    first = cached_column_part_hyb(str(tmp_path), m, n, t(indptr), t(indices), parts, buckets)
    assert len(list(tmp_path.iterdir())) == 1
    again = cached_column_part_hyb(str(tmp_path), m, n, t(indptr), t(indices), parts, buckets)
    assert len(list(tmp_path.iterdir())) == 1
    want = oracle.column_part_hyb(m, n, indptr, indices, parts, buckets)
    for q in range(3):
        for p in range(parts):
            for b in range(len(buckets)):
                assert again[q][p][b].is_cuda and again[q][p][b].dtype == torch.int32
                assert np.array_equal(first[q][p][b].cpu().numpy(), want[q][p][b])
                assert np.array_equal(again[q][p][b].cpu().numpy(), want[q][p][b])
    rows, cols, mask = again
    triples, nrows = [], []
    for p in range(parts):
        for b in range(len(buckets)):
            triples += [mask[p][b].reshape(-1).float(), rows[p][b], cols[p][b].reshape(-1)]
            nrows.append(int(rows[p][b].shape[0]))
    x = np.random.default_rng(1).standard_normal((n, feat), dtype=np.float32)
    c = torch.zeros(m * feat, device=dev)
    ops.build_hyb_csrmm(m, n, feat, parts, buckets, nrows)(t(x.ravel()), c, *triples)
    torch.cuda.synchronize()
    ones = np.ones(len(indices), np.float32)
    exact = spmm_f64(indptr, indices, ones, x)
    scale = spmm_f64(indptr, indices, ones, np.abs(x))
    assert np.all(np.abs(c.cpu().numpy().reshape(m, feat) - exact) <= 1e-5 * scale + 1e-30)
    # a host-side call on the same matrix shares the entry
    host = cached_column_part_hyb(str(tmp_path), m, n, indptr, indices, parts, buckets)
    assert len(list(tmp_path.iterdir())) == 1
    assert isinstance(host[0][0][0], np.ndarray) and np.array_equal(host[1][1][2], want[1][1][2])


# ------------------------------------------------------------------------------- CSFToELL3D

def _device_ell3d(dev, csf, rows_bkt, cols_bkt):
    got = st.csf_to_ell3d(*[torch.from_numpy(a).to(dev) for a in csf], rows_bkt, cols_bkt)
    assert all(a.is_cuda for kind in got for a in kind)
    return [[a.cpu().numpy() for a in kind] for kind in got]


def _assert_same_ell3d(got, want):
    for name, g, w in zip(["indptr", "rows", "cols", "mask"], got, want):
        assert len(g) == len(w)
        for b, (a, c) in enumerate(zip(g, w)):
            assert a.shape == c.shape, (name, b, a.shape, c.shape)
            assert np.array_equal(a, c), (name, b)


@pytest.mark.parametrize("rels,n,edges,rows_bkt,cols_bkt,seed", [
    (3, 30, 200, [4, 2, 1], [1, 2, 4], 0),
    (65, 2000, 40000, [256, 128, 64, 32, 16], [1, 2, 4, 8, 16], 1),
    (7, 100, 3000, [32, 16, 8, 4, 2], [1, 2, 4, 8, 16], 2),   # rows longer than the widest bucket
    (4, 20, 100, [3, 5], [2, 3], 3),                          # widths that are not powers of two
    (2, 10, 0, [2, 1], [1, 2], 4),                            # no edges
    (0, 10, 0, [2, 1], [1, 2], 5),                            # no relations
    (300, 5000, 100000, [64, 8, 1], [1, 8, 64], 6),           # more relations than a workgroup scans at once
    (5, 40000, 300000, [128], [3], 7),                        # one bucket, every row split or padded
    (1, 3, 9, [7, 7], [1, 2], 8),
])
def test_device_csf_to_ell3d_bit_exact(dev, rels, n, edges, rows_bkt, cols_bkt, seed):
    csf = random_csf(rels, n, edges, seed)
    got = _device_ell3d(dev, csf, rows_bkt, cols_bkt)
    _assert_same_ell3d(got, oracle.csf_to_ell3d(*csf, rows_bkt, cols_bkt))


def test_device_csf_to_ell3d_empty_relations_and_hub_rows(dev):
    """Relations without rows at the start, in the middle and at the end, a stored row with
    thousands of columns (one thread of the row pass, many of the entry pass) and stored rows
    without columns."""
    rng = np.random.default_rng(3)
    n = 6000
    indptr0, indices0, indptr1, indices1 = [0], [], [0], []
    for r in range(9):
        rows = [] if r in (0, 4, 8) else sorted(rng.choice(n, size=int(rng.integers(1, 40)), replace=False).tolist())
        for q, row in enumerate(rows):
            cnt = 5000 if (r == 2 and q == 0) else (0 if q % 7 == 3 else int(rng.integers(1, 30)))
            indices1 += sorted(rng.choice(n, size=cnt, replace=False).tolist())
            indptr1.append(len(indices1))
        indices0 += rows
        indptr0.append(len(indices0))
    csf = tuple(np.asarray(a, np.int32) for a in (indptr0, indices0, indptr1, indices1))
    for rows_bkt, cols_bkt in (([16, 8, 4], [1, 4, 16]), ([5], [7]), ([1, 1, 1, 1], [1, 2, 3, 4])):
        got = _device_ell3d(dev, csf, rows_bkt, cols_bkt)
        _assert_same_ell3d(got, oracle.csf_to_ell3d(*csf, rows_bkt, cols_bkt))


def test_device_csf_to_ell3d_config5(dev):
    cfg = datasets.config5()
    csf = (cfg["indptr0"], cfg["indices0"], cfg["indptr1"], cfg["indices1"])
    rows_bkt = [256 // b for b in cfg["buckets"]]
    got = _device_ell3d(dev, csf, rows_bkt, cfg["buckets"])
    _assert_same_ell3d(got, oracle.csf_to_ell3d(*csf, rows_bkt, cfg["buckets"]))


def test_device_csf_to_ell3d_errors(dev):
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    good = (i32([0, 2]), i32([1, 4]), i32([0, 1, 3]), i32([0, 2, 3]))
    st.csf_to_ell3d(*good, [1, 1], [1, 2])
    with pytest.raises(SparseTIRError, match="ascending"):
        st.csf_to_ell3d(*good, [1, 1], [2, 2])
    with pytest.raises(SparseTIRError, match="same length"):
        st.csf_to_ell3d(*good, [1], [1, 2])
    with pytest.raises(SparseTIRError, match="int32"):
        st.csf_to_ell3d(good[0].long(), *good[1:], [1], [1])
    with pytest.raises(SparseTIRError, match="CUDA"):
        st.csf_to_ell3d(good[0].cpu(), *good[1:], [1], [1])
    # the same row id twice in a relation: the sequential rule would let the two share an ELL row
    with pytest.raises(SparseTIRError, match="ascend strictly"):
        st.csf_to_ell3d(i32([0, 2]), i32([4, 4]), good[2], good[3], [1, 1], [1, 2])
    with pytest.raises(SparseTIRError, match="indptr1 decreases"):
        st.csf_to_ell3d(good[0], good[1], i32([0, 4, 3]), good[3], [1, 1], [1, 2])
    with pytest.raises(SparseTIRError, match="do not fit"):
        st.csf_to_ell3d(i32([0, 1]), good[1], good[2], good[3], [1, 1], [1, 2])
    with pytest.raises(SparseTIRError, match="indptr0 decreases"):
        st.csf_to_ell3d(i32([0, 3, 2]), good[1], good[2], good[3], [1, 1], [1, 2])


# ------------------------------------------------------------------------------- ConDense

@pytest.mark.parametrize("m,n,nnz,t,g,seed,skew", [
    (130, 90, 2000, 8, 4, 0, 0.0),
    (1000, 1000, 30000, 32, 16, 1, 1.2),     # the setting of the tensor-core SpMM
    (77, 5000, 9000, 1, 1, 2, 1.0),          # tiles of one row, groups of one column
    (513, 40, 12000, 64, 3, 3, 0.0),         # nearly every column in every tile
    (100, 100, 0, 4, 4, 4, 0.0),             # no nonzeros
    (5, 7, 20, 32, 16, 5, 0.0),              # one partial tile
    (20000, 3000, 200000, 32, 16, 6, 1.5),   # a tile with thousands of distinct columns
])
def test_device_condense_bit_exact(dev, m, n, nnz, t, g, seed, skew):
    indptr, indices = random_csr(m, n, nnz, seed, skew=skew, sort=seed % 2 == 0)
    got = st.condense(torch.from_numpy(indptr).to(dev), torch.from_numpy(indices).to(dev), t, g)
    assert all(a.is_cuda for a in got)
    want = oracle.condense(indptr, indices, t, g)
    for name, a, b in zip(["group_indptr", "tile_indices", "mask"], got, want):
        a = a.cpu().numpy()
        assert a.shape == b.shape, (name, a.shape, b.shape)
        assert np.array_equal(a, b), name


def test_device_condense_config2_graph_and_errors(dev):
    g2 = datasets.config2()
    got = st.condense(torch.from_numpy(g2["indptr"]).to(dev), torch.from_numpy(g2["indices"]).to(dev), 32, 16)
    want = oracle.condense(g2["indptr"], g2["indices"], 32, 16)
    for a, b in zip(got, want):
        assert np.array_equal(a.cpu().numpy(), b)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    with pytest.raises(SparseTIRError, match="positive"):
        st.condense(i32([0, 1]), i32([0]), 0, 4)
    with pytest.raises(SparseTIRError, match="int32"):
        st.condense(i32([0, 1]).long(), i32([0]), 4, 4)
    with pytest.raises(SparseTIRError, match="indptr decreases"):
        st.condense(i32([0, 2, 1, 3]), i32([0, 1, 2]), 4, 4)
    with pytest.raises(SparseTIRError, match="from 0 to the number of nonzeros"):
        st.condense(i32([0, 1, 2]), i32([0, 1, 2]), 4, 4)
    with pytest.raises(SparseTIRError, match="negative"):
        st.condense(i32([0, 1, 2]), i32([3, -1]), 4, 4)


def test_on_disk_cache_of_device_ell3d_and_condensed_formats(dev, tmp_path):
    """CUDA inputs: computed on the GPU on a miss, uploaded from disk on a hit, the same arrays
    (the oracle's) both times, and one file per decomposition whoever asked first."""
    from sparsetir_amd.cache import cached_condense, cached_csf_to_ell3d
    t = lambda a: torch.from_numpy(a).to(dev)
    csf = random_csf(6, 300, 5000, 2)
    rb, cb = [8, 4, 2], [1, 2, 4]
    want = oracle.csf_to_ell3d(*csf, rb, cb)
    for turn in range(2):
        got = cached_csf_to_ell3d(str(tmp_path), *[t(a) for a in csf], rb, cb)
        assert all(a.is_cuda for kind in got for a in kind)
        _assert_same_ell3d([[a.cpu().numpy() for a in kind] for kind in got], want)
    host = cached_csf_to_ell3d(str(tmp_path), *csf, rb, cb)  # a host caller hits the file the GPU wrote
    _assert_same_ell3d(host, want)
    assert len(list(tmp_path.iterdir())) == 1
    indptr, indices = random_csr(400, 300, 6000, 3, skew=1.0)
    want = oracle.condense(indptr, indices, 32, 16)
    for turn in range(2):
        got = cached_condense(str(tmp_path), t(indptr), t(indices), 32, 16)
        for a, b in zip(got, want):
            assert a.is_cuda and np.array_equal(a.cpu().numpy(), b)
    assert len(list(tmp_path.iterdir())) == 2
