"""Host format pass of the product (C ABI, no GPU needed) against the oracle: bit-exact
index arrays on seeded inputs, the golden known-answer vectors, and the error behaviour of
the reference's argument checks (src/sparse/format.cc:56-61, 183-219, 355-360)."""
import numpy as np
import pytest

import oracle
import sparsetir_amd as st
from sparsetir_amd._lib import SparseTIRError
from helpers import load_kats, random_csf, random_csr

KATS = load_kats()


def _same(got, want):
    for gp, wp in zip(got, want):
        for g, w in zip(gp, wp):
            assert g.dtype == np.int32 and g.shape == w.shape
            assert np.array_equal(g, w)


@pytest.mark.parametrize("kat", KATS["column_part_hyb"])
def test_column_part_hyb_known_answers(kat):
    r, c, m = st.column_part_hyb(kat["num_rows"], kat["num_cols"], np.asarray(kat["indptr"], np.int32),
                                 np.asarray(kat["indices"], np.int32), kat["num_col_parts"], kat["buckets"])
    for p in range(kat["num_col_parts"]):
        for b, w in enumerate(kat["buckets"]):
            assert np.array_equal(r[p][b], np.asarray(kat["row_indices"][p][b], np.int32))
            assert np.array_equal(c[p][b], np.asarray(kat["col_indices"][p][b], np.int32).reshape(-1, w))
            assert np.array_equal(m[p][b], np.asarray(kat["mask"][p][b], np.int32).reshape(-1, w))


@pytest.mark.parametrize("sort", [True, False])
@pytest.mark.parametrize("m,n,nnz,parts,buckets,seed", [
    (1000, 1000, 10000, 4, [1, 2, 4], 0),
    (2000, 1500, 60000, 2, [1, 2, 4, 8, 16, 32, 64, 128, 256, 512], 1),
    (513, 77, 9000, 16, [1, 2, 4, 8, 16, 32], 2),
    (100, 100, 0, 3, [1, 2], 3),
    (0, 10, 0, 2, [1, 2], 4),
    (64, 4096, 20000, 5, [3, 5, 9], 5),
    (300, 300, 5000, 1, [1], 6),
    (50, 7, 300, 7, [1, 2, 4], 7),
])
def test_column_part_hyb_matches_oracle(m, n, nnz, parts, buckets, seed, sort):
    indptr, indices = random_csr(m, n, nnz, seed, sort=sort, skew=1.1)
    got = st.column_part_hyb(m, n, indptr, indices, parts, buckets)
    want = oracle.column_part_hyb(m, n, indptr, indices, parts, buckets)
    for g, w in zip(got, want):
        _same(g, w)


def test_column_part_hyb_duplicate_entries():
    indptr = np.asarray([0, 5, 7], np.int32)
    indices = np.asarray([2, 2, 2, 0, 3, 1, 1], np.int32)
    got = st.column_part_hyb(2, 4, indptr, indices, 2, [1, 2])
    want = oracle.column_part_hyb(2, 4, indptr, indices, 2, [1, 2])
    for g, w in zip(got, want):
        _same(g, w)


def test_column_part_hyb_accepts_cpu_torch_tensors():
    import torch

    indptr, indices = random_csr(40, 30, 300, 9)
    got = st.column_part_hyb(40, 30, torch.from_numpy(indptr), torch.from_numpy(indices), 2, [1, 2, 4])
    want = oracle.column_part_hyb(40, 30, indptr, indices, 2, [1, 2, 4])
    for g, w in zip(got, want):
        _same(g, w)


def test_column_part_hyb_errors():
    indptr = np.asarray([0, 1, 2], np.int32)
    with pytest.raises(SparseTIRError, match="int32"):
        st.column_part_hyb(2, 3, indptr.astype(np.int64), np.asarray([0, 1], np.int32), 1, [1])
    with pytest.raises(SparseTIRError, match="int32"):
        st.column_part_hyb(2, 3, indptr, np.asarray([0, 1], np.int64), 1, [1])
    with pytest.raises(SparseTIRError, match="outside"):
        st.column_part_hyb(2, 3, indptr, np.asarray([0, 3], np.int32), 1, [1])
    with pytest.raises(SparseTIRError, match="decreases"):
        st.column_part_hyb(2, 3, np.asarray([0, 2, 1], np.int32), np.asarray([0, 1], np.int32), 1, [1])
    with pytest.raises(SparseTIRError):
        st.column_part_hyb(2, 3, indptr, np.asarray([0, 1], np.int32), 0, [1])
    with pytest.raises(SparseTIRError):
        st.column_part_hyb(2, 3, indptr, np.asarray([0, 1], np.int32), 1, [])


@pytest.mark.parametrize("kat", KATS["csf_to_ell3d"])
def test_csf_to_ell3d_known_answer(kat):
    i32 = lambda x: np.asarray(x, np.int32)
    got = st.csf_to_ell3d(i32(kat["indptr0"]), i32(kat["indices0"]), i32(kat["indptr1"]), i32(kat["indices1"]),
                          kat["rows_bkt"], kat["cols_bkt"])
    for name, g in zip(["indptr", "row_indices", "col_indices", "mask"], got):
        for b, arr in enumerate(g):
            assert np.array_equal(arr, i32(kat[name][b])), (name, b)


@pytest.mark.parametrize("rels,n,edges,rows_bkt,cols_bkt,seed", [
    (3, 30, 200, [4, 2, 1], [1, 2, 4], 0),
    (65, 2000, 40000, [256, 128, 64, 32, 16], [1, 2, 4, 8, 16], 1),
    (7, 100, 3000, [32, 16, 8, 4, 2], [1, 2, 4, 8, 16], 2),
    (4, 20, 100, [3, 5], [2, 3], 3),
    (2, 10, 0, [2, 1], [1, 2], 4),
    (0, 10, 0, [2, 1], [1, 2], 5),
])
def test_csf_to_ell3d_matches_oracle(rels, n, edges, rows_bkt, cols_bkt, seed):
    csf = random_csf(rels, n, edges, seed)
    got = st.csf_to_ell3d(*csf, rows_bkt, cols_bkt)
    want = oracle.csf_to_ell3d(*csf, rows_bkt, cols_bkt)
    for g, w in zip(got, want):
        for a, b in zip(g, w):
            assert a.shape == b.shape and np.array_equal(a, b)


def test_csf_to_ell3d_repeated_row_ids_merge_like_the_reference():
    # two stored rows of one relation with the same row id, adjacent in the same bucket:
    # the reference keeps filling the open ELL row (format.cc:253-262)
    i32 = lambda x: np.asarray(x, np.int32)
    csf = (i32([0, 3]), i32([4, 4, 5]), i32([0, 1, 2, 3]), i32([7, 8, 9]))
    got = st.csf_to_ell3d(*csf, [1, 1], [1, 2])
    want = oracle.csf_to_ell3d(*csf, [1, 1], [1, 2])
    for g, w in zip(got, want):
        for a, b in zip(g, w):
            assert np.array_equal(a, b)


def test_csf_to_ell3d_errors():
    i32 = lambda x: np.asarray(x, np.int32)
    csf = (i32([0, 1]), i32([0]), i32([0, 1]), i32([0]))
    with pytest.raises(SparseTIRError, match="ascending"):
        st.csf_to_ell3d(*csf, [1, 1], [2, 2])
    with pytest.raises(SparseTIRError, match="same length"):
        st.csf_to_ell3d(*csf, [1], [1, 2])
    with pytest.raises(SparseTIRError, match="int32"):
        st.csf_to_ell3d(csf[0].astype(np.int64), *csf[1:], [1], [1])


@pytest.mark.parametrize("kat", KATS["condense"])
def test_condense_known_answer(kat):
    gptr, tiles, mask = st.condense(np.asarray(kat["indptr"], np.int32), np.asarray(kat["indices"], np.int32),
                                    kat["t"], kat["g"])
    assert np.array_equal(gptr, kat["group_indptr"])
    assert np.array_equal(tiles, kat["tile_indices"])
    assert np.array_equal(mask, kat["mask"])


@pytest.mark.parametrize("m,n,nnz,t,g,seed", [
    (1000, 1000, 10000, 4, 1, 0), (333, 200, 3000, 8, 4, 1), (50, 40, 0, 4, 2, 2),
    (129, 64, 4000, 16, 8, 3), (7, 9, 30, 3, 5, 4), (0, 5, 0, 4, 1, 5),
])
def test_condense_matches_oracle(m, n, nnz, t, g, seed):
    indptr, indices = random_csr(m, n, nnz, seed, sort=(seed % 2 == 0))
    got = st.condense(indptr, indices, t, g)
    want = oracle.condense(indptr, indices, t, g)
    for a, b in zip(got, want):
        assert a.shape == b.shape and np.array_equal(a, b)


def test_on_disk_cache_round_trip(tmp_path):
    from sparsetir_amd.cache import cached_column_part_hyb

    indptr, indices = random_csr(300, 200, 4000, 12, skew=1.0)
    first = cached_column_part_hyb(str(tmp_path), 300, 200, indptr, indices, 2, [1, 2, 4])
    assert len(list(tmp_path.iterdir())) == 1
    again = cached_column_part_hyb(str(tmp_path), 300, 200, indptr, indices, 2, [1, 2, 4])
    want = oracle.column_part_hyb(300, 200, indptr, indices, 2, [1, 2, 4])
    for a, b, c in zip(first, again, want):
        _same(a, c)
        _same(b, c)
    cached_column_part_hyb(str(tmp_path), 300, 200, indptr, indices, 2, [1, 2])  # other parameters: new entry
    assert len(list(tmp_path.iterdir())) == 2


def test_on_disk_cache_ell3d_and_condense(tmp_path):
    from sparsetir_amd.cache import cached_condense, cached_csf_to_ell3d

    R, n = 5, 60
    rng = np.random.default_rng(4)
    ptr0, idx0, ptr1, idx1 = [0], [], [0], []
    for r in range(R):
        rows = np.sort(rng.choice(n, rng.integers(0, 20), replace=False))
        for i in rows:
            cols = np.sort(rng.choice(n, rng.integers(1, 9), replace=False))
            idx0.append(i)
            idx1.extend(cols)
            ptr1.append(len(idx1))
        ptr0.append(len(idx0))
    csf = [np.asarray(a, np.int32) for a in (ptr0, idx0, ptr1, idx1)]
    rb, cb = [8, 4, 2], [1, 2, 4]
    want = oracle.csf_to_ell3d(*csf, rb, cb)
    first = cached_csf_to_ell3d(str(tmp_path), *csf, rb, cb)
    again = cached_csf_to_ell3d(str(tmp_path), *csf, rb, cb)
    assert len(list(tmp_path.iterdir())) == 1
    for q in range(4):
        for b in range(len(cb)):
            assert np.array_equal(first[q][b], want[q][b])
            assert again[q][b].dtype == np.int32 and again[q][b].shape == want[q][b].shape
            assert np.array_equal(again[q][b], want[q][b])
    indptr, indices = random_csr(90, 70, 900, 3)
    want = oracle.condense(indptr, indices, 8, 4)
    first = cached_condense(str(tmp_path), indptr, indices, 8, 4)
    again = cached_condense(str(tmp_path), indptr, indices, 8, 4)
    assert len(list(tmp_path.iterdir())) == 2
    for a, b, c in zip(first, again, want):
        assert np.array_equal(a, c) and np.array_equal(b, c) and b.shape == c.shape


def test_on_disk_cache_ignores_a_damaged_file(tmp_path):
    from sparsetir_amd.cache import cached_column_part_hyb

    indptr, indices = random_csr(50, 40, 300, 2)
    cached_column_part_hyb(str(tmp_path), 50, 40, indptr, indices, 1, [1, 2])
    (path,) = list(tmp_path.iterdir())
    path.write_bytes(b"not an archive")
    got = cached_column_part_hyb(str(tmp_path), 50, 40, indptr, indices, 1, [1, 2])
    want = oracle.column_part_hyb(50, 40, indptr, indices, 1, [1, 2])
    for a, c in zip(got, want):
        _same(a, c)
    again = cached_column_part_hyb(str(tmp_path), 50, 40, indptr, indices, 1, [1, 2])  # rewritten and readable
    for a, c in zip(again, want):
        _same(a, c)


def test_suggest_decomposition():
    """The decomposition chooser (counterpart of the reference's col_part_config / bucketing_config
    tables, examples/spmm/bench_spmm.py:233-253): one partition, power-of-two widths up to 512 or
    the first one that covers the column count; its output feeds column_part_hyb as it is."""
    import sparsetir_amd as st
    from sparsetir_amd._lib import SparseTIRError
    assert st.suggest_decomposition(2449029, 2449029, 61833585, 128) == (1, [1, 2, 4, 8, 16, 32, 64, 128, 256, 512])
    assert st.suggest_decomposition(100, 5, 200, 32) == (1, [1, 2, 4, 8])
    assert st.suggest_decomposition(3, 1, 3, 4) == (1, [1])
    with pytest.raises(SparseTIRError):
        st.suggest_decomposition(10, 0, 5, 32)
    m, n = 40, 37
    indptr, indices = random_csr(m, n, 300, 3)
    parts, buckets = st.suggest_decomposition(m, n, len(indices), 64)
    rows, cols, mask = st.column_part_hyb(m, n, indptr, indices, parts, buckets)
    assert len(rows) == 1 and len(rows[0]) == len(buckets)
    assert sum(int(k.sum()) for k in mask[0]) == len(indices)
