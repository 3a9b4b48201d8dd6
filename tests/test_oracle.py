"""Pins the CPU oracle (oracle/) against checks that do not share its code:
hand-traced known-answer vectors, restatements of the comparators the reference's own tests
use, pure-Python closed forms on small inputs, decode/padding invariants, and float64
scipy/numpy closed forms for the numeric kernels."""
import numpy as np
import pytest

import oracle
from helpers import (assert_close, brute_force_column_part_hyb, brute_force_csf_to_ell3d, bsr_f64,
                     coo_pairs, decode_hyb, load_kats, numpy_condense_g1, random_csf, random_csr,
                     rgms_f64, scipy_style_column_part_hyb, sddmm_f64, spmm_f64)

KATS = load_kats()


def _eq_nested(got, want, widths=None):
    for p, (gp, wp) in enumerate(zip(got, want)):
        for b, (g, w) in enumerate(zip(gp, wp)):
            w = np.asarray(w, np.int32)
            if widths is not None and w.size == 0:
                w = w.reshape(0, widths[b])
            assert g.dtype == np.int32
            assert g.shape == w.shape, (p, b, g.shape, w.shape)
            assert np.array_equal(g, w), (p, b)


@pytest.mark.parametrize("kat", KATS["column_part_hyb"])
def test_column_part_hyb_known_answers(kat):
    r, c, m = oracle.column_part_hyb(kat["num_rows"], kat["num_cols"], kat["indptr"], kat["indices"],
                                     kat["num_col_parts"], kat["buckets"])
    _eq_nested(r, kat["row_indices"])
    _eq_nested(c, kat["col_indices"], kat["buckets"])
    _eq_nested(m, kat["mask"], kat["buckets"])


@pytest.mark.parametrize("m,n,nnz,parts,buckets,seed", [
    (1000, 1000, 10000, 4, [1, 2, 4], 0),      # the reference test's shape and parameters
    (300, 500, 4000, 3, [1, 2, 4, 8], 1),
    (64, 64, 2000, 1, [1, 2, 4, 8, 16], 2),
    (200, 50, 3000, 2, [2, 3, 7], 3),          # widths that are not powers of two
])
def test_column_part_hyb_vs_reference_test_comparator(m, n, nnz, parts, buckets, seed):
    indptr, indices = random_csr(m, n, nnz, seed, skew=0.8)
    r, c, _ = oracle.column_part_hyb(m, n, indptr, indices, parts, buckets)
    rs, cs = scipy_style_column_part_hyb(indptr, indices, m, n, parts, buckets)
    nb = len(buckets)
    for p in range(parts):
        for b in range(nb):
            assert np.array_equal(r[p][b], rs[p * nb + b])
            assert np.array_equal(c[p][b], cs[p * nb + b])


@pytest.mark.parametrize("sort", [True, False])
@pytest.mark.parametrize("m,n,nnz,parts,buckets,seed", [
    (40, 37, 300, 3, [1, 2, 4], 10),
    (25, 90, 500, 4, [1, 4, 16], 11),
    (10, 10, 0, 2, [1, 2], 12),
    (8, 200, 700, 1, [1], 13),
    (30, 30, 400, 30, [1, 2], 14),
])
def test_column_part_hyb_vs_brute_force(m, n, nnz, parts, buckets, seed, sort):
    indptr, indices = random_csr(m, n, nnz, seed, sort=sort, skew=0.5)
    got = oracle.column_part_hyb(m, n, indptr, indices, parts, buckets)
    want = brute_force_column_part_hyb(indptr, indices, m, n, parts, buckets)
    for g, w in zip(got, want):
        _eq_nested(g, w)


def test_column_part_hyb_invariants():
    m = n = 500
    parts, buckets = 4, [1, 2, 4, 8]
    indptr, indices = random_csr(m, n, 9000, 21, skew=1.0)
    rows, cols, mask = oracle.column_part_hyb(m, n, indptr, indices, parts, buckets)
    psize = (n + parts - 1) // parts
    assert np.array_equal(decode_hyb(rows, cols, mask), coo_pairs(indptr, indices))
    for p in range(parts):
        for b, w in enumerate(buckets):
            r, c, k = rows[p][b], cols[p][b], mask[p][b]
            assert c.shape == (len(r), w) and k.shape == c.shape
            assert set(np.unique(k)) <= {0, 1}
            assert np.all(c[k == 0] == 0)
            assert np.all((c[k == 1] // psize) == p)
            # mask is a prefix of ones in every ELL row, never empty
            assert np.all(np.diff(k, axis=1) <= 0) and (len(r) == 0 or np.all(k[:, 0] == 1))
            assert np.all(np.diff(r) >= 0)
            if b < len(buckets) - 1:
                assert np.all(np.diff(r) > 0)  # one ELL row per row outside the last bucket
                cnt = k.sum(axis=1)
                lower = 0 if b == 0 else buckets[b - 1]
                assert np.all((cnt > lower) & (cnt <= w))
            else:
                same = np.nonzero(np.diff(r) == 0)[0]
                assert np.all(k[same].sum(axis=1) == w)  # all but the last chunk of a row are full


def test_column_part_hyb_rejects_bad_column():
    with pytest.raises(ValueError):
        oracle.column_part_hyb(2, 3, [0, 1, 2], [0, 3], 1, [1, 2])


@pytest.mark.parametrize("kat", KATS["csf_to_ell3d"])
def test_csf_to_ell3d_known_answer(kat):
    got = oracle.csf_to_ell3d(kat["indptr0"], kat["indices0"], kat["indptr1"], kat["indices1"],
                              kat["rows_bkt"], kat["cols_bkt"])
    for name, g in zip(["indptr", "row_indices", "col_indices", "mask"], got):
        for b, arr in enumerate(g):
            assert np.array_equal(arr, np.asarray(kat[name][b], np.int32)), (name, b)


@pytest.mark.parametrize("rels,n,edges,rows_bkt,cols_bkt,seed", [
    (3, 30, 200, [4, 2, 1], [1, 2, 4], 0),
    (5, 50, 600, [8, 4, 2, 1], [1, 2, 4, 8], 1),
    (4, 20, 100, [3, 5], [2, 3], 2),
    (2, 10, 0, [2, 1], [1, 2], 3),
])
def test_csf_to_ell3d_vs_brute_force(rels, n, edges, rows_bkt, cols_bkt, seed):
    csf = random_csf(rels, n, edges, seed)
    got = oracle.csf_to_ell3d(*csf, rows_bkt, cols_bkt)
    want = brute_force_csf_to_ell3d(*csf, rows_bkt, cols_bkt)
    for b in range(len(cols_bkt)):
        for q in range(4):
            assert got[q][b].shape == want[b][q].shape, (b, q)
            assert np.array_equal(got[q][b], want[b][q]), (b, q)


def test_csf_to_ell3d_decode_and_padding():
    rels, n = 6, 80
    rows_bkt, cols_bkt = [8, 4, 2, 1], [1, 2, 4, 8]
    p0, i0, p1, i1 = random_csf(rels, n, 1500, 7)
    ptr, rows, cols, mask = oracle.csf_to_ell3d(p0, i0, p1, i1, rows_bkt, cols_bkt)
    triples = []
    for b in range(len(cols_bkt)):
        G, rb, cb = cols[b].shape
        assert ptr[b][0] == 0 and ptr[b][-1] == G and np.all(np.diff(ptr[b]) >= 0)
        rel_of_group = np.repeat(np.arange(rels), np.diff(ptr[b]))
        assert np.all(cols[b][mask[b] == 0] == 0)
        rr = np.broadcast_to(rows[b][:, :, None], cols[b].shape)
        gg = np.broadcast_to(rel_of_group[:, None, None], cols[b].shape)
        sel = mask[b] == 1
        triples.append(np.stack([gg[sel], rr[sel], cols[b][sel]], axis=1))
    got = np.concatenate(triples)
    got = got[np.lexsort((got[:, 2], got[:, 1], got[:, 0]))]
    want = []
    for r in range(rels):
        for i in range(p0[r], p0[r + 1]):
            for j in range(p1[i], p1[i + 1]):
                want.append((r, i0[i], i1[j]))
    want = np.asarray(sorted(want), np.int64).reshape(-1, 3)
    assert np.array_equal(got, want)


def test_csf_to_ell3d_rejects_unsorted_buckets():
    with pytest.raises(ValueError):
        oracle.csf_to_ell3d([0, 1], [0], [0, 1], [0], [1, 1], [2, 2])


@pytest.mark.parametrize("kat", KATS["condense"])
def test_condense_known_answer(kat):
    gptr, tiles, mask = oracle.condense(kat["indptr"], kat["indices"], kat["t"], kat["g"])
    assert np.array_equal(gptr, kat["group_indptr"])
    assert np.array_equal(tiles, kat["tile_indices"])
    assert np.array_equal(mask, kat["mask"])


@pytest.mark.parametrize("m,n,nnz,t,seed", [(1000, 1000, 10000, 4, 0), (333, 200, 3000, 8, 1), (50, 40, 0, 4, 2)])
def test_condense_vs_reference_test_comparator(m, n, nnz, t, seed):
    indptr, indices = random_csr(m, n, nnz, seed)
    gptr, tiles, _ = oracle.condense(indptr, indices, t, 1)
    ptr_np, idx_np = numpy_condense_g1(indptr, indices, t)
    assert np.array_equal(gptr, ptr_np)
    assert np.array_equal(tiles.ravel(), idx_np)


@pytest.mark.parametrize("t,g", [(4, 2), (8, 4), (16, 8), (3, 5)])
def test_condense_mask_decodes_to_input(t, g):
    m, n = 157, 120
    indptr, indices = random_csr(m, n, 2500, 5, skew=0.7)
    gptr, tiles, mask = oracle.condense(indptr, indices, t, g)
    pairs = []
    for tile in range(len(gptr) - 1):
        for grp in range(gptr[tile], gptr[tile + 1]):
            rl, sl = np.nonzero(mask[grp])
            pairs += [(tile * t + r, tiles[grp, s]) for r, s in zip(rl, sl)]
        # tiles inside a row tile are the sorted unique columns, zero padded at the end only
        flat = tiles[gptr[tile]:gptr[tile + 1]].ravel()
        u = np.unique(indices[indptr[tile * t]:indptr[min((tile + 1) * t, m)]])
        assert np.array_equal(flat[:len(u)], u) and np.all(flat[len(u):] == 0)
    got = np.asarray(sorted(pairs), np.int64).reshape(-1, 2)
    assert np.array_equal(got, coo_pairs(indptr, indices))


@pytest.mark.parametrize("kat", KATS["sddmm_mid"])
def test_sddmm_mid_known_answer(kat):
    mid = oracle.sddmm_mid(kat["indptr"], kat["indptr"][-1])
    assert np.array_equal(mid, kat["mid"])


def test_sddmm_mid_closed_form():
    indptr, _ = random_csr(300, 100, 4000, 3, skew=1.0)
    nnz = int(indptr[-1])
    want = np.searchsorted(indptr, np.arange(nnz), side="right") - 1
    assert np.array_equal(oracle.sddmm_mid(indptr, nnz), want)


# ------------------------------------------------------------------ numeric oracles vs float64

def test_csrmm_matches_float64_and_skips_empty_rows():
    m, n, feat = 200, 150, 32
    indptr, indices = random_csr(m, n, 3000, 0, skew=0.9)
    rng = np.random.default_rng(0)
    vals = rng.random(len(indices), dtype=np.float32)
    x = rng.standard_normal((n, feat), dtype=np.float32)
    c0 = np.full(m * feat, 7.0, np.float32)
    got = oracle.csrmm(vals, x, indptr, indices, feat, C=c0)
    want = spmm_f64(indptr, indices, vals, x)
    empty = np.diff(indptr) == 0
    assert empty.any()
    assert np.all(got[empty] == 7.0)  # init happens at a row's first nonzero only
    scale = spmm_f64(indptr, indices, np.abs(vals), np.abs(x))
    assert np.all(np.abs(got[~empty] - want[~empty]) <= 1e-5 * scale[~empty] + 1e-30)


def test_hyb_spmm_matches_float64():
    m = n = 300
    feat, parts, buckets = 16, 3, [1, 2, 4]
    indptr, indices = random_csr(m, n, 5000, 1, skew=1.0)
    rows, cols, mask = oracle.column_part_hyb(m, n, indptr, indices, parts, buckets)
    x = np.random.default_rng(1).standard_normal((n, feat), dtype=np.float32)
    triples = [(mask[p][b].astype(np.float32), rows[p][b], cols[p][b])
               for p in range(parts) for b in range(len(buckets))]
    got = oracle.hyb_spmm(m, feat, x, triples, parts)
    want = spmm_f64(indptr, indices, np.ones(len(indices), np.float32), x)
    scale = spmm_f64(indptr, indices, np.ones(len(indices), np.float32), np.abs(x))
    assert np.all(np.abs(got - want) <= 1e-5 * scale + 1e-30)


def test_sddmm_matches_float64():
    m, n, feat = 120, 90, 24
    indptr, indices = random_csr(m, n, 2000, 2)
    rng = np.random.default_rng(2)
    a = rng.standard_normal((m, feat), dtype=np.float32)
    b = rng.standard_normal((n, feat), dtype=np.float32)
    mid = oracle.sddmm_mid(indptr, len(indices))
    got = oracle.sddmm(a, b, indices, mid, feat)
    want = sddmm_f64(indptr, indices, a, b)
    rows = np.repeat(np.arange(m), np.diff(indptr))
    scale = np.einsum("ek,ek->e", np.abs(a)[rows], np.abs(b)[indices])
    assert np.all(np.abs(got - want) <= 1e-5 * scale)


def test_bsrmm_matches_float64():
    mb, nb, blk, feat = 6, 5, 8, 16
    rng = np.random.default_rng(3)
    present = rng.random((mb, nb)) < 0.4
    indptr = np.zeros(mb + 1, np.int32)
    np.cumsum(present.sum(1), out=indptr[1:])
    indices = np.nonzero(present)[1].astype(np.int32)
    data = rng.standard_normal((len(indices), blk, blk), dtype=np.float32)
    x = rng.standard_normal((nb * blk, feat), dtype=np.float32)
    got = oracle.bsrmm(data, x, indptr, indices, blk, feat)
    want = bsr_f64(indptr, indices, data, x, mb, nb, blk)
    assert_close(got, want, rtol=1e-5, atol=1e-4, what="bsrmm oracle")


def test_rgms_matches_float64():
    rels, n, fin, fout = 4, 40, 8, 12
    p0, i0, p1, i1 = random_csf(rels, n, 400, 4)
    rng = np.random.default_rng(4)
    x = rng.standard_normal((n, fin), dtype=np.float32)
    w = rng.standard_normal((rels, fin, fout), dtype=np.float32)
    a = rng.random(len(i1), dtype=np.float32)
    got = oracle.rgms(w, x, a, p0, i0, p1, i1, n)
    want = rgms_f64(p0, i0, p1, i1, a, x, w, n)
    assert_close(got, want, rtol=1e-5, atol=1e-4, what="rgms oracle")


def test_rgms_fp32_forms_match_float64():
    """fp32 RGMS with W[r, fo, fi] (feat_in != feat_out, so a transposed W fails), on the CSF
    arrays and on the ELL3D buckets made from them; both against the float64 closed form."""
    rels, n, fin, fout = 4, 40, 8, 12
    p0, i0, p1, i1 = random_csf(rels, n, 400, 5)
    rng = np.random.default_rng(5)
    x = rng.standard_normal((n, fin), dtype=np.float32)
    w = rng.standard_normal((rels, fout, fin), dtype=np.float32)
    a = rng.random(len(i1), dtype=np.float32)
    want = rgms_f64(p0, i0, p1, i1, a, x, np.ascontiguousarray(w.transpose(0, 2, 1)), n)
    got = oracle.rgms_csf_f32(a, w, x, p0, i0, p1, i1, n)
    assert_close(got, want, rtol=1e-5, atol=1e-4, what="rgms csf fp32 oracle")
    # ELL3D form with the 0/1 mask as weights == CSF form with unit weights
    ones = np.ones(len(i1), np.float32)
    want1 = rgms_f64(p0, i0, p1, i1, ones, x, np.ascontiguousarray(w.transpose(0, 2, 1)), n)
    rows_bkt, cols_bkt = [4, 2, 1], [1, 2, 4]
    ptr, rows, cols, mask = oracle.csf_to_ell3d(p0, i0, p1, i1, rows_bkt, cols_bkt)
    bk = [(mask[b].astype(np.float32), rows[b], cols[b],
           np.repeat(np.arange(rels, dtype=np.int32), np.diff(ptr[b]))) for b in range(3)]
    got1 = oracle.rgms_ell3d_f32(w, x, bk, n)
    assert_close(got1, want1, rtol=1e-5, atol=1e-4, what="rgms ell3d fp32 oracle")
