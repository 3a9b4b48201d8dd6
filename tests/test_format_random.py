"""Randomised comparison of the host format routines with the oracle (hypothesis): arbitrary
small CSR / CSF inputs, including duplicate and unsorted columns, empty rows, single-row and
single-column matrices, bucket lists of any ascending widths.  Index arrays must be bit-exact."""
import numpy as np
from hypothesis import given, settings, strategies as hs

import oracle
import sparsetir_amd as st
from helpers import brute_force_column_part_hyb


def _same(got, want):
    for g, w in zip(got, want):
        if isinstance(w, (list, tuple)):
            _same(g, w)
        else:
            assert g.shape == w.shape and g.dtype == w.dtype and np.array_equal(g, w)


@hs.composite
def csr(draw, max_rows=12, max_cols=12, max_deg=9):
    m = draw(hs.integers(1, max_rows))
    n = draw(hs.integers(1, max_cols))
    rows = [draw(hs.lists(hs.integers(0, n - 1), max_size=max_deg)) for _ in range(m)]
    indptr = np.concatenate([[0], np.cumsum([len(r) for r in rows])]).astype(np.int32)
    indices = np.asarray([c for r in rows for c in r], np.int32)
    return m, n, indptr, indices


@hs.composite
def widths(draw, max_len=4, max_w=9):
    k = draw(hs.integers(1, max_len))
    return sorted(draw(hs.lists(hs.integers(1, max_w), min_size=k, max_size=k, unique=True)))


@settings(max_examples=300, deadline=None)
@given(csr(), hs.integers(1, 5), widths())
def test_column_part_hyb_any_input(mat, parts, buckets):
    m, n, indptr, indices = mat
    got = st.column_part_hyb(m, n, indptr, indices, parts, buckets)
    _same(got, oracle.column_part_hyb(m, n, indptr, indices, parts, buckets))
    _same(got, brute_force_column_part_hyb(indptr, indices, m, n, parts, buckets))


@hs.composite
def csf(draw):
    rels = draw(hs.integers(1, 4))
    n = draw(hs.integers(1, 10))
    p0, i0, p1, i1 = [0], [], [0], []
    for _ in range(rels):
        rows = draw(hs.lists(hs.integers(0, n - 1), max_size=6))          # may repeat, any order
        for r in rows:
            cols = draw(hs.lists(hs.integers(0, n - 1), min_size=0, max_size=7))
            i0.append(r)
            i1 += cols
            p1.append(len(i1))
        p0.append(len(i0))
    i32 = lambda x: np.asarray(x, np.int32)
    return i32(p0), i32(i0), i32(p1), i32(i1)


@settings(max_examples=300, deadline=None)
@given(csf(), widths(max_len=3, max_w=6), hs.integers(1, 5))
def test_csf_to_ell3d_any_input(arrays, cols_bkt, rb):
    rows_bkt = [rb] * len(cols_bkt)
    got = st.csf_to_ell3d(*arrays, rows_bkt, cols_bkt)
    _same(got, oracle.csf_to_ell3d(*arrays, rows_bkt, cols_bkt))


@settings(max_examples=300, deadline=None)
@given(csr(max_rows=14, max_cols=10, max_deg=8), hs.integers(1, 5), hs.integers(1, 4))
def test_condense_any_input(mat, t, g):
    m, n, indptr, indices = mat
    got = st.condense(indptr, indices, t, g)
    _same(got, oracle.condense(indptr, indices, t, g))
