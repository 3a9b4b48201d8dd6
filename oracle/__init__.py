"""CPU oracle for the SparseTIR hot path -- TEST INFRASTRUCTURE ONLY.

Thin ctypes front-end over ``oracle/sparsetir_oracle.c`` (a sequential C restatement of
the reference's algorithms; the header of that file lists the reference file:line each
function follows).  Only the test-suite, the smoke check and the benchmark's
``cpu_baseline`` leg may import this package; the shipped library never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libsparsetir_oracle.so")


def build(force=False):
    """Compile the C oracle with gcc (``make -C oracle``)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


_i32p = ctypes.POINTER(ctypes.c_int32)
_f32p = ctypes.POINTER(ctypes.c_float)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    if a.dtype == np.int32:
        return a.ctypes.data_as(_i32p)
    if a.dtype == np.float32:
        return a.ctypes.data_as(_f32p)
    if a.dtype == np.int64:
        return a.ctypes.data_as(ctypes.POINTER(ctypes.c_int64))
    raise TypeError(a.dtype)


def _ptr_array(arrs):
    return (_i32p * len(arrs))(*[_p(a) for a in arrs])


def column_part_hyb(num_rows, num_cols, indptr, indices, num_col_parts, buckets):
    """Returns (row_indices, col_indices, mask), each [num_col_parts][len(buckets)] of
    int32 arrays shaped (nrows,), (nrows, b), (nrows, b)."""
    indptr, indices, widths = _i32(indptr), _i32(indices), _i32(buckets)
    nb = len(widths)
    nk = num_col_parts * nb
    nrows = np.zeros(nk, np.int64)
    L = lib()
    rc = L.oracle_column_part_hyb(num_rows, num_cols, _p(indptr), _p(indices), num_col_parts,
                                  _p(widths), nb, _p(nrows), None, None, None)
    if rc != 0:
        raise ValueError("column index out of range")
    rows = [np.empty(int(nrows[k]), np.int32) for k in range(nk)]
    cols = [np.empty((int(nrows[k]), int(widths[k % nb])), np.int32) for k in range(nk)]
    mask = [np.empty((int(nrows[k]), int(widths[k % nb])), np.int32) for k in range(nk)]
    L.oracle_column_part_hyb(num_rows, num_cols, _p(indptr), _p(indices), num_col_parts,
                             _p(widths), nb, _p(nrows), _ptr_array(rows), _ptr_array(cols),
                             _ptr_array(mask))
    nest = lambda xs: [[xs[p * nb + b] for b in range(nb)] for p in range(num_col_parts)]
    return nest(rows), nest(cols), nest(mask)


def csf_to_ell3d(indptr0, indices0, indptr1, indices1, nnz_rows_bkt, nnz_cols_bkt):
    """Returns (indptr, row_indices, col_indices, mask), each a list over buckets with
    shapes (R+1,), (G, rb), (G, rb, cb), (G, rb, cb)."""
    indptr0, indices0 = _i32(indptr0), _i32(indices0)
    indptr1, indices1 = _i32(indptr1), _i32(indices1)
    rb, cb = _i32(nnz_rows_bkt), _i32(nnz_cols_bkt)
    if len(rb) != len(cb):
        raise ValueError("Input nnz_rows and nnz_cols should have same length.")
    nb = len(cb)
    num_rels = len(indptr0) - 1
    groups = np.zeros(nb, np.int64)
    L = lib()
    rc = L.oracle_csf_to_ell3d(num_rels, _p(indptr0), _p(indices0), _p(indptr1), _p(indices1),
                               _p(rb), _p(cb), nb, _p(groups), None, None, None, None)
    if rc != 0:
        raise ValueError("The given nnz_cols_bkt should be ascending.")
    out_ptr = [np.empty(num_rels + 1, np.int32) for _ in range(nb)]
    rows = [np.empty((int(groups[b]), int(rb[b])), np.int32) for b in range(nb)]
    cols = [np.empty((int(groups[b]), int(rb[b]), int(cb[b])), np.int32) for b in range(nb)]
    mask = [np.empty((int(groups[b]), int(rb[b]), int(cb[b])), np.int32) for b in range(nb)]
    L.oracle_csf_to_ell3d(num_rels, _p(indptr0), _p(indices0), _p(indptr1), _p(indices1),
                          _p(rb), _p(cb), nb, _p(groups), _ptr_array(out_ptr), _ptr_array(rows),
                          _ptr_array(cols), _ptr_array(mask))
    return out_ptr, rows, cols, mask


def condense(indptr, indices, t, g):
    """Returns (group_indptr (tiles+1,), tile_indices (G, g), mask (G, t, g))."""
    indptr, indices = _i32(indptr), _i32(indices)
    n = len(indptr) - 1
    tiles = (n + t - 1) // t
    gptr = np.empty(tiles + 1, np.int32)
    ng = np.zeros(1, np.int64)
    L = lib()
    L.oracle_condense(n, _p(indptr), _p(indices), t, g, _p(ng), _p(gptr), None, None)
    G = int(ng[0])
    tile_indices = np.empty((G, g), np.int32)
    mask = np.empty((G, t, g), np.int32)
    L.oracle_condense(n, _p(indptr), _p(indices), t, g, _p(ng), _p(gptr), _p(tile_indices),
                      _p(mask))
    return gptr, tile_indices, mask


def csrmm(A, B, indptr, indices, feat, C=None):
    """C[i, :] = sum_p A[p] * B[indices[p], :]; rows without nonzeros keep C's content."""
    A, B, indptr, indices = _f32(A).ravel(), _f32(B).ravel(), _i32(indptr), _i32(indices)
    m = len(indptr) - 1
    if C is None:
        C = np.zeros(m * feat, np.float32)
    lib().oracle_csrmm(m, feat, _p(A), _p(B), _p(C), _p(indptr), _p(indices))
    return C.reshape(m, feat)


def hyb_spmm(m, feat, B, buckets, num_col_parts):
    """``buckets`` is the flat list (part-major, bucket-minor) of (A_k, rows_k, cols_k) with
    cols_k shaped (nrows, width).  Store for non-atomic buckets, add for atomic ones, where
    atomic = (num_col_parts > 1) or last bucket of its partition."""
    B = _f32(B).ravel()
    C = np.zeros(m * feat, np.float32)
    nb = len(buckets) // num_col_parts
    for k, (A_k, rows_k, cols_k) in enumerate(buckets):
        cols_k = _i32(cols_k)
        nrows = cols_k.shape[0]
        if nrows == 0:
            continue
        w = cols_k.shape[1]
        atomic = num_col_parts > 1 or (k % nb) == nb - 1
        A_k, rows_k = _f32(A_k).ravel(), _i32(rows_k)
        cflat = cols_k.ravel()
        lib().oracle_ell_spmm(ctypes.c_int64(nrows), w, feat, _p(A_k), _p(rows_k), _p(cflat),
                              _p(B), _p(C), int(atomic))
    return C.reshape(m, feat)


def sddmm_mid(indptr, nnz):
    indptr = _i32(indptr)
    mid = np.empty(nnz, np.int32)
    lib().oracle_sddmm_mid(len(indptr) - 1, ctypes.c_int64(nnz), _p(indptr), _p(mid))
    return mid


def sddmm(A, B, indices, mid, feat):
    A, B, indices, mid = _f32(A).ravel(), _f32(B).ravel(), _i32(indices), _i32(mid)
    C = np.empty(len(indices), np.float32)
    lib().oracle_sddmm(ctypes.c_int64(len(indices)), feat, _p(A), _p(B), _p(C), _p(indices),
                       _p(mid))
    return C


def bsrmm(A, X, indptr, indices, blk, feat):
    """A: (nnzb, blk, blk), X: (nb*blk, feat), both float32 holding values already rounded to
    the storage type; fp32 accumulation."""
    A, X, indptr, indices = _f32(A).ravel(), _f32(X).ravel(), _i32(indptr), _i32(indices)
    mb = len(indptr) - 1
    Y = np.empty(mb * blk * feat, np.float32)
    lib().oracle_bsrmm(mb, blk, feat, _p(A), _p(X), _p(Y), _p(indptr), _p(indices))
    return Y.reshape(mb * blk, feat)


def rgms(W, X, A, indptr0, indices0, indptr1, indices1, m):
    """W: (R, fin, fout), X: (n, fin), A: per stored column value; returns Y (m, fout)."""
    W, X, A = _f32(W), _f32(X), _f32(A).ravel()
    R, fin, fout = W.shape
    indptr0, indices0 = _i32(indptr0), _i32(indices0)
    indptr1, indices1 = _i32(indptr1), _i32(indices1)
    Y = np.zeros(m * fout, np.float32)
    Wf, Xf = W.ravel(), X.ravel()
    lib().oracle_rgms(R, fin, fout, _p(Wf), _p(Xf), _p(Y), _p(A), _p(indptr0), _p(indices0),
                      _p(indptr1), _p(indices1))
    return Y.reshape(m, fout)


def rgms_csf_f32(A, W, X, indptr_i, indices_i, indptr_j, indices_j, m):
    """W: (R, fout, fin), X: (n, fin), A: (nnz_j,); returns Y (m, fout)."""
    W, X, A = _f32(W), _f32(X), _f32(A).ravel()
    R, fout, fin = W.shape
    indptr_i, indices_i = _i32(indptr_i), _i32(indices_i)
    indptr_j, indices_j = _i32(indptr_j), _i32(indices_j)
    Y = np.zeros(m * fout, np.float32)
    Wf, Xf = W.ravel(), X.ravel()
    lib().oracle_rgms_csf_f32(R, fin, fout, _p(A), _p(Wf), _p(Xf), _p(Y), _p(indptr_i), _p(indices_i),
                              _p(indptr_j), _p(indices_j))
    return Y.reshape(m, fout)


def rgms_ell3d_f32(W, X, buckets, m):
    """``buckets``: list of (A (G, rb, cb) f32, rows (G, rb), cols (G, rb, cb), mids (G,)).
    W: (R, fout, fin).  Returns Y (m, fout)."""
    W, X = _f32(W), _f32(X)
    R, fout, fin = W.shape
    Y = np.zeros(m * fout, np.float32)
    Wf, Xf = W.ravel(), X.ravel()
    for A, rows, cols, mids in buckets:
        G, rb, cb = cols.shape
        if G == 0:
            continue
        A, rows, cols, mids = _f32(A).ravel(), _i32(rows).ravel(), _i32(cols).ravel(), _i32(mids).ravel()
        lib().oracle_rgms_ell3d_f32(ctypes.c_int64(G), rb, cb, fin, fout, _p(A), _p(rows), _p(cols), _p(mids),
                                    _p(Wf), _p(Xf), _p(Y))
    return Y.reshape(m, fout)
