"""Independent restatements used to pin the oracle and the product (numpy / scipy only).

None of these share code with ``oracle/`` or ``sparsetir_amd/csrc``: they are written from the
mathematics (closed forms, textbook routines) or restate the comparators the reference's own
tests use, so that an indexing mistake in one place cannot hide in another.
"""
import json
import os

import numpy as np
import scipy.sparse as sp

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_kats():
    with open(os.path.join(GOLDEN, "format_kats.json")) as f:
        return json.load(f)


def random_csr(m, n, nnz, seed, sort=True, skew=0.0):
    """Random int32 CSR without duplicate entries; optionally power-law-ish row skew and
    unsorted columns inside rows."""
    rng = np.random.default_rng(seed)
    if m == 0 or n == 0 or nnz == 0:
        return np.zeros(m + 1, np.int32), np.zeros(0, np.int32)
    if skew > 0:
        w = (np.arange(1, m + 1, dtype=np.float64)) ** (-skew)
        rows = rng.choice(m, size=nnz, p=w / w.sum())
    else:
        rows = rng.integers(0, m, nnz)
    cols = rng.integers(0, n, nnz)
    key = np.unique(rows.astype(np.int64) * n + cols)
    rows, cols = (key // n).astype(np.int32), (key % n).astype(np.int32)
    indptr = np.zeros(m + 1, np.int32)
    np.cumsum(np.bincount(rows, minlength=m), out=indptr[1:])
    if not sort:
        for i in range(m):
            seg = cols[indptr[i]:indptr[i + 1]]
            rng.shuffle(seg)
    return indptr, cols


def scipy_style_column_part_hyb(indptr, indices, m, n, parts, buckets):
    """The comparator of the reference's test_column_part_hyb
    (tests/python/sparsetir/test_format_conversion_routine.py:28-101), restated: slice the
    matrix by column ranges with scipy, bucket rows by their degree in the slice, split rows
    longer than the widest bucket into consecutive chunks.  Returns flat lists (partition
    major) of row-id arrays and column arrays.  Needs at least two buckets, like the original.
    """
    mat = sp.csr_matrix((np.ones(len(indices), np.int8), indices, indptr), shape=(m, n))
    mat.sort_indices()
    psize = (n + parts - 1) // parts
    out_rows, out_cols = [], []
    for p in range(parts):
        sub = mat[:, p * psize:(p + 1) * psize]
        deg = np.diff(sub.indptr)
        for bi, b in enumerate(buckets):
            lower = 0 if bi == 0 else buckets[bi - 1]
            last = bi == len(buckets) - 1
            sel = np.nonzero(deg > lower)[0] if last else np.nonzero((deg > lower) & (deg <= b))[0]
            rows, cols = [], []
            for r in sel:
                seg = sub.indices[sub.indptr[r]:sub.indptr[r + 1]] + p * psize
                for off in range(0, len(seg), b):
                    chunk = np.zeros(b, np.int32)
                    piece = seg[off:off + b]
                    chunk[:len(piece)] = piece
                    rows.append(r)
                    cols.append(chunk)
            out_rows.append(np.asarray(rows, np.int32))
            out_cols.append(np.asarray(cols, np.int32).reshape(len(rows), b))
    return out_rows, out_cols


def brute_force_column_part_hyb(indptr, indices, m, n, parts, buckets):
    """Closed form in pure Python, valid for unsorted rows too: per (row, partition) the
    entries in CSR order go to the first bucket wide enough (else the last), chunked into
    ELL rows of that width."""
    psize = (n + parts - 1) // parts
    nb = len(buckets)
    R = [[[] for _ in range(nb)] for _ in range(parts)]
    C = [[[] for _ in range(nb)] for _ in range(parts)]
    M = [[[] for _ in range(nb)] for _ in range(parts)]
    for i in range(m):
        per_part = {}
        for e in range(indptr[i], indptr[i + 1]):
            per_part.setdefault(int(indices[e]) // psize, []).append(int(indices[e]))
        for p, cols in per_part.items():
            d = len(cols)
            k = next((j for j, b in enumerate(buckets) if b >= d), nb - 1)
            b = buckets[k]
            for off in range(0, d, b):
                piece = cols[off:off + b]
                R[p][k].append(i)
                C[p][k].append(piece + [0] * (b - len(piece)))
                M[p][k].append([1] * len(piece) + [0] * (b - len(piece)))
    arr = lambda x, b: np.asarray(x, np.int32).reshape(len(x), b)
    rows = [[np.asarray(R[p][k], np.int32) for k in range(nb)] for p in range(parts)]
    cols = [[arr(C[p][k], buckets[k]) for k in range(nb)] for p in range(parts)]
    mask = [[arr(M[p][k], buckets[k]) for k in range(nb)] for p in range(parts)]
    return rows, cols, mask


def decode_hyb(rows, cols, mask):
    """Sorted (row, col) pairs stored in a hyb decomposition."""
    pairs = []
    for rp, cp, mp in zip(rows, cols, mask):
        for r, c, k in zip(rp, cp, mp):
            if r.shape[0] == 0:
                continue
            rr = np.repeat(r[:, None], c.shape[1], axis=1)
            sel = k == 1
            pairs.append(np.stack([rr[sel], c[sel]], axis=1))
    if not pairs:
        return np.zeros((0, 2), np.int64)
    allp = np.concatenate(pairs).astype(np.int64)
    return allp[np.lexsort((allp[:, 1], allp[:, 0]))]


def coo_pairs(indptr, indices):
    rows = np.repeat(np.arange(len(indptr) - 1), np.diff(indptr))
    allp = np.stack([rows, indices], axis=1).astype(np.int64)
    return allp[np.lexsort((allp[:, 1], allp[:, 0]))]


def numpy_condense_g1(indptr, indices, t):
    """The comparator of the reference's test_condense (test_format_conversion_routine.py:130-143):
    per row tile, the sorted unique columns."""
    m = len(indptr) - 1
    out_ptr, out_idx = [0], []
    for tile in range((m + t - 1) // t):
        a = indptr[tile * t]
        b = indptr[min((tile + 1) * t, m)]
        u = np.unique(indices[a:b])
        out_ptr.append(out_ptr[-1] + len(u))
        out_idx.append(u)
    cat = np.concatenate(out_idx) if out_idx else np.zeros(0, np.int32)
    return np.asarray(out_ptr), cat


def random_csf(num_rels, n, edges, seed):
    """Random CSF (relation -> rows with edges -> cols), global ids, int32."""
    rng = np.random.default_rng(seed)
    indptr0, indices0, indptr1, indices1 = [0], [], [0], []
    for r in range(num_rels):
        e = int(rng.integers(0, max(1, 2 * edges // max(1, num_rels))))
        dst = rng.integers(0, n, e)
        src = rng.integers(0, n, e)
        key = np.unique(dst.astype(np.int64) * n + src)
        dst, src = key // n, key % n
        rows, counts = np.unique(dst, return_counts=True)
        indptr0.append(indptr0[-1] + len(rows))
        indices0 += rows.tolist()
        for c in counts:
            indptr1.append(indptr1[-1] + int(c))
        indices1 += src.tolist()
    i32 = lambda x: np.asarray(x, np.int32)
    return i32(indptr0), i32(indices0), i32(indptr1), i32(indices1)


def brute_force_csf_to_ell3d(indptr0, indices0, indptr1, indices1, rows_bkt, cols_bkt):
    """Closed form in pure Python for CSF whose stored rows are distinct inside a relation."""
    R = len(indptr0) - 1
    nb = len(cols_bkt)
    out = []
    for k in range(nb):
        rb, cb = rows_bkt[k], cols_bkt[k]
        ptr, rows, cols, mask = [0], [], [], []
        for r in range(R):
            rel_rows, rel_cols, rel_mask = [], [], []
            for i in range(indptr0[r], indptr0[r + 1]):
                seg = [int(c) for c in indices1[indptr1[i]:indptr1[i + 1]]]
                d = len(seg)
                kk = next((j for j, b in enumerate(cols_bkt) if b >= d), nb - 1)
                if kk != k or d == 0:
                    continue
                for off in range(0, d, cb):
                    piece = seg[off:off + cb]
                    rel_rows.append(int(indices0[i]))
                    rel_cols.append(piece + [0] * (cb - len(piece)))
                    rel_mask.append([1] * len(piece) + [0] * (cb - len(piece)))
            while len(rel_rows) % rb:
                rel_rows.append(rel_rows[-1])
                rel_cols.append([0] * cb)
                rel_mask.append([0] * cb)
            rows += rel_rows
            cols += rel_cols
            mask += rel_mask
            ptr.append(len(rows) // rb)
        G = len(rows) // rb
        out.append((np.asarray(ptr, np.int32), np.asarray(rows, np.int32).reshape(G, rb),
                    np.asarray(cols, np.int32).reshape(G, rb, cb),
                    np.asarray(mask, np.int32).reshape(G, rb, cb)))
    return out


def spmm_f64(indptr, indices, values, x):
    m = len(indptr) - 1
    a = sp.csr_matrix((values.astype(np.float64), indices, indptr), shape=(m, x.shape[0]))
    return a @ x.astype(np.float64)


def sddmm_f64(indptr, indices, a, b):
    rows = np.repeat(np.arange(len(indptr) - 1), np.diff(indptr))
    return np.einsum("ek,ek->e", a.astype(np.float64)[rows], b.astype(np.float64)[indices])


def bsr_f64(indptr, indices, data, x, mb, nb, blk):
    a = sp.bsr_matrix((data.astype(np.float64), indices, indptr), shape=(mb * blk, nb * blk))
    return a.toarray() @ x.astype(np.float64)


def rgms_f64(indptr0, indices0, indptr1, indices1, avals, x, w, m):
    """Y += A_r @ (X @ W_r) per relation, float64 (the form of the reference's
    get_ground_truth, examples/rgms/rgcn/bench_rgcn_tensorcore.py:865-890)."""
    R = len(indptr0) - 1
    n = x.shape[0]
    y = np.zeros((m, w.shape[2]), np.float64)
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    for r in range(R):
        i0, i1 = indptr0[r], indptr0[r + 1]
        if i1 == i0:
            continue
        counts = np.diff(indptr1[i0:i1 + 1])
        rows = np.repeat(indices0[i0:i1], counts)
        e0, e1 = indptr1[i0], indptr1[i1]
        a = sp.csr_matrix((avals[e0:e1].astype(np.float64), (rows, indices1[e0:e1])), shape=(m, n))
        y += a @ (x64 @ w64[r])
    return y


def assert_close(actual, desired, rtol, atol, what=""):
    """|actual - desired| <= atol + rtol*|desired| elementwise (the form of
    tvm.testing.assert_allclose, python/tvm/testing/utils.py:94-105)."""
    actual = np.asarray(actual, np.float64)
    desired = np.asarray(desired, np.float64)
    err = np.abs(actual - desired)
    bound = atol + rtol * np.abs(desired)
    bad = err > bound
    if bad.any():
        i = np.argmax(err - bound)
        raise AssertionError(
            f"{what}: {bad.sum()} of {bad.size} elements out of tolerance (rtol={rtol}, atol={atol}); "
            f"worst at flat index {i}: got {actual.ravel()[i]!r}, want {desired.ravel()[i]!r}")
