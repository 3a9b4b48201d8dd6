"""Seeded synthetic workloads shaped like the graphs the reference's examples download.

The reference's example scripts fetch ogbn-arxiv / ogbn-products / AIFB-style graphs over
the network (examples/spmm/utils.py:23-52, examples/rgms/rgcn/utils.py:26-38).  Offline we
generate graphs of the same size and degree skew from ``numpy.random.default_rng(seed)``.
Everything here is host-side numpy; rows are destination nodes and columns source nodes,
the orientation ``g.adj_sparse("csc")`` gives the reference (examples/spmm/bench_spmm.py:103).
"""
import numpy as np


def _powerlaw_weights(n, alpha, nnz_target, max_deg, rng):
    """w_i proportional to (rank_i + s)^-alpha over a seeded permutation of the rows; the shift
    s is bisected so that the heaviest row expects about ``max_deg`` entries."""
    rank = np.arange(1, n + 1, dtype=np.float64)

    def top(s):
        w = (rank + s) ** (-alpha)
        return nnz_target * w[0] / w.sum()

    s = 0.0
    if max_deg is not None and top(0.0) > max_deg:
        lo, hi = 0.0, 1.0
        while top(hi) > max_deg:
            hi *= 2.0
        for _ in range(60):
            mid = 0.5 * (lo + hi)
            if top(mid) > max_deg:
                lo = mid
            else:
                hi = mid
        s = hi
    w = (rank + s) ** (-alpha)
    w /= w.sum()
    return w[rng.permutation(n)]


def _to_csr(n, rows, cols):
    """Sort (row, col) pairs, drop duplicates, return int32 CSR with ascending columns."""
    key = rows.astype(np.int64) * n + cols.astype(np.int64)
    key = np.unique(key)
    rows = (key // n).astype(np.int32)
    cols = (key % n).astype(np.int32)
    indptr = np.zeros(n + 1, np.int64)
    np.cumsum(np.bincount(rows, minlength=n), out=indptr[1:])
    return indptr.astype(np.int32), cols


def powerlaw_graph(n, nnz_target, alpha, seed, max_deg=None, self_loops=False,
                   columns="uniform"):
    """Square power-law graph as int32 CSR (indptr, indices), columns ascending per row.

    columns="uniform":   row degrees ~ multinomial(nnz_target, w); each entry's column is
                         uniform over [0, n) (skewed destination degree only).
    columns="symmetric": nnz_target/2 undirected pairs with both endpoints drawn from w,
                         stored in both directions (an undirected graph: row and column
                         degree share the same skew).
    Duplicates are dropped, so the realised nnz is slightly below the target.
    """
    rng = np.random.default_rng(seed)
    w = _powerlaw_weights(n, alpha, nnz_target, max_deg, rng)
    if columns == "uniform":
        deg = rng.multinomial(nnz_target, w)
        rows = np.repeat(np.arange(n, dtype=np.int32), deg)
        cols = rng.integers(0, n, size=rows.shape[0], dtype=np.int32)
    elif columns == "symmetric":
        half = nnz_target // 2
        cdf = np.cumsum(w)
        cdf[-1] = 1.0
        u = np.searchsorted(cdf, rng.random(half), side="right").astype(np.int32)
        v = np.searchsorted(cdf, rng.random(half), side="right").astype(np.int32)
        rows = np.concatenate([u, v])
        cols = np.concatenate([v, u])
    else:
        raise ValueError("columns must be 'uniform' or 'symmetric'")
    if self_loops:
        d = np.arange(n, dtype=np.int32)
        rows = np.concatenate([rows, d])
        cols = np.concatenate([cols, d])
    return _to_csr(n, rows, cols)


def config1(seed=0):
    """CSR SpMM fp32, the reference's CPU-runnable case: 4,096 nodes, ~65k edges (Zipf 1.2
    out-degree) plus self-loops, values U(0,1), X 4096x32 N(0,1)."""
    n, feat = 4096, 32
    indptr, indices = powerlaw_graph(n, 65536, 1.2, seed, max_deg=1024, self_loops=True)
    rng = np.random.default_rng(seed + 1000)
    vals = rng.random(indices.shape[0], dtype=np.float32)
    x = rng.standard_normal((n, feat), dtype=np.float32)
    return dict(m=n, n=n, feat=feat, indptr=indptr, indices=indices, values=vals, x=x)


def config2(seed=1, columns="uniform"):
    """hyb SpMM fp32: 169,343 nodes, ~1.17M edges, Zipf ~1.1, max degree ~13k; 2 column
    partitions and ELL widths 1..512 (features are drawn by the caller per width)."""
    n = 169343
    indptr, indices = powerlaw_graph(n, 1166243, 1.1, seed, max_deg=13000, columns=columns)
    return dict(m=n, n=n, indptr=indptr, indices=indices, num_col_parts=2,
                buckets=[1, 2, 4, 8, 16, 32, 64, 128, 256, 512])


def config3(seed=2, columns="uniform", scale=1.0):
    """Large GNN SpMM + SDDMM fp32: 2,449,029 nodes, ~61.9M edges, Zipf ~1.0.  ``scale``
    shrinks nodes and edges together (tests use a small fraction of the full size)."""
    n = max(64, int(2449029 * scale))
    nnz = max(256, int(61859140 * scale))
    indptr, indices = powerlaw_graph(n, nnz, 1.0, seed, max_deg=max(32, int(17500 * min(1.0, scale * 4))),
                                     columns=columns)
    # The reference's table for a graph of this size uses 16 column partitions and widths
    # 1..32 (examples/spmm/bench_spmm.py:233-253).  On MI355X every extra partition turns
    # stores into device-scope fp32 atomics, which run an order of magnitude below the gather
    # rate, so the default here is one partition and widths up to 512 (hub rows are split in
    # the widest bucket only).
    return dict(m=n, n=n, indptr=indptr, indices=indices, num_col_parts=1,
                buckets=[1, 2, 4, 8, 16, 32, 64, 128, 256, 512])


def features(n, feat, seed, dtype=np.float32):
    rng = np.random.default_rng(seed)
    return rng.standard_normal((n, feat), dtype=np.float32).astype(dtype)


def config4(seed=3, mb=128, nb=128, blk=32, density=0.10, feat=512):
    """BSR block-sparse weight: mb x nb grid of blk x blk blocks, each present with
    probability ``density``; block values N(0, 0.02); activations (nb*blk) x feat N(0,1).
    Values are float32 here; callers round to fp16/bf16."""
    rng = np.random.default_rng(seed)
    present = rng.random((mb, nb)) < density
    indptr = np.zeros(mb + 1, np.int32)
    np.cumsum(present.sum(axis=1), out=indptr[1:])
    indices = np.nonzero(present)[1].astype(np.int32)
    data = (rng.standard_normal((indices.shape[0], blk, blk), dtype=np.float32) * 0.02)
    x = rng.standard_normal((nb * blk, feat), dtype=np.float32)
    return dict(mb=mb, nb=nb, blk=blk, feat=feat, indptr=indptr, indices=indices, data=data, x=x)


def config5(seed=4, n=100000, num_rels=65, num_edges=2000000, feat=32):
    """Heterogeneous graph for RGMS: ``num_edges`` split over ``num_rels`` relations by
    Zipf(1.0); per relation uniform random (dst, src) pairs, deduplicated, stored as CSF
    (relation -> destination rows with at least one edge -> source columns, global ids)."""
    rng = np.random.default_rng(seed)
    w = 1.0 / np.arange(1, num_rels + 1, dtype=np.float64)
    w /= w.sum()
    per_rel = rng.multinomial(num_edges, w)
    indptr0 = [0]
    indices0, indptr1, indices1 = [], [np.zeros(1, np.int64)], []
    base = 0
    for r in range(num_rels):
        e = int(per_rel[r])
        dst = rng.integers(0, n, size=e, dtype=np.int64)
        src = rng.integers(0, n, size=e, dtype=np.int64)
        key = np.unique(dst * n + src)
        dst, src = key // n, key % n
        rows, counts = np.unique(dst, return_counts=True)
        indptr0.append(indptr0[-1] + rows.shape[0])
        indices0.append(rows.astype(np.int32))
        indptr1.append(base + np.cumsum(counts))
        indices1.append(src.astype(np.int32))
        base += src.shape[0]
    cat = lambda xs, dt: np.concatenate(xs).astype(dt) if xs else np.zeros(0, dt)
    x = rng.standard_normal((n, feat), dtype=np.float32)
    wgt = rng.standard_normal((num_rels, feat, feat), dtype=np.float32) * 0.1
    return dict(m=n, n=n, num_rels=num_rels, feat_in=feat, feat_out=feat,
                indptr0=np.asarray(indptr0, np.int32), indices0=cat(indices0, np.int32),
                indptr1=cat(indptr1, np.int32), indices1=cat(indices1, np.int32),
                x=x, w=wgt, buckets=[1, 2, 4, 8, 16])
