"""Format-decomposition routines with the reference's Python surface.

Mirrors ``python/tvm/sparse/format.py`` of the reference: ``column_part_hyb`` (:89-116),
``condense`` (:119-139) and ``csf_to_ell3d`` (:142-170) keep their names, argument order and
return nesting.  Where the reference takes ``tvm.nd`` CPU arrays and returns nested
``Array<NDArray>``, these take numpy arrays / CPU torch tensors and return nested lists of
numpy ``int32`` arrays.  ``column_part_hyb`` additionally accepts CUDA torch tensors, in which
case the decomposition runs on the GPU and returns CUDA tensors.
"""
import ctypes

import numpy as np

from . import _lib


def _host_i32(a, name):
    """int32 contiguous numpy view of a numpy array / CPU torch tensor (reference:
    'Only support int32 index data type', src/sparse/format.cc:56-59)."""
    if hasattr(a, "detach") and hasattr(a, "numpy"):
        if a.device.type != "cpu":
            raise _lib.SparseTIRError(f"Only support {name} conversion on CPU.")
        a = a.detach().numpy()
    a = np.asarray(a)
    if a.dtype != np.int32:
        raise _lib.SparseTIRError(
            f"Only support int32 index data type, got {a.dtype.itemsize * 8} bits for {name}.")
    return np.ascontiguousarray(a)


def _vp(a):
    return ctypes.c_void_p(a.ctypes.data)


def _is_cuda_tensor(a):
    return hasattr(a, "is_cuda") and a.is_cuda


def column_part_hyb(num_rows, num_cols, indptr_nd, indices_nd, num_col_parts, buckets, values=None):
    """Partition a CSR matrix by columns and collect rows into ELL buckets by their number of
    nonzeros per partition.

    Returns ``(row_indices, col_indices, mask)``; each is a list over column partitions of
    lists over buckets of int32 arrays shaped ``(nrows,)``, ``(nrows, b)``, ``(nrows, b)``.

    Extension (GPU path only): with ``values`` (float32 CUDA tensor aligned with ``indices``) a
    fourth nested list is returned holding the per-bucket value arrays ``A_k`` of shape
    ``(nrows, b)``, i.e. the result of the reference's "rewrite_A_k" preprocess blocks.
    """
    if _is_cuda_tensor(indptr_nd) or _is_cuda_tensor(indices_nd):
        return _column_part_hyb_device(num_rows, num_cols, indptr_nd, indices_nd,
                                       num_col_parts, buckets, values)
    if values is not None:
        raise _lib.SparseTIRError("ColumnPartHyb: the value rewrite needs CUDA tensors")
    L = _lib.lib()
    indptr = _host_i32(indptr_nd, "indptr")
    indices = _host_i32(indices_nd, "indices")
    if indptr.shape[0] != num_rows + 1:
        raise _lib.SparseTIRError("ColumnPartHyb: indptr must have num_rows + 1 entries")
    widths = np.ascontiguousarray(np.asarray(list(buckets), dtype=np.int32))
    nb = len(widths)
    nk = num_col_parts * nb
    nrows = np.zeros(max(nk, 1), np.int64)
    _lib.check(L.stir_column_part_hyb_sizes(num_rows, num_cols, _vp(indptr), _vp(indices),
                                            num_col_parts, _vp(widths), nb, _vp(nrows)))
    rows = [np.empty(int(nrows[k]), np.int32) for k in range(nk)]
    cols = [np.empty((int(nrows[k]), int(widths[k % nb])), np.int32) for k in range(nk)]
    mask = [np.empty((int(nrows[k]), int(widths[k % nb])), np.int32) for k in range(nk)]
    _lib.check(L.stir_column_part_hyb_fill(
        num_rows, num_cols, _vp(indptr), _vp(indices), num_col_parts, _vp(widths), nb,
        _lib.ptr_table([a.ctypes.data for a in rows]),
        _lib.ptr_table([a.ctypes.data for a in cols]),
        _lib.ptr_table([a.ctypes.data for a in mask])))
    nest = lambda xs: [[xs[p * nb + b] for b in range(nb)] for p in range(num_col_parts)]
    return nest(rows), nest(cols), nest(mask)


def _column_part_hyb_device(num_rows, num_cols, indptr, indices, num_col_parts, buckets, values=None):
    import torch

    L = _lib.lib()
    for t, name in ((indptr, "indptr"), (indices, "indices")):
        if not _is_cuda_tensor(t):
            raise _lib.SparseTIRError("ColumnPartHyb(device): indptr and indices must both be CUDA tensors")
        if t.dtype != torch.int32:
            raise _lib.SparseTIRError(
                f"Only support int32 index data type, got {t.element_size() * 8} bits for {name}.")
    indptr, indices = indptr.contiguous(), indices.contiguous()
    if indptr.shape[0] != num_rows + 1:
        raise _lib.SparseTIRError("ColumnPartHyb: indptr must have num_rows + 1 entries")
    dev = indptr.device
    widths = np.ascontiguousarray(np.asarray(list(buckets), dtype=np.int32))
    nb = len(widths)
    nk = num_col_parts * nb
    with torch.cuda.device(dev):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        ws_bytes = L.stir_column_part_hyb_device_workspace_bytes(num_rows, num_col_parts, nb, indices.numel())
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
        nrows = np.zeros(max(nk, 1), np.int64)
        _lib.check(L.stir_column_part_hyb_device_sizes(
            num_rows, num_cols, ctypes.c_void_p(indptr.data_ptr()),
            ctypes.c_void_p(indices.data_ptr()), num_col_parts, _vp(widths), nb,
            ctypes.c_void_p(ws.data_ptr()), _vp(nrows), stream))
        # one allocation per kind, the buckets are 256-byte aligned views into it
        def carve(dtype, shapes):
            offs, total = [], 0
            for shp in shapes:
                offs.append(total)
                total += (int(np.prod(shp)) + 63) // 64 * 64
            pool = torch.empty(max(total, 1), dtype=dtype, device=dev)
            return [pool[o:o + int(np.prod(shp))].view(shp) for o, shp in zip(offs, shapes)]

        wide = [(int(nrows[k]), int(widths[k % nb])) for k in range(nk)]
        rows = carve(torch.int32, [(int(nrows[k]),) for k in range(nk)])
        cols = carve(torch.int32, wide)
        mask = carve(torch.int32, wide)
        _lib.check(L.stir_column_part_hyb_device_fill(
            num_rows, num_cols, ctypes.c_void_p(indptr.data_ptr()),
            ctypes.c_void_p(indices.data_ptr()), num_col_parts, _vp(widths), nb,
            ctypes.c_void_p(ws.data_ptr()),
            _lib.ptr_table([a.data_ptr() for a in rows]),
            _lib.ptr_table([a.data_ptr() for a in cols]),
            _lib.ptr_table([a.data_ptr() for a in mask]), stream))
        avals = None
        if values is not None:
            if not _is_cuda_tensor(values) or values.dtype != torch.float32 or values.numel() != indices.numel():
                raise _lib.SparseTIRError("ColumnPartHyb: values must be a float32 CUDA tensor aligned with indices")
            values = values.contiguous()
            avals = carve(torch.float32, wide)
            _lib.check(L.stir_column_part_hyb_device_values(
                num_rows, num_cols, ctypes.c_void_p(indptr.data_ptr()),
                ctypes.c_void_p(indices.data_ptr()), ctypes.c_void_p(values.data_ptr()),
                num_col_parts, _vp(widths), nb, ctypes.c_void_p(ws.data_ptr()), _vp(nrows),
                _lib.ptr_table([a.data_ptr() for a in avals]), stream))
        # the workspace is read by the fill kernels: keep it alive until they are done
        torch.cuda.current_stream().synchronize()
    nest = lambda xs: [[xs[p * nb + b] for b in range(nb)] for p in range(num_col_parts)]
    if avals is not None:
        return nest(rows), nest(cols), nest(mask), nest(avals)
    return nest(rows), nest(cols), nest(mask)


def suggest_decomposition(num_rows, num_cols, nnz, feat):
    """``(num_col_parts, buckets)`` to hand to :func:`column_part_hyb` for hyb SpMM on an MI355X:
    the counterpart of the per-graph tables ``col_part_config`` / ``bucketing_config`` of the
    reference (examples/spmm/bench_spmm.py:233-253), which were tuned by hand for another GPU.

    The rule is what was measured on MI355X, at every size and feature width tried: **one column
    partition, widths 1, 2, 4, ... 512**.

    * Column partitions never pay.  A partition's slice of the dense operand would have to fit the
      4 MB L2 of an XCD to raise the hit rate, i.e. hundreds of partitions for a graph of millions
      of nodes, while every partition beyond the first reads and writes the output once more.
      2.45 M nodes / 61.8 M edges, 128 features: 1 / 2 / 4 / 8 / 16 partitions take
      5.07 / 5.29 / 5.62 / 5.23 / 5.21 ms with uniform columns and 4.04 / 4.03 / 4.11 / 4.27 / 4.29 ms
      with power-law columns; 169 k nodes / 1.16 M edges: 24 / 32 / 47 / 83 / 83 us at 32 features,
      189 / 237 / 232 / 236 / 236 us at 256 (CSR row-split: 39 and 202 us).
    * The widest bucket should reach a few hundred slots: rows above it are cut into several ELL
      rows that meet in atomics.  Widest bucket 32 / 64 / 128 / 256 / 512 / 1024 on the large
      graph: 6.2 / 4.4 / 4.1 / 4.0 / 4.0 / 4.0 ms.  Empty buckets cost nothing.

    ``num_rows``, ``nnz`` and ``feat`` do not change the answer today; they are part of the
    signature because the rule is a measured one and may come to depend on them.  The widths stop
    at the first power of two that covers ``num_cols`` (no row has more distinct columns)."""
    if min(int(num_rows), int(num_cols), int(feat)) <= 0 or int(nnz) < 0:
        raise _lib.SparseTIRError("suggest_decomposition: sizes must be positive")
    buckets = [1]
    while buckets[-1] < 512 and buckets[-1] < int(num_cols):
        buckets.append(buckets[-1] * 2)
    return 1, buckets


def csr_to_bsr(indptr, indices, values, shape, blocksize, dtype=None):
    """Pack a CSR matrix (CUDA tensors: int32 indptr/indices, float32 values, no duplicate
    entries) into BSR with ``blocksize x blocksize`` blocks on the GPU.

    Returns ``(bsr_indptr, bsr_indices, bsr_data)`` as CUDA tensors; block columns ascend in
    each block row and ``bsr_data`` is ``(nnzb, blocksize, blocksize)`` of ``dtype``
    (float32 by default, float16 / bfloat16 for direct use by the BSR SpMM operator) -- the
    arrays ``scipy.sparse.csr_matrix.tobsr`` returns, which is how the reference's BSR example
    builds its input (examples/blocksparse/bsr_spmm.py:441-445).
    """
    import torch

    L = _lib.lib()
    m, n = int(shape[0]), int(shape[1])
    blk = int(blocksize)
    dtype = torch.float32 if dtype is None else dtype
    codes = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}
    if dtype not in codes:
        raise _lib.SparseTIRError("csr_to_bsr: dtype must be float32, float16 or bfloat16")
    for t, name, dt in ((indptr, "indptr", torch.int32), (indices, "indices", torch.int32),
                        (values, "values", torch.float32)):
        if not _is_cuda_tensor(t):
            raise _lib.SparseTIRError(f"csr_to_bsr: {name} must be a CUDA tensor")
        if t.dtype != dt:
            raise _lib.SparseTIRError(f"csr_to_bsr: {name} must be {dt}")
    if indptr.numel() != m + 1 or values.numel() != indices.numel():
        raise _lib.SparseTIRError("csr_to_bsr: array lengths do not fit the shape")
    indptr, indices, values = indptr.contiguous(), indices.contiguous(), values.contiguous()
    dev = indptr.device
    with torch.cuda.device(dev):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        ws = torch.empty(max(256, L.stir_csr_to_bsr_workspace_bytes(m, n, blk)), dtype=torch.uint8, device=dev)
        if blk <= 0 or m % blk or n % blk:
            raise _lib.SparseTIRError(f"csr_to_bsr: shape {m} x {n} is not a multiple of the block size {blk}")
        bptr = torch.empty(m // blk + 1, dtype=torch.int32, device=dev)
        nnzb = ctypes.c_int64(0)
        p = lambda t: ctypes.c_void_p(t.data_ptr())
        _lib.check(L.stir_csr_to_bsr_sizes(m, n, blk, p(indptr), p(indices), p(ws), p(bptr),
                                           ctypes.byref(nnzb), stream))
        bidx = torch.empty(nnzb.value, dtype=torch.int32, device=dev)
        bdata = torch.empty((nnzb.value, blk, blk), dtype=dtype, device=dev)
        _lib.check(L.stir_csr_to_bsr_fill(m, n, blk, p(indptr), p(indices), p(values), p(ws), p(bptr),
                                          ctypes.c_void_p(bidx.data_ptr() if nnzb.value else 0),
                                          ctypes.c_void_p(bdata.data_ptr() if nnzb.value else 0),
                                          codes[dtype], nnzb.value, stream))
        torch.cuda.current_stream().synchronize()
    return bptr, bidx, bdata


def condense(indptr_nd, indices_nd, t, g):
    """Condense a CSR matrix to (t x 1) tiles and group g tiles together.

    Returns ``(group_indptr, tile_indices, mask)`` shaped ``(ceil(n/t)+1,)``, ``(G, g)``,
    ``(G, t, g)``.

    Extension: CUDA tensors are condensed on the GPU and CUDA tensors come back (the reference
    accepts CPU arrays only, src/sparse/format.cc:360-361).
    """
    if _is_cuda_tensor(indptr_nd) or _is_cuda_tensor(indices_nd):
        return _condense_device(indptr_nd, indices_nd, t, g)
    L = _lib.lib()
    indptr = _host_i32(indptr_nd, "indptr")
    indices = _host_i32(indices_nd, "indices")
    n = indptr.shape[0] - 1
    if t <= 0 or g <= 0:
        raise _lib.SparseTIRError(f"ConDense: t={t} g={g} must be positive")
    tiles = (n + t - 1) // t
    gptr = np.empty(tiles + 1, np.int32)
    ng = np.zeros(1, np.int64)
    _lib.check(L.stir_condense_sizes(n, _vp(indptr), _vp(indices), t, g, _vp(gptr), _vp(ng)))
    G = int(ng[0])
    tile_indices = np.empty((G, g), np.int32)
    mask = np.empty((G, t, g), np.int32)
    _lib.check(L.stir_condense_fill(n, _vp(indptr), _vp(indices), t, g, _vp(tile_indices),
                                    _vp(mask)))
    return gptr, tile_indices, mask


def csf_to_ell3d(csf_indptr_0, csf_indices_0, csf_indptr_1, csf_indices_1, nnz_rows_bkt,
                 nnz_cols_bkt):
    """Convert CSF (relation -> row -> column) to the bucketed ELL3D format.

    Returns ``(indptr, row_indices, col_indices, mask)``, each a list over buckets, shaped
    ``(R+1,)``, ``(G, rb)``, ``(G, rb, cb)``, ``(G, rb, cb)``.

    Extension: CUDA tensors are converted on the GPU and CUDA tensors come back (the reference
    accepts CPU arrays only, src/sparse/format.cc:195-202); the row ids of every relation must
    then ascend strictly.
    """
    if any(_is_cuda_tensor(a) for a in (csf_indptr_0, csf_indices_0, csf_indptr_1, csf_indices_1)):
        return _csf_to_ell3d_device(csf_indptr_0, csf_indices_0, csf_indptr_1, csf_indices_1,
                                    nnz_rows_bkt, nnz_cols_bkt)
    L = _lib.lib()
    p0 = _host_i32(csf_indptr_0, "csf_indptr_0")
    i0 = _host_i32(csf_indices_0, "csf_indices_0")
    p1 = _host_i32(csf_indptr_1, "csf_indptr_1")
    i1 = _host_i32(csf_indices_1, "csf_indices_1")
    rb = np.ascontiguousarray(np.asarray(list(nnz_rows_bkt), dtype=np.int32))
    cb = np.ascontiguousarray(np.asarray(list(nnz_cols_bkt), dtype=np.int32))
    if len(rb) != len(cb):
        raise _lib.SparseTIRError("Input nnz_rows and nnz_cols should have same length.")
    nb = len(cb)
    num_rels = p0.shape[0] - 1
    groups = np.zeros(max(nb, 1), np.int64)
    _lib.check(L.stir_csf_to_ell3d_sizes(num_rels, _vp(p0), _vp(i0), _vp(p1), _vp(i1), _vp(rb),
                                         _vp(cb), nb, _vp(groups)))
    out_ptr = [np.empty(num_rels + 1, np.int32) for _ in range(nb)]
    rows = [np.empty((int(groups[b]), int(rb[b])), np.int32) for b in range(nb)]
    cols = [np.empty((int(groups[b]), int(rb[b]), int(cb[b])), np.int32) for b in range(nb)]
    mask = [np.empty((int(groups[b]), int(rb[b]), int(cb[b])), np.int32) for b in range(nb)]
    _lib.check(L.stir_csf_to_ell3d_fill(
        num_rels, _vp(p0), _vp(i0), _vp(p1), _vp(i1), _vp(rb), _vp(cb), nb,
        _lib.ptr_table([a.ctypes.data for a in out_ptr]),
        _lib.ptr_table([a.ctypes.data for a in rows]),
        _lib.ptr_table([a.ctypes.data for a in cols]),
        _lib.ptr_table([a.ctypes.data for a in mask])))
    return out_ptr, rows, cols, mask


def _csf_to_ell3d_device(p0, i0, p1, i1, nnz_rows_bkt, nnz_cols_bkt):
    import torch

    L = _lib.lib()
    names = ("csf_indptr_0", "csf_indices_0", "csf_indptr_1", "csf_indices_1")
    for t, name in zip((p0, i0, p1, i1), names):
        if not _is_cuda_tensor(t):
            raise _lib.SparseTIRError("CSFToELL3D(device): the four CSF arrays must all be CUDA tensors")
        if t.dtype != torch.int32:
            raise _lib.SparseTIRError(
                f"Only support int32 index data type, got {t.element_size() * 8} bits for {name}.")
    p0, i0, p1, i1 = (t.contiguous().reshape(-1) for t in (p0, i0, p1, i1))
    rb = np.ascontiguousarray(np.asarray(list(nnz_rows_bkt), dtype=np.int32))
    cb = np.ascontiguousarray(np.asarray(list(nnz_cols_bkt), dtype=np.int32))
    if len(rb) != len(cb):
        raise _lib.SparseTIRError("Input nnz_rows and nnz_cols should have same length.")
    nb = len(cb)
    num_rels = p0.numel() - 1
    stored, nnz = i0.numel(), i1.numel()
    if num_rels < 0 or p1.numel() != stored + 1:
        raise _lib.SparseTIRError("CSFToELL3D: csf_indptr_1 must have one entry more than csf_indices_0")
    dev = p0.device
    dp = lambda t: ctypes.c_void_p(t.data_ptr())
    with torch.cuda.device(dev):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        ws_bytes = L.stir_csf_to_ell3d_device_workspace_bytes(num_rels, stored, max(nb, 1))
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
        groups = np.zeros(max(nb, 1), np.int64)
        _lib.check(L.stir_csf_to_ell3d_device_sizes(num_rels, stored, nnz, dp(p0), dp(i0), dp(p1), dp(i1),
                                                    _vp(rb), _vp(cb), nb, dp(ws), _vp(groups), stream))
        out_ptr = [torch.empty(num_rels + 1, dtype=torch.int32, device=dev) for _ in range(nb)]
        rows = [torch.empty((int(groups[b]), int(rb[b])), dtype=torch.int32, device=dev) for b in range(nb)]
        cols = [torch.empty((int(groups[b]), int(rb[b]), int(cb[b])), dtype=torch.int32, device=dev)
                for b in range(nb)]
        mask = [torch.empty((int(groups[b]), int(rb[b]), int(cb[b])), dtype=torch.int32, device=dev)
                for b in range(nb)]
        table = lambda xs: _lib.ptr_table([a.data_ptr() if a.numel() else 0 for a in xs])
        _lib.check(L.stir_csf_to_ell3d_device_fill(num_rels, stored, nnz, dp(p0), dp(i0), dp(p1), dp(i1),
                                                   _vp(rb), _vp(cb), nb, dp(ws), _vp(groups), table(out_ptr),
                                                   table(rows), table(cols), table(mask), stream))
        # the workspace is read by the fill kernels: keep it alive until they are done
        torch.cuda.current_stream().synchronize()
    return out_ptr, rows, cols, mask


def _condense_device(indptr, indices, t, g):
    import torch

    L = _lib.lib()
    for a, name in ((indptr, "indptr"), (indices, "indices")):
        if not _is_cuda_tensor(a):
            raise _lib.SparseTIRError("ConDense(device): indptr and indices must both be CUDA tensors")
        if a.dtype != torch.int32:
            raise _lib.SparseTIRError(
                f"Only support int32 index data type, got {a.element_size() * 8} bits for {name}.")
    t, g = int(t), int(g)
    if t <= 0 or g <= 0:
        raise _lib.SparseTIRError(f"ConDense: t={t} g={g} must be positive")
    indptr, indices = indptr.contiguous().reshape(-1), indices.contiguous().reshape(-1)
    n, nnz = indptr.numel() - 1, indices.numel()
    if n < 0:
        raise _lib.SparseTIRError("ConDense: indptr must have at least one entry")
    dev = indptr.device
    dp = lambda a: ctypes.c_void_p(a.data_ptr() if a.numel() else 0)
    with torch.cuda.device(dev):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        ws = torch.empty(max(L.stir_condense_device_workspace_bytes(n, nnz, t), 256), dtype=torch.uint8, device=dev)
        gptr = torch.empty((n + t - 1) // t + 1, dtype=torch.int32, device=dev)
        ng = ctypes.c_int64(0)
        _lib.check(L.stir_condense_device_sizes(n, nnz, dp(indptr), dp(indices), t, g, dp(ws), dp(gptr),
                                                ctypes.byref(ng), stream))
        G = ng.value
        tile_indices = torch.empty((G, g), dtype=torch.int32, device=dev)
        mask = torch.empty((G, t, g), dtype=torch.int32, device=dev)
        _lib.check(L.stir_condense_device_fill(n, nnz, dp(indptr), dp(indices), t, g, dp(ws), dp(gptr), G,
                                               dp(tile_indices), dp(mask), stream))
        # the workspace is read by the fill kernels: keep it alive until they are done
        torch.cuda.current_stream().synchronize()
    return gptr, tile_indices, mask
