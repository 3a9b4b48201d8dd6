"""On-disk cache of decomposed formats.

The reference keeps the result of ``column_part_hyb`` in a module-level variable so that one
process decomposes a graph once (examples/spmm/bench_spmm.py:88,107-114).  This keeps it across
processes: the index arrays are stored as one ``.npz`` per (graph, parameters), keyed by a hash of
the CSR arrays and the parameters.
"""
import hashlib
import os

import numpy as np

from . import format as _format


def _key(indptr, indices, params):
    h = hashlib.sha1()
    h.update(np.ascontiguousarray(indptr, dtype=np.int32).tobytes())
    h.update(np.ascontiguousarray(indices, dtype=np.int32).tobytes())
    h.update(repr(params).encode())
    return h.hexdigest()


def cached_column_part_hyb(cache_dir, num_rows, num_cols, indptr, indices, num_col_parts, buckets):
    """``column_part_hyb`` on host arrays, memoised under ``cache_dir``.  Returns the same nested
    lists of int32 numpy arrays as :func:`sparsetir_amd.format.column_part_hyb`."""
    indptr = np.ascontiguousarray(indptr, dtype=np.int32)
    indices = np.ascontiguousarray(indices, dtype=np.int32)
    buckets = [int(b) for b in buckets]
    params = ("column_part_hyb", int(num_rows), int(num_cols), int(num_col_parts), tuple(buckets))
    path = os.path.join(cache_dir, _key(indptr, indices, params) + ".npz")
    nb = len(buckets)
    if os.path.exists(path):
        with np.load(path) as z:
            get = lambda name: [[z[f"{name}_{p}_{b}"] for b in range(nb)] for p in range(num_col_parts)]
            return get("rows"), get("cols"), get("mask")
    rows, cols, mask = _format.column_part_hyb(num_rows, num_cols, indptr, indices, num_col_parts, buckets)
    os.makedirs(cache_dir, exist_ok=True)
    arrays = {}
    for p in range(num_col_parts):
        for b in range(nb):
            arrays[f"rows_{p}_{b}"] = rows[p][b]
            arrays[f"cols_{p}_{b}"] = cols[p][b]
            arrays[f"mask_{p}_{b}"] = mask[p][b]
    tmp = path + f".tmp{os.getpid()}.npz"
    np.savez(tmp, **arrays)
    os.replace(tmp, path)
    return rows, cols, mask
