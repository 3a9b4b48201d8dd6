"""On-disk cache of decomposed formats.

The reference keeps the result of its format pass in a module-level variable so that one process
decomposes a graph once (examples/spmm/bench_spmm.py:88,107-114; the RGCN and TC-SpMM examples
rebuild theirs on every run).  This keeps the results across processes: the index arrays of one
decomposition are stored as one ``.npz`` per (input arrays, parameters), keyed by a hash of both.

All three routines are covered -- ``column_part_hyb``, ``csf_to_ell3d`` and ``condense`` -- with the
return nesting of :mod:`sparsetir_amd.format`.  All three also take CUDA tensors: the routine then
runs on the GPU, host copies go to disk, and a later hit is uploaded to the device the inputs live
on, so the result can be handed to the operators either way.

A file is written under a temporary name and renamed, so a reader never sees half a file; a file
that cannot be read (truncated, foreign) is ignored and rewritten.
"""
import hashlib
import os
import zipfile

import numpy as np

from . import format as _format


def _is_cuda(a):
    return hasattr(a, "is_cuda") and a.is_cuda


def _host(a):
    """Contiguous int32 numpy copy/view of a numpy array or a (CPU or CUDA) torch tensor."""
    if hasattr(a, "detach"):
        a = a.detach().cpu().numpy()
    return np.ascontiguousarray(a, dtype=np.int32)


def _key(arrays, params):
    h = hashlib.sha1()
    for a in arrays:
        h.update(str(a.shape).encode())
        h.update(a.tobytes())
    h.update(repr(params).encode())
    return h.hexdigest()


def _load(path, names):
    """The named arrays of a cache file, or None when the file is absent or unreadable."""
    if not os.path.exists(path):
        return None
    try:
        with np.load(path, allow_pickle=False) as z:
            return {k: z[k] for k in names}
    except (OSError, ValueError, KeyError, zipfile.BadZipFile):
        return None


def _store(cache_dir, path, arrays):
    os.makedirs(cache_dir, exist_ok=True)
    tmp = path + f".tmp{os.getpid()}.npz"
    np.savez(tmp, **arrays)
    os.replace(tmp, path)


def cached_column_part_hyb(cache_dir, num_rows, num_cols, indptr, indices, num_col_parts, buckets):
    """``column_part_hyb`` memoised under ``cache_dir``.  Host arrays in: nested lists of int32
    numpy arrays out, as :func:`sparsetir_amd.format.column_part_hyb`.  CUDA tensors in: the same
    nesting of CUDA tensors on the inputs' device (computed on the GPU on a miss)."""
    on_device = _is_cuda(indptr) or _is_cuda(indices)
    h_ptr, h_idx = _host(indptr), _host(indices)
    buckets = [int(b) for b in buckets]
    nb, parts = len(buckets), int(num_col_parts)
    params = ("column_part_hyb", int(num_rows), int(num_cols), parts, tuple(buckets))
    path = os.path.join(cache_dir, _key((h_ptr, h_idx), params) + ".npz")
    names = [f"{kind}_{p}_{b}" for kind in ("rows", "cols", "mask") for p in range(parts) for b in range(nb)]
    z = _load(path, names)
    if z is None:
        rows, cols, mask = _format.column_part_hyb(num_rows, num_cols, indptr if on_device else h_ptr,
                                                   indices if on_device else h_idx, parts, buckets)
        z = {}
        for p in range(parts):
            for b in range(nb):
                for kind, nest in (("rows", rows), ("cols", cols), ("mask", mask)):
                    a = nest[p][b]
                    z[f"{kind}_{p}_{b}"] = a.cpu().numpy() if on_device else a
        _store(cache_dir, path, z)
        return rows, cols, mask
    if on_device:
        import torch

        dev = indptr.device if _is_cuda(indptr) else indices.device
        put = lambda a: torch.from_numpy(a).to(dev)
    else:
        put = lambda a: a
    get = lambda kind: [[put(z[f"{kind}_{p}_{b}"]) for b in range(nb)] for p in range(parts)]
    return get("rows"), get("cols"), get("mask")


def _device_of(arrays):
    for a in arrays:
        if _is_cuda(a):
            return a.device
    return None


def _uploader(dev):
    """Identity for host callers; for CUDA callers a function that puts a cached array on `dev`."""
    if dev is None:
        return lambda a: a
    import torch

    return lambda a: torch.from_numpy(a).to(dev)


def _on_host(a):
    return a.cpu().numpy() if hasattr(a, "detach") else a


def cached_csf_to_ell3d(cache_dir, csf_indptr_0, csf_indices_0, csf_indptr_1, csf_indices_1, nnz_rows_bkt,
                        nnz_cols_bkt):
    """``csf_to_ell3d`` memoised under ``cache_dir``: ``(indptr, row_indices, col_indices, mask)``,
    each a list over buckets of int32 numpy arrays -- or, when the CSF arrays are CUDA tensors, of
    CUDA tensors on their device (converted on the GPU on a miss; host copies go to disk)."""
    given = (csf_indptr_0, csf_indices_0, csf_indptr_1, csf_indices_1)
    dev = _device_of(given)
    csf = [_host(a) for a in given]
    rb, cb = [int(v) for v in nnz_rows_bkt], [int(v) for v in nnz_cols_bkt]
    nb = len(cb)
    path = os.path.join(cache_dir, _key(csf, ("csf_to_ell3d", tuple(rb), tuple(cb))) + ".npz")
    kinds = ("indptr", "rows", "cols", "mask")
    z = _load(path, [f"{kind}_{b}" for kind in kinds for b in range(nb)])
    if z is None:
        out = _format.csf_to_ell3d(*(given if dev is not None else csf), rb, cb)
        _store(cache_dir, path, {f"{kind}_{b}": _on_host(out[q][b]) for q, kind in enumerate(kinds) for b in range(nb)})
        return out
    put = _uploader(dev)
    return tuple([put(z[f"{kind}_{b}"]) for b in range(nb)] for kind in kinds)


def cached_condense(cache_dir, indptr, indices, t, g):
    """``condense`` memoised under ``cache_dir``: ``(group_indptr, tile_indices, mask)``, numpy arrays
    for host inputs and CUDA tensors for CUDA inputs (condensed on the GPU on a miss)."""
    dev = _device_of((indptr, indices))
    h_ptr, h_idx = _host(indptr), _host(indices)
    path = os.path.join(cache_dir, _key((h_ptr, h_idx), ("condense", int(t), int(g))) + ".npz")
    z = _load(path, ["group_indptr", "tile_indices", "mask"])
    if z is None:
        if dev is not None:
            gptr, tiles, mask = _format.condense(indptr, indices, t, g)
        else:
            gptr, tiles, mask = _format.condense(h_ptr, h_idx, t, g)
        _store(cache_dir, path, {"group_indptr": _on_host(gptr), "tile_indices": _on_host(tiles), "mask": _on_host(mask)})
        return gptr, tiles, mask
    put = _uploader(dev)
    return put(z["group_indptr"]), put(z["tile_indices"]), put(z["mask"])
