"""The TVM-PackedFunc entry points on host tensors (no GPU): format pass parity with the
oracle, argument checking, registration into a stand-in runtime table."""
import ctypes
import os
import re

import numpy as np
import pytest

import oracle
from sparsetir_amd import _lib, packed
from sparsetir_amd._lib import SparseTIRError
from helpers import random_csf, random_csr

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_and_registry_agree():
    text = open(os.path.join(ROOT, "include", "sparsetir_amd_packed.h")).read()
    declared = set(re.findall(r'^ \* "([a-zA-Z0-9_.]+)"', text, flags=re.M))
    assert declared == set(packed.list_global_func_names())
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for sym in re.findall(r"\b(stir_[a-z0-9_]+)\s*\(", re.sub(r"/\*.*?\*/", "", text, flags=re.S)):
        assert hasattr(lib, sym), sym


def test_column_part_hyb_packed_matches_oracle():
    m, n, parts, buckets = 400, 300, 3, [1, 2, 4, 8]
    indptr, indices = random_csr(m, n, 6000, 0, skew=1.0)
    b = np.asarray(buckets, np.int32)
    nrows = np.zeros(parts * len(buckets), np.int64)
    packed.get_global_func("tir.sparse.ColumnPartHyb.sizes")(m, n, indptr, indices, parts, b, nrows)
    outs = []
    for k, r in enumerate(nrows):
        w = buckets[k % len(buckets)]
        outs += [np.empty(r, np.int32), np.empty(r * w, np.int32), np.empty(r * w, np.int32)]
    packed.get_global_func("tir.sparse.ColumnPartHyb.fill")(m, n, indptr, indices, parts, b, *outs)
    rows, cols, mask = oracle.column_part_hyb(m, n, indptr, indices, parts, buckets)
    for p in range(parts):
        for q in range(len(buckets)):
            k = p * len(buckets) + q
            assert np.array_equal(outs[3 * k], rows[p][q])
            assert np.array_equal(outs[3 * k + 1], cols[p][q].ravel())
            assert np.array_equal(outs[3 * k + 2], mask[p][q].ravel())


def test_csf_to_ell3d_packed_matches_oracle():
    csf = random_csf(6, 80, 1500, 1)
    rb, cb = np.asarray([8, 4, 2, 1], np.int32), np.asarray([1, 2, 4, 8], np.int32)
    groups = np.zeros(4, np.int64)
    packed.get_global_func("tir.sparse.CSFToELL3D.sizes")(*csf, rb, cb, groups)
    outs = []
    for b in range(4):
        g = int(groups[b])
        outs += [np.empty(7, np.int32), np.empty(g * rb[b], np.int32), np.empty(g * rb[b] * cb[b], np.int32),
                 np.empty(g * rb[b] * cb[b], np.int32)]
    packed.get_global_func("tir.sparse.CSFToELL3D.fill")(*csf, rb, cb, *outs)
    want = oracle.csf_to_ell3d(*csf, rb, cb)
    for b in range(4):
        for q in range(4):
            assert np.array_equal(outs[4 * b + q], want[q][b].ravel())


def test_condense_packed_matches_oracle():
    indptr, indices = random_csr(130, 90, 2000, 2)
    t, g = 8, 4
    gptr = np.empty((130 + t - 1) // t + 1, np.int32)
    ng = np.zeros(1, np.int64)
    packed.get_global_func("tir.sparse.ConDense.sizes")(indptr, indices, t, g, gptr, ng)
    tiles = np.empty(int(ng[0]) * g, np.int32)
    mask = np.empty(int(ng[0]) * t * g, np.int32)
    packed.get_global_func("tir.sparse.ConDense.fill")(indptr, indices, t, g, tiles, mask)
    want = oracle.condense(indptr, indices, t, g)
    assert np.array_equal(gptr, want[0])
    assert np.array_equal(tiles, want[1].ravel())
    assert np.array_equal(mask, want[2].ravel())


def test_packed_argument_checks():
    f = packed.get_global_func("tir.sparse.ColumnPartHyb.sizes")
    indptr, indices = random_csr(10, 10, 30, 3)
    b = np.asarray([1, 2], np.int32)
    nrows = np.zeros(2, np.int64)
    with pytest.raises(SparseTIRError, match="num_args should be 7"):
        f(10, 10, indptr, indices, 1, b, nrows, 5)
    with pytest.raises(SparseTIRError, match="dtype"):
        f(10, 10, indptr.astype(np.int64), indices, 1, b, nrows)
    with pytest.raises(SparseTIRError, match="ndim"):
        f(10, 10, indptr.reshape(1, -1), indices, 1, b, nrows)
    with pytest.raises(SparseTIRError, match="to be int"):
        f(indptr, 10, indptr, indices, 1, b, nrows)
    with pytest.raises(SparseTIRError, match="compact"):
        f(10, 10, np.repeat(indptr, 2)[::2], indices, 1, b, nrows)
    with pytest.raises(SparseTIRError, match="shape"):
        f(9, 10, indptr, indices, 1, b, nrows)
    with pytest.raises(SparseTIRError, match="GPU"):
        packed.get_global_func("sparsetir.csrmm")(np.zeros(1, np.float32), np.zeros(4, np.float32),
                                                  np.zeros(4, np.float32), np.zeros(2, np.int32),
                                                  np.zeros(1, np.int32))


def test_register_all_fills_a_runtime_table():
    """stir_register_all drives TVMFuncCreateFromCFunc / TVMFuncRegisterGlobal; a stand-in for
    both records what a TVM runtime would end up holding."""
    L = _lib.lib()
    table, handles = {}, []
    CREATE = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                              ctypes.POINTER(ctypes.c_void_p))
    REGISTER = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_char_p, ctypes.c_void_p, ctypes.c_int)

    def create(fn, resource, fin, out):
        handles.append(fn)
        out[0] = len(handles)  # opaque function handle
        return 0

    def register(name, handle, override):
        table[name.decode()] = (handles[handle - 1], override)
        return 0

    c, r = CREATE(create), REGISTER(register)
    L.stir_register_all.argtypes = [CREATE, REGISTER, ctypes.c_int]
    assert L.stir_register_all(c, r, 1) == 0
    assert sorted(table) == packed.list_global_func_names()
    assert all(ov == 1 for _, ov in table.values())
    assert "tir.sparse.ColumnPartHyb.sizes" in table and "sparsetir.hyb_csrmm" in table


def test_error_hook_receives_messages():
    L = _lib.lib()
    seen = []
    HOOK = ctypes.CFUNCTYPE(None, ctypes.c_char_p)
    hook = HOOK(lambda msg: seen.append(msg.decode()))
    L.stir_set_error_hook.argtypes = [HOOK]
    L.stir_set_error_hook(hook)
    try:
        with pytest.raises(SparseTIRError):
            packed.get_global_func("tir.sparse.ConDense.sizes")(1, 2, 3)
        assert seen and "num_args should be 6" in seen[-1]
    finally:
        L.stir_set_error_hook(ctypes.cast(None, HOOK))
