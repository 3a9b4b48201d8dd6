"""Calls the library's TVM-PackedFunc entry points without a TVM runtime.

``get_global_func(name)`` looks an operator up by its global name (the names a TVM runtime
would hold after ``stir_register_all``) and returns a Python callable that marshals its
arguments exactly as TVM's FFI does: integers as ``v_int64`` with type code kTVMArgInt, arrays
as ``DLTensor*`` with type code kTVMDLTensorHandle (python/tvm/_ffi/_ctypes/packed_func.py in the
reference).  Arrays may be torch tensors (CPU or GPU) or numpy arrays; they are passed by
pointer, never copied.
"""
import ctypes

import numpy as np

from . import _lib

kDLCPU, kDLROCM = 1, 10
kDLInt, kDLUInt, kDLFloat, kDLBfloat = 0, 1, 2, 4
kTVMArgInt, kTVMDLTensorHandle = 0, 7


class DLDevice(ctypes.Structure):
    _fields_ = [("device_type", ctypes.c_int), ("device_id", ctypes.c_int32)]


class DLDataType(ctypes.Structure):
    _fields_ = [("code", ctypes.c_uint8), ("bits", ctypes.c_uint8), ("lanes", ctypes.c_uint16)]


class DLTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("device", DLDevice), ("ndim", ctypes.c_int32),
                ("dtype", DLDataType), ("shape", ctypes.POINTER(ctypes.c_int64)),
                ("strides", ctypes.POINTER(ctypes.c_int64)), ("byte_offset", ctypes.c_uint64)]


class TVMValue(ctypes.Union):
    _fields_ = [("v_int64", ctypes.c_int64), ("v_float64", ctypes.c_double),
                ("v_handle", ctypes.c_void_p), ("v_str", ctypes.c_char_p)]


PackedCFunc = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.POINTER(TVMValue), ctypes.POINTER(ctypes.c_int),
                               ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p)

_NP_CODES = {"i": kDLInt, "u": kDLUInt, "f": kDLFloat}


def to_dltensor(a):
    """DLTensor view of a torch tensor or numpy array (the returned object keeps ``a`` alive)."""
    t = DLTensor()
    if isinstance(a, np.ndarray):
        t.data = a.ctypes.data
        t.device = DLDevice(kDLCPU, 0)
        t.dtype = DLDataType(_NP_CODES[a.dtype.kind], a.dtype.itemsize * 8, 1)
        shape = a.shape
        strides = [s // a.dtype.itemsize for s in a.strides]
    else:
        import torch

        t.data = a.data_ptr()
        t.device = DLDevice(kDLROCM if a.is_cuda else kDLCPU, a.device.index or 0)
        if a.dtype == torch.bfloat16:
            t.dtype = DLDataType(kDLBfloat, 16, 1)
        elif a.dtype.is_floating_point:
            t.dtype = DLDataType(kDLFloat, a.element_size() * 8, 1)
        else:
            t.dtype = DLDataType(kDLInt, a.element_size() * 8, 1)
        shape = tuple(a.shape)
        strides = list(a.stride())
    t.ndim = len(shape)
    t._shape = (ctypes.c_int64 * max(1, len(shape)))(*shape)
    t._strides = (ctypes.c_int64 * max(1, len(shape)))(*strides)
    t.shape = ctypes.cast(t._shape, ctypes.POINTER(ctypes.c_int64))
    t.strides = ctypes.cast(t._strides, ctypes.POINTER(ctypes.c_int64))
    t.byte_offset = 0
    t._owner = a
    return t


def _table():
    L = _lib.lib()
    L.stir_packed_count.restype = ctypes.c_int
    L.stir_packed_name.restype = ctypes.c_char_p
    L.stir_packed_name.argtypes = [ctypes.c_int]
    L.stir_packed_func.restype = ctypes.c_void_p
    L.stir_packed_func.argtypes = [ctypes.c_int]
    return {L.stir_packed_name(i).decode(): L.stir_packed_func(i) for i in range(L.stir_packed_count())}


def list_global_func_names():
    return sorted(_table())


class PackedFunc:
    def __init__(self, name, addr):
        self.name = name
        self._fn = PackedCFunc(addr)

    def __call__(self, *args):
        n = len(args)
        values = (TVMValue * max(1, n))()
        codes = (ctypes.c_int * max(1, n))()
        keep = []
        for i, a in enumerate(args):
            if isinstance(a, (int, np.integer)):
                values[i].v_int64 = int(a)
                codes[i] = kTVMArgInt
            else:
                t = to_dltensor(a)
                keep.append(t)
                values[i].v_handle = ctypes.addressof(t)
                codes[i] = kTVMDLTensorHandle
        rc = self._fn(values, codes, n, None, None)
        if rc != 0:
            raise _lib.SparseTIRError(_lib.lib().stir_last_error().decode())


def get_global_func(name):
    tab = _table()
    if name not in tab:
        raise ValueError(f"Cannot find global function {name}")
    return PackedFunc(name, tab[name])


def set_stream(stream_handle):
    """Stream (integer hipStream_t) for packed operator calls made by this thread."""
    L = _lib.lib()
    L.stir_set_stream.argtypes = [ctypes.c_void_p]
    L.stir_set_stream.restype = None
    L.stir_set_stream(ctypes.c_void_p(stream_handle))


def plan_builds():
    """Plans made by the packed operators since the library was loaded."""
    L = _lib.lib()
    L.stir_packed_plan_builds.restype = ctypes.c_int64
    L.stir_packed_plan_builds.argtypes = []
    return int(L.stir_packed_plan_builds())
