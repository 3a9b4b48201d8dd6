"""ctypes binding of ``libsparsetir_amd.so`` (declared in ``include/sparsetir_amd.h``).

There is no fallback: if the library has not been built, importing this module raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsparsetir_amd.so")

c_i32p = ctypes.POINTER(ctypes.c_int32)
c_i64p = ctypes.POINTER(ctypes.c_int64)
c_f32p = ctypes.POINTER(ctypes.c_float)
c_pp = ctypes.POINTER(ctypes.c_void_p)
I32, I64, VP, SZ = ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p, ctypes.c_size_t

# name -> (restype, argtypes); every symbol the header declares is listed here and
# tests/test_abi.py checks the two stay in step.
SIGNATURES = {
    "stir_last_error": (ctypes.c_char_p, []),
    "stir_version": (ctypes.c_char_p, []),
    "stir_column_part_hyb_sizes": (I32, [I32, I32, VP, VP, I32, VP, I32, VP]),
    "stir_column_part_hyb_fill": (I32, [I32, I32, VP, VP, I32, VP, I32, VP, VP, VP]),
    "stir_csf_to_ell3d_sizes": (I32, [I32, VP, VP, VP, VP, VP, VP, I32, VP]),
    "stir_csf_to_ell3d_fill": (I32, [I32, VP, VP, VP, VP, VP, VP, I32, VP, VP, VP, VP]),
    "stir_condense_sizes": (I32, [I32, VP, VP, I32, I32, VP, VP]),
    "stir_condense_fill": (I32, [I32, VP, VP, I32, I32, VP, VP]),
    "stir_column_part_hyb_device_workspace_bytes": (SZ, [I32, I32, I32, I64]),
    "stir_column_part_hyb_device_sizes": (I32, [I32, I32, VP, VP, I32, VP, I32, VP, VP, VP]),
    "stir_column_part_hyb_device_fill": (I32, [I32, I32, VP, VP, I32, VP, I32, VP, VP, VP, VP, VP]),
    "stir_column_part_hyb_device_values": (I32, [I32, I32, VP, VP, VP, I32, VP, I32, VP, VP, VP, VP]),
    "stir_csf_to_ell3d_device_workspace_bytes": (SZ, [I32, I64, I32]),
    "stir_csf_to_ell3d_device_sizes": (I32, [I32, I64, I64, VP, VP, VP, VP, VP, VP, I32, VP, VP, VP]),
    "stir_csf_to_ell3d_device_fill": (I32, [I32, I64, I64, VP, VP, VP, VP, VP, VP, I32, VP, VP, VP, VP, VP, VP, VP]),
    "stir_condense_device_workspace_bytes": (SZ, [I32, I64, I32]),
    "stir_condense_device_sizes": (I32, [I32, I64, VP, VP, I32, I32, VP, VP, VP, VP]),
    "stir_condense_device_fill": (I32, [I32, I64, VP, VP, I32, I32, VP, VP, I64, VP, VP, VP]),
    "stir_csr_to_bsr_workspace_bytes": (SZ, [I32, I32, I32]),
    "stir_csr_to_bsr_sizes": (I32, [I32, I32, I32, VP, VP, VP, VP, VP, VP]),
    "stir_csr_to_bsr_fill": (I32, [I32, I32, I32, VP, VP, VP, VP, VP, VP, VP, I32, I64, VP]),
    "stir_csr_spmm_f32": (I32, [I32, I32, I32, I64, VP, VP, VP, VP, VP, VP]),
    "stir_hyb_plan_create": (I32, [VP, I32, I32, I32, I32, VP, VP, VP, VP, VP]),
    "stir_hyb_plan_create_ex": (I32, [VP, I32, I32, I32, I32, VP, VP, VP, VP, VP, ctypes.c_uint32]),
    "stir_hyb_spmm_f32": (I32, [VP, I32, VP, VP, VP]),
    "stir_hyb_plan_destroy": (I32, [VP]),
    "stir_hyb_spmm_f32_noalloc": (I32, [I32, I32, I32, I32, VP, VP, VP, VP, VP, I32, VP, VP, VP]),
    "stir_sddmm_preproc": (I32, [I32, I64, VP, VP, VP]),
    "stir_sddmm_f32": (I32, [I32, I32, I32, I64, VP, VP, VP, VP, VP, VP, VP]),
    "stir_sddmm_scaled_f32": (I32, [I32, I32, I32, I64, VP, VP, VP, VP, VP, VP, VP, VP]),
    "stir_bsr_spmm": (I32, [I32, I32, I32, I32, I32, I32, I64, VP, VP, VP, VP, VP, VP]),
    "stir_dbsr_spmm": (I32, [I32, I32, I32, I32, I32, I32, I64, VP, VP, VP, VP, VP, VP, VP]),
    "stir_tc_spmm_f16": (I32, [I32, I32, I32, I32, I32, I64, VP, VP, VP, VP, VP, VP]),
    "stir_tc_plan_create": (I32, [VP, I32, VP, VP]),
    "stir_tc_spmm_f16_planned": (I32, [VP, I32, I32, I32, I32, I32, I64, VP, VP, VP, VP, VP, VP]),
    "stir_tc_plan_destroy": (I32, [VP]),
    "stir_rgms_plan_create": (I32, [VP, I32, VP, VP, VP, VP, VP, VP, VP]),
    "stir_rgms_f16": (I32, [VP, I32, I32, I32, I32, I32, VP, VP, VP, VP]),
    "stir_rgms_f16_out_f16": (I32, [VP, I32, I32, I32, I32, I32, VP, VP, VP, VP]),
    "stir_rgms_bf16": (I32, [VP, I32, I32, I32, I32, I32, VP, VP, VP, VP]),
    "stir_rgms_plan_set_static_weights": (I32, [VP, I32]),
    "stir_rgms_plan_set_addresses_only": (I32, [VP, I32]),
    "stir_rgms_plan_destroy": (I32, [VP]),
    "stir_rgms_f32_plan_create": (I32, [VP, I32, VP, VP, VP, VP, VP, VP, VP]),
    "stir_rgms_f32": (I32, [VP, I32, I32, I32, I32, I32, VP, VP, VP, VP]),
    "stir_rgms_f32_plan_set_deterministic": (I32, [VP, I32]),
    "stir_rgms_f32_plan_destroy": (I32, [VP]),
    "stir_rgms_csf_f32_plan_create": (I32, [VP, I64, I64, VP, VP, VP, VP, VP]),
    "stir_rgms_csf_f32_planned": (I32, [VP, I32, I32, I32, I32, I32, VP, VP, VP, VP]),
    "stir_rgms_csf_f32_plan_destroy": (I32, [VP]),
    "stir_rgms_csf_f32": (I32, [I32, I32, I32, I32, I32, I64, I64, VP, VP, VP, VP, VP, VP, VP, VP, VP]),
}

_lib = None


class SparseTIRError(RuntimeError):
    """Raised when a C ABI call returns -1; carries stir_last_error()."""


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m sparsetir_amd.build` "
                "(hipcc, --offload-arch=gfx950). There is no CPU fallback.")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise SparseTIRError(lib().stir_last_error().decode())


def ptr_table(ptrs):
    """ctypes array of void* from a list of integer addresses (0 for absent)."""
    return (ctypes.c_void_p * max(1, len(ptrs)))(*[ctypes.c_void_p(int(p)) for p in ptrs])
