"""sparsetir_amd: hand-written MI355X (gfx950) kernels behind SparseTIR's operator surface.

``sparsetir_amd.format`` mirrors ``tvm.sparse`` format conversion (column_part_hyb, condense,
csf_to_ell3d); ``sparsetir_amd.ops`` gives the built operators (CSR / hyb SpMM, SDDMM, BSR
SpMM, RGMS).  Everything runs through ``libsparsetir_amd.so`` (C ABI, include/sparsetir_amd.h);
importing the operators without a built library raises.
"""
from .format import column_part_hyb, condense, csf_to_ell3d, csr_to_bsr, suggest_decomposition  # noqa: F401

__all__ = ["column_part_hyb", "condense", "csf_to_ell3d", "csr_to_bsr", "suggest_decomposition"]
