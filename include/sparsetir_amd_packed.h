/*
 * sparsetir_amd -- the operators with TVM's PackedFunc calling convention over DLPack tensors.
 *
 * Every operator below has the signature of TVMPackedCFunc
 * (include/tvm/runtime/c_runtime_api.h:296-306 of the reference):
 *
 *   int f(TVMValue* args, int* type_codes, int num_args, TVMRetValueHandle ret, void* resource);
 *
 * returning 0 on success and -1 after recording a message (stir_last_error(), forwarded to
 * TVMAPISetLastError when a hook is installed).  Array arguments are DLTensor* passed with type
 * code kTVMDLTensorHandle, kTVMNDArrayHandle or kTVMOpaqueHandle, integer arguments are
 * v_int64 with kTVMArgInt, exactly what the reference's generated host stubs accept
 * (src/tir/transforms/make_packed_api.cc:243-248).  Arrays are checked like BindDLTensor does
 * (src/tir/transforms/arg_binder.cc:152+): one dimension, dtype code/bits/lanes, compact strides,
 * byte_offset applied, all on one device (kDLROCM, or kDLCUDA as PyTorch-ROCm exports it).
 * Sizes are taken from the tensor shapes; what the shapes cannot give is passed as trailing
 * integers (the reference bakes those into the built module when it specialises the kernel).
 *
 * The types below repeat the public DLPack / TVM C definitions so that this header stands alone;
 * include <dlpack/dlpack.h> and <tvm/runtime/c_runtime_api.h> first to use the originals.
 */
#ifndef SPARSETIR_AMD_PACKED_H_
#define SPARSETIR_AMD_PACKED_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef DLPACK_DLPACK_H_
#define DLPACK_DLPACK_H_
typedef enum {
  kDLCPU = 1,
  kDLCUDA = 2,
  kDLCUDAHost = 3,
  kDLROCM = 10,
  kDLROCMHost = 11
} DLDeviceType;
typedef struct {
  DLDeviceType device_type;
  int32_t device_id;
} DLDevice;
typedef enum { kDLInt = 0U, kDLUInt = 1U, kDLFloat = 2U, kDLOpaqueHandle = 3U, kDLBfloat = 4U } DLDataTypeCode;
typedef struct {
  uint8_t code;
  uint8_t bits;
  uint16_t lanes;
} DLDataType;
typedef struct {
  void* data;
  DLDevice device;
  int32_t ndim;
  DLDataType dtype;
  int64_t* shape;
  int64_t* strides;
  uint64_t byte_offset;
} DLTensor;
#endif /* DLPACK_DLPACK_H_ */

#ifndef TVM_RUNTIME_C_RUNTIME_API_H_
typedef union {
  int64_t v_int64;
  double v_float64;
  void* v_handle;
  const char* v_str;
  DLDataType v_type;
  DLDevice v_device;
} TVMValue;
typedef void* TVMRetValueHandle;
typedef void* TVMFunctionHandle;
typedef int (*TVMPackedCFunc)(TVMValue* args, int* type_codes, int num_args, TVMRetValueHandle ret,
                              void* resource_handle);
typedef void (*TVMPackedCFuncFinalizer)(void* resource_handle);
enum {
  kTVMArgInt = 0,
  kTVMArgFloat = 2,
  kTVMOpaqueHandle = 3,
  kTVMNullptr = 4,
  kTVMDLTensorHandle = 7,
  kTVMNDArrayHandle = 13
};
#endif

/*
 * Operators (global names as registered by stir_register_all):
 *
 * "sparsetir.csrmm"          (A, B, C, indptr, indices)
 *      examples/spmm/bench_spmm_naive.py:121-129
 * "sparsetir.hyb_csrmm"      (B, C, A_0, rows_0, cols_0, ..., feat, num_col_parts)
 *      examples/spmm/bench_spmm.py:208-225; bucket k of partition p is triple p*nb + k
 * "sparsetir.sddmm_preproc"  (A, B, C, indptr, indices, mid)
 * "sparsetir.sddmm"          (A, B, C, indptr, indices, mid)
 *      examples/sddmm/bench_sddmm.py:106-115, 170-171
 * "sparsetir.bsrmm"          (A, X, Y, indptr, indices, blk, feat)    A, X f16 or bf16
 *      examples/blocksparse/bsr_spmm.py:427-433
 * "sparsetir.dbsrmm"         (A, X, Y, indptr_0, indices_0, indptr_1, indices_1, blk, feat)
 *      examples/blocksparse/bsr_spmm.py:66-102; only the block rows listed in indices_0 are stored
 * "sparsetir.tcspmm"         (A, B, C, indptr, indices, feat, tile_size, group_size)
 *      examples/spmm/bench_tc_spmm.py:650-656
 * "sparsetir.rgms"           (W, X, Y, A_0, rows_0, cols_0, ..., mids_0, ..., feat_in, feat_out)
 *      examples/rgms/rgcn/bench_rgcn_tensorcore.py:840-852         fp16 or bf16, W [R, feat_in, feat_out]
 * "sparsetir.rgms_f32"       same argument list, every array fp32, W [R, feat_out, feat_in]
 *      examples/rgms/rgcn/bench_rgcn_composable.py:208-221
 * "sparsetir.rgms_csf"       (A, W, X, Y, indptr_i, indices_i, indptr_j, indices_j, feat_in, feat_out)
 *      examples/rgms/rgcn/bench_rgcn_non_composable.py:109         fp32, W [R, feat_out, feat_in]
 * "sparsetir.static_structure" (on)
 *      no counterpart in the reference, whose built operators read their index arrays on every
 *      call.  Default off: "sparsetir.hyb_csrmm" and "sparsetir.rgms" then do the same -- their
 *      cached plans hold the addresses and sizes of the arrays and nothing derived from their
 *      contents (hyb: one launch, atomics in every adding bucket, the rule of
 *      examples/spmm/bench_spmm.py:170; rgms: one fp32 atomic per ELL row and output feature;
 *      rgms_f32 plans never hold more, rgms_csf has no plan), so
 *      rows / cols / mids may be rewritten in place, or freed and replaced by arrays of the same
 *      sizes at the same addresses, at any time.  on != 0 is the promise that these index arrays
 *      keep their contents for as long as they keep their addresses, which is how every script of
 *      the reference uses them (decomposed once, then timed).  Plans made from then on keep what
 *      they derive from the contents: rgms the edge index by destination tile that its first
 *      launch over 8192 slots or more builds (about four times faster at 2M edges), hyb_csrmm with
 *      2 to 4 partitions whether its buckets need atomics, with more than 4 the slot list of every
 *      output row.  Changing the setting drops the cached plans.  Edge weights (A_k), W, X, B may
 *      change freely under either setting.
 * "sparsetir.invalidate_plans" ()
 *      no counterpart in the reference.  "sparsetir.hyb_csrmm", "sparsetir.rgms" and
 *      "sparsetir.rgms_f32" each keep the eight plans used last, found again by the addresses and
 *      sizes of a call's arrays (a ninth plan replaces the one whose last use lies furthest back),
 *      so a caller that alternates between a few graphs builds each plan once.  This call
 *      destroys them all.  A caller that has promised static structure and then does rewrite
 *      rows / cols / mids in place calls it before the next operator call.
 * "sparsetir.rgms_static_weights" (on)
 *      no counterpart in the reference.  on != 0: the plans "sparsetir.rgms" makes from now on carry
 *      the promise of stir_rgms_plan_set_static_weights -- the A_k keep the values they have at the
 *      plan's first call (the reference's A_k is the 0/1 mask of CSFToELL3D, written once) -- and
 *      leave the zero-weight padding slots out of their edge index.  Takes effect together with
 *      "sparsetir.static_structure"(1): without that promise no index is kept.  Drops the cached
 *      plans when the setting changes.  Default off.
 *
 * Format pass (host tensors, kDLCPU, as in the reference, or device tensors; the reference returns
 * nested Array<NDArray>, which needs libtvm objects, so here a sizing call is followed by a fill
 * call into caller-made tensors):
 *
 * "tir.sparse.ColumnPartHyb.sizes" (num_rows, num_cols, indptr, indices, num_col_parts, buckets, nrows_out)
 * "tir.sparse.ColumnPartHyb.fill"  (num_rows, num_cols, indptr, indices, num_col_parts, buckets,
 *                                   rows_0, cols_0, mask_0, rows_1, ...)      src/sparse/format.cc:46-168
 *      buckets: int32 tensor; nrows_out: int64 tensor of num_col_parts*len(buckets).
 *      With kDLROCM/kDLCUDA indptr and indices the decomposition runs on the GPU.
 * "tir.sparse.CSFToELL3D.sizes"    (indptr0, indices0, indptr1, indices1, rows_bkt, cols_bkt, groups_out)
 * "tir.sparse.CSFToELL3D.fill"     (indptr0, indices0, indptr1, indices1, rows_bkt, cols_bkt,
 *                                   indptr_0, rows_0, cols_0, mask_0, indptr_1, ...) src/sparse/format.cc:180-343
 *      With kDLROCM/kDLCUDA CSF arrays the conversion runs on the GPU and the outputs are device
 *      tensors (row ids must ascend strictly inside a relation; .sizes first, on the same thread).
 * "tir.sparse.ConDense.sizes"      (indptr, indices, t, g, group_indptr_out, num_groups_out)
 * "tir.sparse.ConDense.fill"       (indptr, indices, t, g, tile_indices_out, mask_out)  src/sparse/format.cc:353-429
 *      With kDLROCM/kDLCUDA indptr and indices the condensing runs on the GPU: group_indptr_out and
 *      the outputs of .fill are device tensors, and .fill takes the filled group_indptr as a seventh
 *      argument (.sizes first, on the same thread).
 */
int stir_packed_csrmm(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_hyb_csrmm(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_sddmm_preproc(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_sddmm(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_bsrmm(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_dbsrmm(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_tcspmm(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_rgms(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_rgms_f32(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_rgms_csf(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_invalidate_plans(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_rgms_static_weights(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_static_structure(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_column_part_hyb_sizes(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_column_part_hyb_fill(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_csf_to_ell3d_sizes(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_csf_to_ell3d_fill(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_condense_sizes(TVMValue*, int*, int, TVMRetValueHandle, void*);
int stir_packed_condense_fill(TVMValue*, int*, int, TVMRetValueHandle, void*);

/* Plans the packed operators have made since the library was loaded (a call that finds its
 * plan among the cached ones makes none): lets a caller see that alternating graphs reuse plans. */
int64_t stir_packed_plan_builds(void);

/* Number of packed operators, and the i-th one's global name / function. */
int stir_packed_count(void);
const char* stir_packed_name(int i);
TVMPackedCFunc stir_packed_func(int i);

/*
 * Registers every operator in a TVM runtime: pass the runtime's TVMFuncCreateFromCFunc
 * (c_runtime_api.h:336) and TVMFuncRegisterGlobal (c_runtime_api.h:348).  override != 0
 * replaces existing globals of the same name.  Returns 0, or the first failing status.
 */
int stir_register_all(int (*create_from_cfunc)(TVMPackedCFunc, void*, TVMPackedCFuncFinalizer,
                                               TVMFunctionHandle*),
                      int (*register_global)(const char*, TVMFunctionHandle, int), int override);

/* Forward error messages to the host runtime (e.g. TVMAPISetLastError); NULL removes the hook. */
void stir_set_error_hook(void (*hook)(const char* msg));

/* Stream (hipStream_t) that packed operator calls made by this thread launch on; NULL = default.
 * The reference keeps the same thread-local state behind TVMSetStream (c_runtime_api.h:482). */
void stir_set_stream(void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SPARSETIR_AMD_PACKED_H_ */
