/*
 * sparsetir_amd -- C ABI of the MI355X (gfx950) implementation of the kernels that
 * SparseTIR generates for SpMM / SDDMM / BSR / RGMS, and of its format-decomposition pass.
 *
 * Conventions
 *   - Every function returns 0 on success and -1 on failure; stir_last_error() then gives
 *     the reason (same convention as TVMAPISetLastError / TVMGetLastError,
 *     include/tvm/runtime/c_runtime_api.h:181-190 of the reference).
 *   - All index arrays are int32, all buffers are flat and contiguous, exactly the layout
 *     the reference's lowered functions take (src/tir/transforms/lower_sparse_buffer.cc:46-58).
 *   - "d_" parameters are device pointers on the current HIP device; others are host pointers.
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream).  Launches are
 *     asynchronous, like the reference's ROCMWrappedFunc (src/runtime/rocm/rocm_module.cc:146-189).
 *   - Kernels write into caller-owned outputs; outputs that are accumulated with atomics
 *     (hyb, RGMS) must be zero-filled by the caller, as in the reference
 *     (examples/spmm/bench_spmm.py:206, examples/rgms/rgcn/bench_rgcn_tensorcore.py:843).
 */
#ifndef SPARSETIR_AMD_H_
#define SPARSETIR_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Message of the last failure on the calling thread. */
const char* stir_last_error(void);

/* Library version string. */
const char* stir_version(void);

/* Element types of 16-bit / 32-bit floating-point operands. */
enum { STIR_F16 = 0, STIR_BF16 = 1, STIR_F32 = 2 };

/* ------------------------------------------------------------------ format pass (host) */

/*
 * ColumnPartHyb, src/sparse/format.cc:46-168 (Python: python/tvm/sparse/format.py:89-116).
 * Two calls: _sizes fills nrows[num_col_parts*num_buckets] (ELL rows per (part, bucket),
 * part-major); _fill writes, for k = part*num_buckets + bucket, row_indices[k] (nrows[k]),
 * col_indices[k] and mask[k] (nrows[k]*buckets[bucket]) -- all host int32, fully written.
 */
int stir_column_part_hyb_sizes(int32_t num_rows, int32_t num_cols, const int32_t* indptr,
                               const int32_t* indices, int32_t num_col_parts,
                               const int32_t* buckets, int32_t num_buckets, int64_t* nrows);
int stir_column_part_hyb_fill(int32_t num_rows, int32_t num_cols, const int32_t* indptr,
                              const int32_t* indices, int32_t num_col_parts,
                              const int32_t* buckets, int32_t num_buckets,
                              int32_t* const* row_indices, int32_t* const* col_indices,
                              int32_t* const* mask);

/*
 * CSFToELL3D, src/sparse/format.cc:180-343 (Python: python/tvm/sparse/format.py:142-170).
 * _sizes fills groups[num_buckets]; _fill writes per bucket b: indptr[b] (num_rels+1),
 * row_indices[b] (groups*rows_bkt[b]), col_indices[b] / mask[b] (groups*rows_bkt[b]*cols_bkt[b]).
 */
int stir_csf_to_ell3d_sizes(int32_t num_rels, const int32_t* indptr0, const int32_t* indices0,
                            const int32_t* indptr1, const int32_t* indices1,
                            const int32_t* rows_bkt, const int32_t* cols_bkt,
                            int32_t num_buckets, int64_t* groups);
int stir_csf_to_ell3d_fill(int32_t num_rels, const int32_t* indptr0, const int32_t* indices0,
                           const int32_t* indptr1, const int32_t* indices1,
                           const int32_t* rows_bkt, const int32_t* cols_bkt,
                           int32_t num_buckets, int32_t* const* indptr,
                           int32_t* const* row_indices, int32_t* const* col_indices,
                           int32_t* const* mask);

/*
 * ConDense, src/sparse/format.cc:353-429 (Python: python/tvm/sparse/format.py:119-139).
 * _sizes fills group_indptr[ceil(n/t)+1] and *num_groups; _fill writes tile_indices
 * (num_groups*g) and mask (num_groups*t*g).
 */
int stir_condense_sizes(int32_t n, const int32_t* indptr, const int32_t* indices, int32_t t,
                        int32_t g, int32_t* group_indptr, int64_t* num_groups);
int stir_condense_fill(int32_t n, const int32_t* indptr, const int32_t* indices, int32_t t,
                       int32_t g, int32_t* tile_indices, int32_t* mask);

/* ---------------------------------------------------------------- format pass (device) */

/*
 * ColumnPartHyb on the GPU, bit-exact with the host routine above (the reference runs this on
 * the CPU only, src/sparse/format.cc:58-59).  CSR rows whose entries are ordered by column
 * partition -- ascending columns in particular -- take the fast path; other input is first
 * regrouped by (row, partition) with a stable sort, which keeps the order the sequential
 * routine produces.  d_workspace must hold
 * stir_column_part_hyb_device_workspace_bytes(num_rows, num_col_parts, num_buckets, nnz) bytes
 * and must stay untouched between the _sizes and the _fill / _values calls.  _sizes
 * synchronises the stream to return nrows on the host; _fill writes device arrays through host
 * tables of device pointers (k = part*num_buckets + bucket).
 */
size_t stir_column_part_hyb_device_workspace_bytes(int32_t num_rows, int32_t num_col_parts,
                                                   int32_t num_buckets, int64_t nnz);
int stir_column_part_hyb_device_sizes(int32_t num_rows, int32_t num_cols,
                                      const int32_t* d_indptr, const int32_t* d_indices,
                                      int32_t num_col_parts, const int32_t* buckets,
                                      int32_t num_buckets, void* d_workspace, int64_t* nrows,
                                      void* stream);
int stir_column_part_hyb_device_fill(int32_t num_rows, int32_t num_cols,
                                     const int32_t* d_indptr, const int32_t* d_indices,
                                     int32_t num_col_parts, const int32_t* buckets,
                                     int32_t num_buckets, void* d_workspace,
                                     int32_t* const* d_row_indices,
                                     int32_t* const* d_col_indices, int32_t* const* d_mask,
                                     void* stream);

/*
 * Value rewrite for hyb: after _sizes and _fill (same workspace), gathers the CSR values into the
 * per-bucket arrays, d_A[k][slot] = d_values[e] for the slot nonzero e was placed in, padding
 * slots zero.  This is what the reference's "rewrite_A_k" preprocess blocks compute
 * (tests/python/sparsetir/sparse_tir_composable_format_scripts.py:331-351); its example scripts
 * feed the 0/1 mask instead (examples/spmm/bench_spmm.py:211-213), which handles unweighted
 * graphs only.
 */
int stir_column_part_hyb_device_values(int32_t num_rows, int32_t num_cols, const int32_t* d_indptr,
                                       const int32_t* d_indices, const float* d_values,
                                       int32_t num_col_parts, const int32_t* buckets,
                                       int32_t num_buckets, void* d_workspace, const int64_t* nrows,
                                       float* const* d_A, void* stream);

/*
 * CSFToELL3D on the GPU, bit-exact with stir_csf_to_ell3d_sizes / _fill above (the reference runs
 * this on the CPU only, src/sparse/format.cc:195-202).  num_stored_rows is the length of
 * csf_indices_0, nnz that of csf_indices_1.  The row ids of every relation must ascend strictly
 * (the sequential routine lets two stored rows with one id share an ELL row; the device pass
 * rejects such input, the host routine takes it).  At most 32 buckets.  d_workspace must hold
 * stir_csf_to_ell3d_device_workspace_bytes(num_rels, num_stored_rows, num_buckets) bytes and stay
 * untouched between _sizes and _fill; _sizes synchronises the stream and returns groups on the
 * host, _fill takes them back and writes device arrays through host tables of device pointers.
 */
size_t stir_csf_to_ell3d_device_workspace_bytes(int32_t num_rels, int64_t num_stored_rows,
                                                int32_t num_buckets);
int stir_csf_to_ell3d_device_sizes(int32_t num_rels, int64_t num_stored_rows, int64_t nnz,
                                   const int32_t* d_indptr0, const int32_t* d_indices0,
                                   const int32_t* d_indptr1, const int32_t* d_indices1,
                                   const int32_t* rows_bkt, const int32_t* cols_bkt,
                                   int32_t num_buckets, void* d_workspace, int64_t* groups,
                                   void* stream);
int stir_csf_to_ell3d_device_fill(int32_t num_rels, int64_t num_stored_rows, int64_t nnz,
                                  const int32_t* d_indptr0, const int32_t* d_indices0,
                                  const int32_t* d_indptr1, const int32_t* d_indices1,
                                  const int32_t* rows_bkt, const int32_t* cols_bkt,
                                  int32_t num_buckets, void* d_workspace, const int64_t* groups,
                                  int32_t* const* d_indptr, int32_t* const* d_row_indices,
                                  int32_t* const* d_col_indices, int32_t* const* d_mask,
                                  void* stream);

/*
 * ConDense on the GPU, bit-exact with stir_condense_sizes / _fill above (the reference runs this
 * on the CPU only, src/sparse/format.cc:360-361).  nnz is the length of indices; column indices
 * must not be negative.  d_workspace must hold stir_condense_device_workspace_bytes(n, nnz, t)
 * bytes (32 bytes per nonzero plus sort scratch) and stay untouched between _sizes and _fill.
 * _sizes writes d_group_indptr (ceil(n/t) + 1 entries, a device array), synchronises the stream
 * and returns the number of groups on the host; _fill writes d_tile_indices (num_groups * g) and
 * d_mask (num_groups * t * g).
 */
size_t stir_condense_device_workspace_bytes(int32_t n, int64_t nnz, int32_t t);
int stir_condense_device_sizes(int32_t n, int64_t nnz, const int32_t* d_indptr,
                               const int32_t* d_indices, int32_t t, int32_t g, void* d_workspace,
                               int32_t* d_group_indptr, int64_t* num_groups, void* stream);
int stir_condense_device_fill(int32_t n, int64_t nnz, const int32_t* d_indptr,
                              const int32_t* d_indices, int32_t t, int32_t g, void* d_workspace,
                              const int32_t* d_group_indptr, int64_t num_groups,
                              int32_t* d_tile_indices, int32_t* d_mask, void* stream);

/*
 * CSR -> BSR packing on the GPU (blk x blk blocks; m and n multiples of blk): the canonical BSR
 * arrays that scipy's csr_matrix.tobsr hands the reference's example
 * (examples/blocksparse/bsr_spmm.py:441-445) -- block columns ascending in each block row,
 * absent entries of a stored block zero.  The CSR input must hold no duplicate entries.
 * _sizes fills d_bsr_indptr (m/blk + 1) and *nnzb (host; synchronises the stream); _fill writes
 * d_bsr_indices (nnzb) and d_bsr_data (nnzb*blk*blk of data_dtype: STIR_F32, STIR_F16 or
 * STIR_BF16, converted from the fp32 values with round-to-nearest-even).  d_workspace holds
 * stir_csr_to_bsr_workspace_bytes(...) bytes and must stay untouched between the two calls.
 */
size_t stir_csr_to_bsr_workspace_bytes(int32_t m, int32_t n, int32_t blk);
int stir_csr_to_bsr_sizes(int32_t m, int32_t n, int32_t blk, const int32_t* d_indptr,
                          const int32_t* d_indices, void* d_workspace, int32_t* d_bsr_indptr,
                          int64_t* nnzb, void* stream);
int stir_csr_to_bsr_fill(int32_t m, int32_t n, int32_t blk, const int32_t* d_indptr,
                         const int32_t* d_indices, const float* d_values, void* d_workspace,
                         const int32_t* d_bsr_indptr, int32_t* d_bsr_indices, void* d_bsr_data,
                         int32_t data_dtype, int64_t nnzb, void* stream);

/* ------------------------------------------------------------------------------ kernels */

/*
 * CSR row-split SpMM fp32, C[i,:] = sum_p A[p] * B[indices[p],:].
 * Argument list of the reference's built operator: [A, B, C, indptr, indices]
 * (examples/spmm/bench_spmm_naive.py:121-129; lowered form
 * tests/python/sparsetir/sparse_tir_lowered_buffer_scripts.py:22-70).  Rows without
 * nonzeros are written as zeros (the GPU schedule's init block, bench_spmm_naive.py:113).
 */
int stir_csr_spmm_f32(int32_t m, int32_t n, int32_t feat, int64_t nnz, const float* d_A,
                      const float* d_B, float* d_C, const int32_t* d_indptr,
                      const int32_t* d_indices, void* stream);

/*
 * hyb SpMM fp32: all ELL buckets of all column partitions in one launch.
 * The reference specialises and builds one fused kernel per (graph, bucket list)
 * (examples/spmm/bench_spmm.py:116-199); the plan is that built object.  Bucket k =
 * part*num_buckets + bucket has width bucket_widths[bucket], nrows[k] ELL rows and the
 * device arrays d_A[k] (nrows*width f32), d_rows[k] (nrows), d_cols[k] (nrows*width), the
 * (A_k, rows_k, cols_k) triples of the reference's argument list (bench_spmm.py:208-222).
 * A bucket is added to C when num_col_parts > 1 or it is the last bucket of its partition,
 * and stored otherwise (bench_spmm.py:170).  Adding is done with atomics, except that with 2 to
 * 4 partitions the partitions run one after the other on the stream and only the last bucket of
 * each needs atomics -- provided that inside every partition an output row is fed either by one
 * ELL row of one bucket other than the last, or by ELL rows of the last bucket only, as in
 * ColumnPartHyb output.  stir_hyb_plan_create tests this on the row arrays as they are when it is
 * called (it synchronises the device and reads them once) and keeps atomics for every bucket when
 * it does not hold; row ids outside [0, m) are an error.  A caller that rewrites the row arrays
 * of a plan with 2 to 4 partitions must make a new plan.  With more than 4 partitions the plan
 * lists the slots of every output row once (column ids copied, values read through their
 * addresses at every call; 12 bytes of device memory per slot, skipped when that is more than a
 * quarter of the free memory) and its launches write every output row once instead of once per
 * partition; a caller that rewrites the row or column arrays of such a plan must make a new one.
 * The plan keeps the pointers of the value arrays, not copies: the arrays must outlive it.
 */
typedef struct stir_hyb_plan stir_hyb_plan;
int stir_hyb_plan_create(stir_hyb_plan** plan, int32_t m, int32_t n, int32_t num_col_parts,
                         int32_t num_buckets, const int32_t* bucket_widths,
                         const int64_t* nrows, const float* const* d_A,
                         const int32_t* const* d_rows, const int32_t* const* d_cols);
/*
 * The same with flags.  STIR_PLAN_ADDRESSES_ONLY: the plan holds the addresses and sizes of the
 * arrays and nothing derived from what they contain -- always one launch with atomics in every
 * adding bucket (the rule of examples/spmm/bench_spmm.py:170), whatever the partition count --
 * so the arrays may be rewritten in place between launches, as with the reference's built
 * operator, which reads them at every call.  It is what the PackedFunc layer uses until the
 * caller promises static index arrays ("sparsetir.static_structure").
 */
#define STIR_PLAN_ADDRESSES_ONLY 1u
int stir_hyb_plan_create_ex(stir_hyb_plan** plan, int32_t m, int32_t n, int32_t num_col_parts,
                            int32_t num_buckets, const int32_t* bucket_widths,
                            const int64_t* nrows, const float* const* d_A,
                            const int32_t* const* d_rows, const int32_t* const* d_cols, uint32_t flags);
int stir_hyb_spmm_f32(const stir_hyb_plan* plan, int32_t feat, const float* d_B, float* d_C,
                      void* stream);
int stir_hyb_plan_destroy(stir_hyb_plan* plan);

/*
 * hyb SpMM fp32 without a plan and without any allocation.  No counterpart in the reference: it
 * is for callers that cannot allocate device memory -- code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  Takes the arguments of stir_hyb_plan_create
 * followed by those of stir_hyb_spmm_f32 and computes what that pair computes; the bucket
 * descriptors that a plan keeps in allocated device memory go, on every call, into a fixed
 * 128 KiB array that the library holds on each GPU it runs on until the process ends.  Limit: at
 * most 1024 buckets with rows (over all partitions); more is an error.  Always one launch of the
 * SpMM kernel (plus one small launch per 32 buckets that writes the descriptors): with several
 * partitions every bucket adds with atomics, as in the reference (examples/spmm/bench_spmm.py:170).
 * Calls on one GPU share that array: calls that overlap in time on one GPU (different streams or
 * threads) race; calls on one stream are ordered and safe.  The first call on a device looks up
 * the array's address (hipGetDevice, hipGetSymbolAddress) and must happen outside a stream
 * capture; later calls may be recorded into a graph -- the descriptors travel inside the recorded
 * fill kernels' arguments, so every replay writes them again before its SpMM kernel reads them.
 */
int stir_hyb_spmm_f32_noalloc(int32_t m, int32_t n, int32_t num_col_parts, int32_t num_buckets,
                              const int32_t* bucket_widths, const int64_t* nrows,
                              const float* const* d_A, const int32_t* const* d_rows,
                              const int32_t* const* d_cols, int32_t feat, const float* d_B,
                              float* d_C, void* stream);

/*
 * SDDMM fp32.  _preproc is the reference's binary-search block: mid[e] = index of the row
 * that owns nonzero e (tests/python/sparsetir/sparse_tir_lowered_buffer_scripts.py:531-551);
 * stir_sddmm_f32 computes C[e] = <A[mid[e],:], B[indices[e],:]> with the reference's
 * argument list [A, B, C, indptr, indices, mid] (examples/sddmm/bench_sddmm.py:170).
 */
int stir_sddmm_preproc(int32_t m, int64_t nnz, const int32_t* d_indptr, int32_t* d_mid,
                       void* stream);
int stir_sddmm_f32(int32_t m, int32_t n, int32_t feat, int64_t nnz, const float* d_A,
                   const float* d_B, float* d_C, const int32_t* d_indptr,
                   const int32_t* d_indices, const int32_t* d_mid, void* stream);
/* The same with every result scaled by its nonzero's value, C[e] = E[e] * <A[mid[e],:], B[indices[e],:]>
 * (the form sampled dense-dense products take on a weighted graph; the reference's operator,
 * examples/sddmm/bench_sddmm.py:32-55, is the E = 1 case). */
int stir_sddmm_scaled_f32(int32_t m, int32_t n, int32_t feat, int64_t nnz, const float* d_A,
                          const float* d_B, float* d_C, const int32_t* d_indptr,
                          const int32_t* d_indices, const int32_t* d_mid, const float* d_edge_values,
                          void* stream);

/*
 * BSR SpMM on MFMA, 16-bit inputs, fp32 accumulation; argument list [A, X, Y, indptr,
 * indices] of examples/blocksparse/bsr_spmm.py:427-432.  A: nnzb*blk*blk, X: nb*blk*feat,
 * Y: mb*blk*feat.  dtype: STIR_F16 or STIR_BF16 for A and X; out_dtype: the same 16-bit
 * type or STIR_F32.  blk: a multiple of 16 (the reference's schedule splits both block axes by 16,
 * bsr_spmm.py:379-380); feat: a multiple of 32.
 */
int stir_bsr_spmm(int32_t dtype, int32_t out_dtype, int32_t mb, int32_t nb, int32_t blk,
                  int32_t feat, int64_t nnzb, const void* d_A, const void* d_X, void* d_Y,
                  const int32_t* d_indptr, const int32_t* d_indices, void* stream);

/*
 * Doubly-compressed BSR ("dbsrmm", examples/blocksparse/bsr_spmm.py:66-102): only nnz_rows block
 * rows are stored; stored block row i is block row d_row_ids[i] of Y (the reference's indices_0;
 * its indptr_0 is [0, nnz_rows]), d_indptr (nnz_rows+1) / d_indices index its blocks.  Block rows
 * of Y that are not stored are left untouched.
 */
int stir_dbsr_spmm(int32_t dtype, int32_t out_dtype, int32_t nnz_rows, int32_t nb, int32_t blk,
                   int32_t feat, int64_t nnzb, const void* d_A, const void* d_X, void* d_Y,
                   const int32_t* d_row_ids, const int32_t* d_indptr, const int32_t* d_indices,
                   void* stream);

/*
 * SpMM over the condensed format of ConDense on MFMA ("TC-SpMM"), fp16 inputs, fp32
 * accumulation; argument list [A, B, C, indptr, indices] of examples/spmm/bench_tc_spmm.py:650-656
 * (operator :538-565).  A: nnzb*t*g (the 0/1 mask of ConDense as fp16, or edge weights),
 * B: dense features, at least max(indices)+1 rows of feat, C: mb*t*feat of out_dtype (STIR_F16
 * as in the reference, or STIR_F32), indptr: group_indptr (mb+1), indices: tile_indices
 * (nnzb*g).  The MFMA path takes tile_size t = 8 or 16 (the two sizes the reference condenses
 * with, examples/spmm/bench_tc_spmm.py:584-585,670: t = mma_m of m8n32k16 / m16n16k16) or 32, and
 * group_size g = 16 (= mma_k).  C is written, not
 * accumulated into; with fp32 output this takes two launches (row tiles with very many groups
 * are cleared, then summed by several workgroups).
 */
int stir_tc_spmm_f16(int32_t out_dtype, int32_t mb, int32_t tile_size, int32_t group_size,
                     int32_t feat, int64_t nnzb, const void* d_A, const void* d_B, void* d_C,
                     const int32_t* d_indptr, const int32_t* d_indices, void* stream);

/*
 * The same operator with a plan made once from the group counts (the reference
 * has no counterpart: its built operator, examples/spmm/bench_tc_spmm.py:650-656, reads nothing
 * ahead of the launch).  stir_tc_plan_create reads d_indptr (mb+1 entries) on `stream`,
 * synchronises it, and lists the row tiles of more than 16 steps (32 gathered rows each), longest
 * first, cut into pieces of at most 128 steps.  stir_tc_spmm_f16_planned then takes the arguments
 * of stir_tc_spmm_f16: the short tiles as there, then one workgroup per
 * piece -- none is started only to find its tile short, and the hub tiles of a power-law graph
 * are spread over many compute units from the start of the launch.  The pieces of a tile leave
 * fp32 partial tiles, and the workgroup that finishes last among them (a counter per tile and
 * feature tile, which it sets back to zero) adds them in piece order and rounds once: no atomics
 * on C, the same bits on every run (the sums are those of stir_tc_spmm_f16 up to the order of
 * the fp32 additions).  The partial tiles and counters live in memory the plan owns, sized by the
 * first launch with a given feat (that launch allocates): launches with one plan must not overlap
 * on the GPU.  The plan describes the contents of d_indptr at its
 * creation; make a new one when they change.  It belongs to the device that was current at
 * its creation, and a launch with another device current is refused.
 */
typedef struct stir_tc_plan stir_tc_plan;
int stir_tc_plan_create(stir_tc_plan** plan, int32_t mb, const int32_t* d_indptr, void* stream);
int stir_tc_spmm_f16_planned(stir_tc_plan* plan, int32_t out_dtype, int32_t mb, int32_t tile_size,
                             int32_t group_size, int32_t feat, int64_t nnzb, const void* d_A, const void* d_B,
                             void* d_C, const int32_t* d_indptr, const int32_t* d_indices, void* stream);
int stir_tc_plan_destroy(stir_tc_plan* plan);

/*
 * RGMS (relational gather-matmul-scatter), fp16 inputs, fp32 accumulation and output,
 * on the ELL3D buckets produced by CSFToELL3D.  Mirrors the built operator of
 * examples/rgms/rgcn/bench_rgcn_tensorcore.py:838-851: W is [R, feat_in, feat_out], X is
 * [n, feat_in], Y (zero-filled by the caller) is [m, feat_out] fp32; per bucket b the
 * arrays d_A[b] (groups*rb*cb fp16 edge weights, the 0/1 mask in the reference), d_rows[b]
 * (groups*rb), d_cols[b] (groups*rb*cb) and d_mids[b] (groups: relation of each group).
 * The plan keeps the array pointers.  From 8192 slots on, the first launch builds an edge index
 * from the three index arrays (they must not change afterwards; the weights may), and the first
 * launch with given feature sizes a work list for them (both allocate and synchronise the
 * stream; later launches do neither).  W is read anew at every launch.  W that does not fit the
 * LDS of a compute unit beside the kernel's tiles (about 130 KB: 65 relations of 32 x 32) is
 * served as up to three ranges of relations, each with an index and a launch of its own.  With
 * more relations than that, with feat_in above 64 or a d_W that is not 16-byte aligned, every
 * launch rewrites a packed copy of W held by the plan; a plan therefore serves one call at a
 * time.
 */
typedef struct stir_rgms_plan stir_rgms_plan;
int stir_rgms_plan_create(stir_rgms_plan** plan, int32_t num_buckets, const int32_t* rows_bkt,
                          const int32_t* cols_bkt, const int64_t* groups,
                          const void* const* d_A, const int32_t* const* d_rows,
                          const int32_t* const* d_cols, const int32_t* const* d_mids);
int stir_rgms_f16(const stir_rgms_plan* plan, int32_t m, int32_t n, int32_t num_rels,
                  int32_t feat_in, int32_t feat_out, const void* d_W, const void* d_X,
                  float* d_Y, void* stream);
/*
 * Optional promise, made before the first launch of a plan: the slot weights d_A[b] keep the
 * values they have at that first launch for as long as the plan lives.  This is how the reference
 * uses the operator -- its A_k is the 0/1 mask of CSFToELL3D, written once
 * (examples/rgms/rgcn/bench_rgcn_tensorcore.py:840-851).  With the promise, plans over 8192 slots
 * or more (and at most 2048 relations) leave slots of weight zero -- the ELL3D padding, 11 % of
 * the slots at 100k nodes / 65 relations / 2M edges -- out of their edge index and keep the
 * weights inside it (8 bytes per edge instead of 16, no weight loads at run time).  Without it
 * (the default) weights are read at every launch and may change between launches.  Fails once the
 * plan has been launched with the other setting.
 */
int stir_rgms_plan_set_static_weights(stir_rgms_plan* plan, int32_t on);
/*
 * The opposite choice, made before the first launch: the plan never builds an edge index, so
 * nothing in it depends on what the index arrays hold and they may be rewritten in place between
 * launches (the reference's built operator reads them at every call,
 * examples/rgms/rgcn/bench_rgcn_tensorcore.py:852).  Every launch is then the kernel of the small
 * inputs at any size: one fp32 atomic per (ELL row, output feature), about four times the run
 * time of the indexed form at 2M edges.  Fails once the plan has built its index.
 */
int stir_rgms_plan_set_addresses_only(stir_rgms_plan* plan, int32_t on);
/*
 * The same with an fp16 Y: the operator of examples/rgms/rgcn/bench_rgcn_tensorcore.py:564-607
 * built with dtype "float16" (its main program builds "float32" only, :893).  d_Y is [m, feat_out]
 * fp16, 4-byte aligned, and is added to.  Sums are kept in fp32 (the reference's WMMA fragments
 * accumulate in fp16); a row tile is rounded to fp16 once when it is written, and the few tiles
 * that are cut between workgroups -- or every ELL row, for plans below 8192 slots -- are added
 * with packed fp16 atomics, rounded once per addition.  Same plans as stir_rgms_f16.
 */
int stir_rgms_f16_out_f16(const stir_rgms_plan* plan, int32_t m, int32_t n, int32_t num_rels,
                          int32_t feat_in, int32_t feat_out, const void* d_W, const void* d_X,
                          void* d_Y, void* stream);
/* The same with bf16 W, X and slot weights (the reference has an fp16 example only). */
int stir_rgms_bf16(const stir_rgms_plan* plan, int32_t m, int32_t n, int32_t num_rels,
                   int32_t feat_in, int32_t feat_out, const void* d_W, const void* d_X,
                   float* d_Y, void* stream);
int stir_rgms_plan_destroy(stir_rgms_plan* plan);

/*
 * RGMS in fp32 on ELL3D buckets: the composable fp32 operator of
 * examples/rgms/rgcn/bench_rgcn_composable.py:186-225 (rgcn_hetero_forward of
 * examples/rgms/rgcn/utils.py:55-87 after format_decompose).  As stir_rgms_f16, except that
 * every array is fp32 and W is [R, feat_out, feat_in].  feat_in: a multiple of 4, at most 128;
 * W and X 16-byte aligned.  Y is accumulated into with one fp32 atomic per (ELL row, output
 * feature); the plan holds the addresses and sizes of the arrays and nothing derived from their
 * contents.
 */
typedef struct stir_rgms_f32_plan stir_rgms_f32_plan;
int stir_rgms_f32_plan_create(stir_rgms_f32_plan** plan, int32_t num_buckets, const int32_t* rows_bkt,
                              const int32_t* cols_bkt, const int64_t* groups,
                              const float* const* d_A, const int32_t* const* d_rows,
                              const int32_t* const* d_cols, const int32_t* const* d_mids);
int stir_rgms_f32(const stir_rgms_f32_plan* plan, int32_t m, int32_t n, int32_t num_rels,
                  int32_t feat_in, int32_t feat_out, const float* d_W, const float* d_X,
                  float* d_Y, void* stream);
/*
 * Optional (no counterpart in the reference): sums that come out the same, bit for bit, on every
 * run, and faster.  From 8192 slots on, with feat_in and feat_out of at most 64, the first launch
 * of a plan switched to this mode builds an edge index from the three index arrays (sorted by
 * 64-row tile of Y, relation, row; it allocates and synchronises the stream, later launches only
 * rewrite a packed copy of W held by the plan; the index arrays must not change afterwards, the
 * weights may) and every tile of Y is summed on chip in a fixed order and written once, without
 * atomics: 134 us against 159 us on 100k nodes, 65 relations, 2M edges.  Inputs outside these
 * limits, or whose index would not fit its 64-bit sort keys, run the atomic kernels.
 * A plan in this mode serves one call at a time.
 */
int stir_rgms_f32_plan_set_deterministic(stir_rgms_f32_plan* plan, int32_t on);
int stir_rgms_f32_plan_destroy(stir_rgms_f32_plan* plan);

/*
 * RGMS in fp32 straight from the CSF arrays (relation -> stored row -> column): the
 * non-composable operator of examples/rgms/rgcn/bench_rgcn_non_composable.py:82-112, argument
 * list [A, W, X, Y, indptr_i, indices_i, indptr_j, indices_j] (:109).  A: nnz_j edge values,
 * W: [R, feat_out, feat_in], X: [n, feat_in], Y: [m, feat_out] zero-filled by the caller and
 * accumulated into with atomics (the schedule's atomic write-back, :89-90), indptr_i: R+1,
 * indices_i: nnz_i output rows, indptr_j: nnz_i+1, indices_j: nnz_j.
 */
int stir_rgms_csf_f32(int32_t m, int32_t n, int32_t num_rels, int32_t feat_in, int32_t feat_out,
                      int64_t nnz_i, int64_t nnz_j, const float* d_A, const float* d_W,
                      const float* d_X, float* d_Y, const int32_t* d_indptr_i,
                      const int32_t* d_indices_i, const int32_t* d_indptr_j,
                      const int32_t* d_indices_j, void* stream);

/*
 * The same operator without atomics (no counterpart in the reference): sums that come out the
 * same, bit for bit, on every run, and faster than stir_rgms_csf_f32 (122 against 159 us on 100k
 * nodes, 65 relations, 2M edges).  The plan keeps the pointers of the five arrays; from 8192 edges
 * on, with feat_in and feat_out of at most 64, its first launch builds the edge index described
 * at stir_rgms_f32_plan_set_deterministic from the four index arrays (they must not change
 * afterwards, the edge values may) and every 64-row tile of Y is written once.  Other inputs run
 * stir_rgms_csf_f32.  A plan serves one call at a time.
 */
typedef struct stir_rgms_csf_f32_plan stir_rgms_csf_f32_plan;
int stir_rgms_csf_f32_plan_create(stir_rgms_csf_f32_plan** plan, int64_t nnz_i, int64_t nnz_j, const float* d_A,
                                  const int32_t* d_indptr_i, const int32_t* d_indices_i,
                                  const int32_t* d_indptr_j, const int32_t* d_indices_j);
int stir_rgms_csf_f32_planned(stir_rgms_csf_f32_plan* plan, int32_t m, int32_t n, int32_t num_rels,
                              int32_t feat_in, int32_t feat_out, const float* d_W, const float* d_X,
                              float* d_Y, void* stream);
int stir_rgms_csf_f32_plan_destroy(stir_rgms_csf_f32_plan* plan);

#ifdef __cplusplus
}
#endif
#endif /* SPARSETIR_AMD_H_ */
