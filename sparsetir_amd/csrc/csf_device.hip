// CSFToELL3D on the GPU, bit-exact with the host routine (csrc/format_host.cpp) and the
// reference's sequential append loop (src/sparse/format.cc:180-343), which runs on the CPU only.
//
// The sequential rule -- a stored row of a relation goes to the bucket that fits its number of
// columns, opens an ELL row and another one every time the row is full -- has a closed form when
// the row ids of a relation ascend strictly (no two stored rows of a relation share an id, so no
// ELL row is shared): stored row i with c columns in bucket b takes ceil(c / width_b) ELL rows,
// starting after those of the earlier stored rows of its relation in the same bucket.  Passes:
//   classify   per stored row: relation, bucket; validation of the four CSF arrays
//   scan       per bucket: exclusive sum of the ELL rows over all stored rows (hipCUB)
//   groups     per bucket: ELL rows per relation -> whole groups -> group offsets (the output indptr)
//   base       per stored row: its first ELL row inside the bucket's arrays
//   entries    per nonzero: column, mask and (first slot of an ELL row) the row id
//   pad        per (bucket, relation): the last row id repeated up to the end of the last group
#include <hipcub/hipcub.hpp>

#include <algorithm>
#include <vector>

#include "common.h"
#include "row_lookup.h"
#include "../../include/sparsetir_amd.h"

namespace {

using stir::ceil_div;
using stir::kWave;

constexpr int kMaxBuckets = 32;

struct Buckets {
  int32_t nb;
  int32_t rb[kMaxBuckets], cb[kMaxBuckets];
};

struct Outputs {
  int32_t* rows[kMaxBuckets];
  int32_t* cols[kMaxBuckets];
  int32_t* mask[kMaxBuckets];
};

// the bucket of a stored row with cnt columns: the first whose width holds them, else the last
// (format.cc:244-249: upper_bound over the widths at cnt - 1)
__device__ __forceinline__ int bucket_of(const Buckets& B, int cnt) {
  int b = 0;
  while (b + 1 < B.nb && B.cb[b] < cnt) ++b;
  return b;
}

enum Flag { kBadEnds = 1, kBadIndptr0 = 2, kBadIndptr1 = 4, kRowOrder = 8, kTooLarge = 16 };

// What the workspace holds, in this order (see layout()).
struct Workspace {
  int32_t* flags;     // [16]
  int64_t* totals;    // [nb] groups per bucket
  int32_t* rel_of;    // [rows] relation of a stored row
  int32_t* base;      // [rows] first ELL row of a stored row inside its bucket's arrays
  int32_t* pre;       // [nb][rows + 1] exclusive sum of ELL rows, per bucket
  int32_t* gptr;      // [nb][rels + 1] group offsets
  uint8_t* bkt;       // [rows] bucket of a stored row
  void* scan_tmp;
  size_t scan_bytes;
  size_t total_bytes;
};

struct EllRowsOfBucket {
  const int32_t* indptr1;
  const uint8_t* bkt;
  int64_t rows;
  int32_t bucket, width;
  __host__ __device__ int32_t operator()(int64_t i) const {
    if (i >= rows || bkt[i] != bucket) return 0;
    const int32_t cnt = indptr1[i + 1] - indptr1[i];
    return cnt <= 0 ? 0 : (cnt + width - 1) / width;
  }
};
using EllRowsIter = hipcub::TransformInputIterator<int32_t, EllRowsOfBucket, hipcub::CountingInputIterator<int64_t>>;

size_t scan_temp_bytes(int64_t rows) {
  size_t bytes = 0;
  EllRowsIter it(hipcub::CountingInputIterator<int64_t>(0), EllRowsOfBucket{nullptr, nullptr, 0, 0, 1});
  (void)hipcub::DeviceScan::ExclusiveSum(nullptr, bytes, it, (int32_t*)nullptr, (int)(rows + 1), (hipStream_t) nullptr);
  return bytes;
}

Workspace layout(void* d_ws, int32_t rels, int64_t rows, int32_t nb) {
  Workspace w{};
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char* p = d_ws ? static_cast<char*>(d_ws) + off : nullptr;
    off += (bytes + 255) / 256 * 256;
    return p;
  };
  w.flags = reinterpret_cast<int32_t*>(take(16 * sizeof(int32_t)));
  w.totals = reinterpret_cast<int64_t*>(take(sizeof(int64_t) * nb));
  w.rel_of = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * size_t(rows)));
  w.base = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * size_t(rows)));
  w.pre = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * size_t(nb) * size_t(rows + 1)));
  w.gptr = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * size_t(nb) * size_t(rels + 1)));
  w.bkt = reinterpret_cast<uint8_t*>(take(size_t(rows)));
  w.scan_bytes = scan_temp_bytes(rows);
  w.scan_tmp = take(w.scan_bytes);
  w.total_bytes = off;
  return w;
}

__device__ __forceinline__ int64_t clamp_row(int64_t v, int64_t rows) { return v < 0 ? 0 : (v > rows ? rows : v); }

__global__ __launch_bounds__(256) void csf_classify_kernel(int rels, int64_t rows, int64_t nnz,
                                                           const int32_t* __restrict__ p0,
                                                           const int32_t* __restrict__ i0,
                                                           const int32_t* __restrict__ p1, Buckets B,
                                                           uint8_t* __restrict__ bkt, int32_t* __restrict__ rel_of,
                                                           int32_t* __restrict__ flags) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int bad = 0;
  if (i == 0 && (p0[0] != 0 || p0[rels] != rows || p1[0] != 0 || p1[rows] != nnz)) bad |= kBadEnds;
  if (i < rels && p0[i] > p0[i + 1]) bad |= kBadIndptr0;
  if (i < rows) {
    const int32_t a = p1[i], b = p1[i + 1];
    if (a > b) bad |= kBadIndptr1;
    bkt[i] = (uint8_t)bucket_of(B, b - a);
    // the relation that holds stored row i: the last r with p0[r] <= i
    int lo = 0, hi = rels - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (p0[mid] <= i) lo = mid; else hi = mid - 1;
    }
    rel_of[i] = lo;
    if (i > 0 && i > p0[lo] && i0[i - 1] >= i0[i]) bad |= kRowOrder;  // i > 0: indptr0 may hold anything yet
  }
  if (bad) atomicOr(flags, bad);
}

// One workgroup per bucket: ELL rows per relation -> groups -> offsets.
__global__ __launch_bounds__(256) void csf_groups_kernel(int rels, int64_t rows, const int32_t* __restrict__ p0,
                                                         Buckets B, const int32_t* __restrict__ pre,
                                                         int32_t* __restrict__ gptr, int64_t* __restrict__ totals,
                                                         int32_t* __restrict__ flags) {
  using Scan = hipcub::BlockScan<int64_t, 256>;
  __shared__ typename Scan::TempStorage tmp;
  const int b = blockIdx.x;
  const int32_t* pb = pre + (int64_t)b * (rows + 1);
  int32_t* gb = gptr + (int64_t)b * (rels + 1);
  int64_t carry = 0;
  for (int r0 = 0; r0 < rels; r0 += 256) {
    const int r = r0 + threadIdx.x;
    int64_t g = 0;
    if (r < rels) {
      const int64_t ell = pb[clamp_row(p0[r + 1], rows)] - pb[clamp_row(p0[r], rows)];
      g = ell > 0 ? (ell + B.rb[b] - 1) / B.rb[b] : 0;
    }
    int64_t before, sum;
    Scan(tmp).ExclusiveSum(g, before, sum);
    __syncthreads();
    if (r < rels) gb[r] = (int32_t)(carry + before);
    carry += sum;
  }
  if (threadIdx.x == 0) {
    gb[rels] = (int32_t)carry;
    totals[b] = carry;
    if (carry * B.rb[b] >= (int64_t(1) << 31)) atomicOr(flags, (int)kTooLarge);
  }
}

__global__ __launch_bounds__(256) void csf_base_kernel(int rels, int64_t rows, const int32_t* __restrict__ p0,
                                                       Buckets B, const uint8_t* __restrict__ bkt,
                                                       const int32_t* __restrict__ rel_of,
                                                       const int32_t* __restrict__ pre,
                                                       const int32_t* __restrict__ gptr,
                                                       int32_t* __restrict__ base) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows) return;
  const int b = bkt[i], r = rel_of[i];
  const int32_t* pb = pre + (int64_t)b * (rows + 1);
  base[i] = (int32_t)((int64_t)gptr[(int64_t)b * (rels + 1) + r] * B.rb[b] + pb[i] - pb[clamp_row(p0[r], rows)]);
}

// Arrays of one kind (columns or masks) cleared together: blockIdx.y picks the array.
struct ZeroJobs {
  int32_t* ptr[2 * kMaxBuckets];
  int64_t count[2 * kMaxBuckets];
};
__global__ __launch_bounds__(256) void csf_zero_kernel(ZeroJobs jobs) {
  int32_t* p = jobs.ptr[blockIdx.y];
  const int64_t n = jobs.count[blockIdx.y];
  for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < n; q += (int64_t)gridDim.x * 256) p[q] = 0;
}

constexpr int kEntriesPer = 8;  // nonzeros per lane: a wavefront takes 512 consecutive ones
__global__ __launch_bounds__(256) void csf_entries_kernel(int64_t rows, int64_t nnz, const int32_t* __restrict__ i0,
                                                          const int32_t* __restrict__ p1,
                                                          const int32_t* __restrict__ i1, Buckets B,
                                                          const uint8_t* __restrict__ bkt,
                                                          const int32_t* __restrict__ base, Outputs out) {
  __shared__ int32_t win[4][stir::kRowLookupWindow];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t e0 = ((int64_t)blockIdx.x * 4 + wave) * (kEntriesPer * kWave);
  if (e0 >= nnz) return;
  const int64_t e_last = min(e0 + kEntriesPer * kWave, nnz) - 1;
  stir::for_each_nonzero_row<kEntriesPer>(p1, (int)rows, e0, e_last, win[wave], lane,
                                          [&](int64_t e, int i, int, bool live) {
    if (!live) return;
    const int b = bkt[i];
    const int width = B.cb[b];
    const int t = (int)(e - p1[i]);
    const int64_t ell_row = (int64_t)base[i] + t / width;
    const int slot = t % width;
    const int64_t pos = ell_row * width + slot;
    out.cols[b][pos] = i1[e];
    out.mask[b][pos] = 1;
    if (slot == 0) out.rows[b][ell_row] = i0[i];
  });
}

__global__ __launch_bounds__(256) void csf_pad_kernel(int rels, int64_t rows, const int32_t* __restrict__ p0,
                                                      Buckets B, const int32_t* __restrict__ pre,
                                                      const int32_t* __restrict__ gptr, Outputs out) {
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)B.nb * rels) return;
  const int b = (int)(id / rels), r = (int)(id % rels);
  const int32_t* pb = pre + (int64_t)b * (rows + 1);
  const int64_t ell = pb[clamp_row(p0[r + 1], rows)] - pb[clamp_row(p0[r], rows)];
  if (ell <= 0) return;
  const int32_t* gb = gptr + (int64_t)b * (rels + 1);
  const int64_t first = (int64_t)gb[r] * B.rb[b], end = (int64_t)gb[r + 1] * B.rb[b];
  const int32_t last = out.rows[b][first + ell - 1];
  for (int64_t q = first + ell; q < end; ++q) out.rows[b][q] = last;
}

int check_args(const char* who, int32_t rels, int64_t rows, int64_t nnz, const void* p0, const void* i0,
               const void* p1, const void* i1, const int32_t* rows_bkt, const int32_t* cols_bkt, int32_t nb,
               const void* ws, Buckets& B) {
  STIR_REQUIRE(rels >= 0 && rows >= 0 && nnz >= 0 && p0 && p1, "%s: bad CSF arguments", who);
  STIR_REQUIRE(rows == 0 || i0, "%s: csf_indices_0 is null", who);
  STIR_REQUIRE(nnz == 0 || i1, "%s: csf_indices_1 is null", who);
  STIR_REQUIRE(rows < (int64_t(1) << 31) - 1 && nnz < (int64_t(1) << 31), "%s: more than 2^31 stored rows or nonzeros", who);
  STIR_REQUIRE(nb > 0 && rows_bkt && cols_bkt, "%s: empty bucket list", who);
  STIR_REQUIRE(nb <= kMaxBuckets, "%s: at most %d buckets on the device", who, kMaxBuckets);
  for (int b = 0; b < nb; ++b)
    STIR_REQUIRE(rows_bkt[b] > 0 && cols_bkt[b] > 0, "%s: bucket sizes must be positive", who);
  for (int b = 1; b < nb; ++b)
    STIR_REQUIRE(cols_bkt[b - 1] < cols_bkt[b], "%s: The given nnz_cols_bkt should be ascending.", who);
  STIR_REQUIRE(ws, "%s: workspace is null", who);
  B.nb = nb;
  for (int b = 0; b < nb; ++b) B.rb[b] = rows_bkt[b], B.cb[b] = cols_bkt[b];
  return 0;
}

}  // namespace

extern "C" {

size_t stir_csf_to_ell3d_device_workspace_bytes(int32_t num_rels, int64_t num_stored_rows, int32_t num_buckets) {
  if (num_rels < 0 || num_stored_rows < 0 || num_buckets <= 0) return 0;
  return layout(nullptr, num_rels, num_stored_rows, num_buckets).total_bytes;
}

int stir_csf_to_ell3d_device_sizes(int32_t num_rels, int64_t num_stored_rows, int64_t nnz,
                                   const int32_t* d_indptr0, const int32_t* d_indices0,
                                   const int32_t* d_indptr1, const int32_t* d_indices1,
                                   const int32_t* rows_bkt, const int32_t* cols_bkt, int32_t num_buckets,
                                   void* d_workspace, int64_t* groups, void* stream) {
  const char* who = "CSFToELL3D(device)";
  Buckets B{};
  if (check_args(who, num_rels, num_stored_rows, nnz, d_indptr0, d_indices0, d_indptr1, d_indices1, rows_bkt,
                 cols_bkt, num_buckets, d_workspace, B))
    return -1;
  STIR_REQUIRE(groups, "%s: groups is null", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int nb = num_buckets;
  const int64_t rows = num_stored_rows;
  Workspace w = layout(d_workspace, num_rels, rows, nb);
  if (num_rels == 0) {
    STIR_REQUIRE(rows == 0 && nnz == 0, "%s: stored rows without a relation", who);
    std::fill(groups, groups + nb, int64_t(0));
    STIR_HIP(hipMemsetAsync(w.totals, 0, sizeof(int64_t) * nb, st));
    STIR_HIP(hipMemsetAsync(w.gptr, 0, sizeof(int32_t) * size_t(nb), st));
    STIR_HIP(hipStreamSynchronize(st));
    return 0;
  }
  STIR_HIP(hipMemsetAsync(w.flags, 0, 16 * sizeof(int32_t), st));
  const int64_t items = std::max<int64_t>(rows, num_rels) + 1;
  hipLaunchKernelGGL(csf_classify_kernel, dim3((unsigned)ceil_div(items, 256)), dim3(256), 0, st, num_rels, rows, nnz,
                     d_indptr0, d_indices0, d_indptr1, B, w.bkt, w.rel_of, w.flags);
  STIR_LAUNCH_CHECK();
  // the scans read indptr1 through the bucket of every stored row: stop here when the arrays are bad
  int32_t h_flags = 0;
  STIR_HIP(hipMemcpyAsync(&h_flags, w.flags, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipStreamSynchronize(st));
  STIR_REQUIRE(!(h_flags & kBadEnds),
               "%s: the CSF arrays do not fit each other (indptr0 must run from 0 to the number of stored rows, "
               "indptr1 from 0 to the number of nonzeros)", who);
  STIR_REQUIRE(!(h_flags & kBadIndptr0), "%s: indptr0 decreases", who);
  STIR_REQUIRE(!(h_flags & kBadIndptr1), "%s: indptr1 decreases", who);
  STIR_REQUIRE(!(h_flags & kRowOrder),
               "%s: the row ids of a relation must ascend strictly on the device (the host routine takes any order)",
               who);
  for (int b = 0; b < nb; ++b) {
    EllRowsIter it(hipcub::CountingInputIterator<int64_t>(0), EllRowsOfBucket{d_indptr1, w.bkt, rows, b, B.cb[b]});
    size_t bytes = w.scan_bytes;
    STIR_HIP(hipcub::DeviceScan::ExclusiveSum(w.scan_tmp, bytes, it, w.pre + (int64_t)b * (rows + 1), (int)(rows + 1),
                                              st));
  }
  hipLaunchKernelGGL(csf_groups_kernel, dim3((unsigned)nb), dim3(256), 0, st, num_rels, rows, d_indptr0, B, w.pre,
                     w.gptr, w.totals, w.flags);
  STIR_LAUNCH_CHECK();
  if (rows > 0) {
    hipLaunchKernelGGL(csf_base_kernel, dim3((unsigned)ceil_div(rows, 256)), dim3(256), 0, st, num_rels, rows,
                       d_indptr0, B, w.bkt, w.rel_of, w.pre, w.gptr, w.base);
    STIR_LAUNCH_CHECK();
  }
  STIR_HIP(hipMemcpyAsync(&h_flags, w.flags, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipMemcpyAsync(groups, w.totals, sizeof(int64_t) * nb, hipMemcpyDeviceToHost, st));
  STIR_HIP(hipStreamSynchronize(st));
  STIR_REQUIRE(!(h_flags & kTooLarge), "%s: a bucket needs 2^31 ELL rows or more", who);
  return 0;
}

int stir_csf_to_ell3d_device_fill(int32_t num_rels, int64_t num_stored_rows, int64_t nnz,
                                  const int32_t* d_indptr0, const int32_t* d_indices0,
                                  const int32_t* d_indptr1, const int32_t* d_indices1,
                                  const int32_t* rows_bkt, const int32_t* cols_bkt, int32_t num_buckets,
                                  void* d_workspace, const int64_t* groups, int32_t* const* d_indptr,
                                  int32_t* const* d_row_indices, int32_t* const* d_col_indices,
                                  int32_t* const* d_mask, void* stream) {
  const char* who = "CSFToELL3D(device)";
  Buckets B{};
  if (check_args(who, num_rels, num_stored_rows, nnz, d_indptr0, d_indices0, d_indptr1, d_indices1, rows_bkt,
                 cols_bkt, num_buckets, d_workspace, B))
    return -1;
  STIR_REQUIRE(groups && d_indptr && d_row_indices && d_col_indices && d_mask, "%s: null output table", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int nb = num_buckets;
  const int64_t rows = num_stored_rows;
  Workspace w = layout(d_workspace, num_rels, rows, nb);
  Outputs out{};
  ZeroJobs jobs{};
  int64_t most = 0;
  for (int b = 0; b < nb; ++b) {
    STIR_REQUIRE(groups[b] >= 0 && d_indptr[b], "%s: bad output for bucket %d", who, b);
    STIR_REQUIRE(groups[b] == 0 || (d_row_indices[b] && d_col_indices[b] && d_mask[b]),
                 "%s: null output array for bucket %d", who, b);
    out.rows[b] = d_row_indices[b], out.cols[b] = d_col_indices[b], out.mask[b] = d_mask[b];
    const int64_t slots = groups[b] * B.rb[b] * B.cb[b];
    jobs.ptr[2 * b] = d_col_indices[b], jobs.ptr[2 * b + 1] = d_mask[b];
    jobs.count[2 * b] = jobs.count[2 * b + 1] = slots;
    most = std::max(most, slots);
    STIR_HIP(hipMemcpyAsync(d_indptr[b], w.gptr + (int64_t)b * (num_rels + 1), sizeof(int32_t) * size_t(num_rels + 1),
                            hipMemcpyDeviceToDevice, st));
  }
  if (most > 0) {
    const unsigned gx = (unsigned)std::min<int64_t>(ceil_div(most, 256), 4096);
    hipLaunchKernelGGL(csf_zero_kernel, dim3(gx, (unsigned)(2 * nb)), dim3(256), 0, st, jobs);
    STIR_LAUNCH_CHECK();
  }
  if (nnz > 0) {
    hipLaunchKernelGGL(csf_entries_kernel, dim3((unsigned)ceil_div(nnz, 4 * kEntriesPer * kWave)), dim3(256), 0, st,
                       rows, nnz, d_indices0, d_indptr1, d_indices1, B, w.bkt, w.base, out);
    STIR_LAUNCH_CHECK();
    hipLaunchKernelGGL(csf_pad_kernel, dim3((unsigned)ceil_div((int64_t)nb * num_rels, 256)), dim3(256), 0, st,
                       num_rels, rows, d_indptr0, B, w.pre, w.gptr, out);
    STIR_LAUNCH_CHECK();
  }
  return 0;
}

}  // extern "C"
