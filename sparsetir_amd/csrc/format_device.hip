// ColumnPartHyb on the GPU, bit-exact with the sequential host routine.
//
// The reference's append loop (src/sparse/format.cc:86-139) is order dependent, but for CSR
// rows with ascending columns its result has a closed form: the entries of row i that fall in
// column partition p are one contiguous run [lo, hi) of the row; with d = hi - lo the run goes
// to bucket beta = first width >= d (else the last), occupies rho = ceil(d / width) consecutive
// ELL rows, and starts at ELL row base(i, p) = sum of rho over earlier rows of the same
// (p, beta).  Entry number t of the run lands at flat slot base * width + t; the slots from d
// to rho * width are padding (col 0, mask 0); each of the rho ELL rows carries row id i.
//
// Passes: (0) validate (columns in range, ascending inside rows); (1) per (row, partition)
// binary-search lo and build a per-wavefront histogram of rho per bucket; (2) exclusive scan of
// the histograms along the rows for every (partition, bucket), which also yields the ELL row
// counts; (3) per (row, partition) compute base from the scanned histogram plus the rank inside
// the wavefront, write row ids and padding; (4) per nonzero, scatter the column id and mask.
#include <cstring>
#include <vector>

#include "common.h"
#include "../../include/sparsetir_amd.h"

namespace {

using stir::kWave;

struct Workspace {
  int32_t* lo;       // [P][m]   start of the (row, partition) run inside indices
  int32_t* base;     // [P][m]   first ELL row of the run inside its bucket
  int32_t* hist;     // [P][W][NB] per-wavefront ELL-row counts, scanned in place
  int64_t* totals;   // [P][NB]
  int32_t* widths;   // [NB]
  int32_t* status;   // [1] nonzero: input rejected
  int32_t** rows_tab;  // [P*NB] output pointers
  int32_t** cols_tab;
  int32_t** mask_tab;
  size_t bytes;
};

size_t align_up(size_t x) { return (x + 255) & ~size_t(255); }

Workspace carve(void* p, int32_t m, int32_t P, int32_t NB) {
  Workspace w;
  const int64_t W = stir::ceil_div(m, kWave);
  char* c = static_cast<char*>(p);
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char* r = c ? c + off : nullptr;
    off += align_up(bytes);
    return r;
  };
  w.lo = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * size_t(P) * size_t(m > 0 ? m : 1)));
  w.base = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * size_t(P) * size_t(m > 0 ? m : 1)));
  w.hist = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * size_t(P) * size_t(W > 0 ? W : 1) * NB));
  w.totals = reinterpret_cast<int64_t*>(take(sizeof(int64_t) * size_t(P) * NB));
  w.widths = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * NB));
  w.status = reinterpret_cast<int32_t*>(take(sizeof(int32_t)));
  w.rows_tab = reinterpret_cast<int32_t**>(take(sizeof(void*) * size_t(P) * NB));
  w.cols_tab = reinterpret_cast<int32_t**>(take(sizeof(void*) * size_t(P) * NB));
  w.mask_tab = reinterpret_cast<int32_t**>(take(sizeof(void*) * size_t(P) * NB));
  w.bytes = off;
  return w;
}

enum { kStatusRange = 1, kStatusUnsorted = 2 };

__device__ __forceinline__ int lower_bound_dev(const int32_t* a, int lo, int hi, int64_t key) {
  while (lo < hi) {
    const int mid = lo + ((hi - lo) >> 1);
    if ((int64_t)a[mid] < key) lo = mid + 1; else hi = mid;
  }
  return lo;
}

__device__ __forceinline__ int bucket_of_dev(const int32_t* widths, int nb, int d) {
  int k = 0;
  while (k < nb - 1 && widths[k] < d) ++k;  // first width >= d, else the last bucket
  return k;
}

// (0) every column inside [0, num_cols); columns ascend inside each row
__global__ __launch_bounds__(256) void validate_kernel(int m, int num_cols, int64_t nnz, int32_t first,
                                                       const int32_t* __restrict__ indptr,
                                                       const int32_t* __restrict__ indices,
                                                       int32_t* __restrict__ status) {
  const int64_t e = first + (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= first + nnz) return;
  const int col = indices[e];
  if (col < 0 || col >= num_cols) {
    atomicOr(status, kStatusRange);
    return;
  }
  if (e + 1 < first + nnz && indices[e + 1] < col) {
    // legal only when e+1 opens a row: some indptr entry equals e+1
    const int r = lower_bound_dev(indptr, 0, m + 1, e + 1);
    if (r > m || (int64_t)indptr[r] != e + 1) atomicOr(status, kStatusUnsorted);
  }
}

// (1) lo per (row, partition) and per-wavefront histogram.  grid (ceil(m/256), P).
__global__ __launch_bounds__(256) void count_kernel(int m, int psize, int NB, int64_t W,
                                                    const int32_t* __restrict__ indptr,
                                                    const int32_t* __restrict__ indices,
                                                    const int32_t* __restrict__ widths,
                                                    int32_t* __restrict__ lo_out, int32_t* __restrict__ hist) {
  const int p = blockIdx.y;
  const int P = gridDim.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  int d = 0;
  if (i < m) {
    const int rs = indptr[i], re = indptr[i + 1];
    const int lo = p == 0 ? rs : lower_bound_dev(indices, rs, re, (int64_t)p * psize);
    const int hi = p == P - 1 ? re : lower_bound_dev(indices, lo, re, (int64_t)(p + 1) * psize);
    lo_out[(int64_t)p * m + i] = lo;
    d = hi - lo;
  }
  if (wave >= W) return;
  const int beta = bucket_of_dev(widths, NB, d);
  const int w = widths[beta];
  const int rho = d == 0 ? 0 : (d + w - 1) / w;
  int32_t* h = hist + ((int64_t)p * W + wave) * NB;
  for (int b = 0; b < NB - 1; ++b) {
    const unsigned long long bal = __ballot(d > 0 && beta == b);
    if (lane == 0) h[b] = __popcll(bal);
  }
  int tot = beta == NB - 1 ? rho : 0;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) tot += __shfl_xor(tot, off, kWave);
  if (lane == 0) h[NB - 1] = tot;
}

// (2) exclusive scan of hist[p][.][b] along the wavefront axis.  grid (NB, P), 256 threads.
__global__ __launch_bounds__(256) void scan_kernel(int NB, int64_t W, int32_t* __restrict__ hist,
                                                   int64_t* __restrict__ totals) {
  __shared__ int64_t part[256];
  const int b = blockIdx.x, p = blockIdx.y;
  int32_t* h = hist + (int64_t)p * W * NB + b;
  const int64_t chunk = (W + 255) / 256;
  const int64_t w0 = chunk * threadIdx.x, w1 = min(W, w0 + chunk);
  int64_t sum = 0;
  for (int64_t w = w0; w < w1; ++w) sum += h[w * NB];
  part[threadIdx.x] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    int64_t run = 0;
    for (int t = 0; t < 256; ++t) {
      const int64_t v = part[t];
      part[t] = run;
      run += v;
    }
    totals[(int64_t)p * NB + b] = run;
  }
  __syncthreads();
  int64_t run = part[threadIdx.x];
  for (int64_t w = w0; w < w1; ++w) {
    const int32_t v = h[w * NB];
    h[w * NB] = (int32_t)run;
    run += v;
  }
}

// (3) base per (row, partition); row ids and padding slots.  grid (ceil(m/256), P).
__global__ __launch_bounds__(256) void place_rows_kernel(int m, int NB, int64_t W,
                                                         const int32_t* __restrict__ indptr,
                                                         const int32_t* __restrict__ widths,
                                                         const int32_t* __restrict__ lo_in,
                                                         const int32_t* __restrict__ hist,
                                                         int32_t* __restrict__ base_out,
                                                         int32_t* const* __restrict__ rows_tab,
                                                         int32_t* const* __restrict__ cols_tab,
                                                         int32_t* const* __restrict__ mask_tab) {
  const int p = blockIdx.y;
  const int P = gridDim.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wave >= W) return;
  int d = 0;
  if (i < m) {
    const int lo = lo_in[(int64_t)p * m + i];
    const int hi = p == P - 1 ? indptr[i + 1] : lo_in[(int64_t)(p + 1) * m + i];
    d = hi - lo;
  }
  const int beta = bucket_of_dev(widths, NB, d);
  const int w = widths[beta];
  const int rho = d == 0 ? 0 : (d + w - 1) / w;
  const unsigned long long below = (1ull << lane) - 1ull;
  int rank = 0;
  for (int b = 0; b < NB - 1; ++b) {
    const unsigned long long bal = __ballot(d > 0 && beta == b);
    if (beta == b) rank = __popcll(bal & below);
  }
  // exclusive scan of rho over the lanes that use the last bucket
  int incl = beta == NB - 1 ? rho : 0;
  const int mine = incl;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int up = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += up;
  }
  if (beta == NB - 1) rank = incl - mine;
  if (i >= m || d == 0) return;
  const int64_t base = (int64_t)hist[((int64_t)p * W + wave) * NB + beta] + rank;
  base_out[(int64_t)p * m + i] = (int32_t)base;
  const int k = p * NB + beta;
  int32_t* rows = rows_tab[k];
  for (int j = 0; j < rho; ++j) rows[base + j] = i;
  int32_t* cols = cols_tab[k];
  int32_t* mask = mask_tab[k];
  for (int64_t s = base * w + d; s < (base + rho) * w; ++s) {
    cols[s] = 0;
    mask[s] = 0;
  }
}

// (4) one thread per nonzero: its slot is base * width + (position inside the run).
__global__ __launch_bounds__(256) void place_entries_kernel(int m, int P, int psize, int NB, int64_t nnz,
                                                            int32_t first,
                                                            const int32_t* __restrict__ indptr,
                                                            const int32_t* __restrict__ indices,
                                                            const int32_t* __restrict__ widths,
                                                            const int32_t* __restrict__ lo_in,
                                                            const int32_t* __restrict__ base_in,
                                                            int32_t* const* __restrict__ cols_tab,
                                                            int32_t* const* __restrict__ mask_tab) {
  const int64_t e = first + (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= first + nnz) return;
  const int col = indices[e];
  const int p = col / psize;
  // row that owns e: last r with indptr[r] <= e
  int a = 0, b = m;
  while (a < b) {
    const int mid = a + ((b - a + 1) >> 1);
    if ((int64_t)indptr[mid] <= e) a = mid; else b = mid - 1;
  }
  const int i = a;
  const int lo = lo_in[(int64_t)p * m + i];
  const int hi = p == P - 1 ? indptr[i + 1] : lo_in[(int64_t)(p + 1) * m + i];
  const int d = hi - lo;
  const int beta = bucket_of_dev(widths, NB, d);
  const int64_t pos = (int64_t)base_in[(int64_t)p * m + i] * widths[beta] + (e - lo);
  const int k = p * NB + beta;
  cols_tab[k][pos] = col;
  mask_tab[k][pos] = 1;
}

// Value rewrite: A_k[slot] = values[e] for every nonzero (padding slots stay zero), the
// placement computed exactly as in place_entries_kernel.
__global__ __launch_bounds__(256) void place_values_kernel(int m, int P, int psize, int NB, int64_t nnz,
                                                           int32_t first,
                                                           const int32_t* __restrict__ indptr,
                                                           const int32_t* __restrict__ indices,
                                                           const float* __restrict__ values,
                                                           const int32_t* __restrict__ widths,
                                                           const int32_t* __restrict__ lo_in,
                                                           const int32_t* __restrict__ base_in,
                                                           float* const* __restrict__ a_tab) {
  const int64_t e = first + (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= first + nnz) return;
  const int col = indices[e];
  const int p = col / psize;
  int a = 0, b = m;
  while (a < b) {
    const int mid = a + ((b - a + 1) >> 1);
    if ((int64_t)indptr[mid] <= e) a = mid; else b = mid - 1;
  }
  const int i = a;
  const int lo = lo_in[(int64_t)p * m + i];
  const int hi = p == P - 1 ? indptr[i + 1] : lo_in[(int64_t)(p + 1) * m + i];
  const int beta = bucket_of_dev(widths, NB, hi - lo);
  const int64_t pos = (int64_t)base_in[(int64_t)p * m + i] * widths[beta] + (e - lo);
  a_tab[p * NB + beta][pos] = values[e];
}

int check_args(const char* who, int32_t num_rows, int32_t num_cols, int32_t parts, const int32_t* buckets,
               int32_t nb) {
  STIR_REQUIRE(num_rows >= 0 && num_cols >= 0, "%s: bad matrix shape %d x %d", who, num_rows, num_cols);
  STIR_REQUIRE(parts > 0 && parts <= 65535, "%s: num_col_parts=%d", who, parts);
  STIR_REQUIRE(nb > 0 && nb <= 65535 && buckets, "%s: empty bucket list", who);
  for (int b = 0; b < nb; ++b) STIR_REQUIRE(buckets[b] > 0, "%s: bucket width %d is not positive", who, buckets[b]);
  for (int b = 1; b < nb; ++b) STIR_REQUIRE(buckets[b - 1] <= buckets[b], "%s: bucket widths must ascend", who);
  return 0;
}

}  // namespace

extern "C" {

size_t stir_column_part_hyb_device_workspace_bytes(int32_t num_rows, int32_t num_col_parts,
                                                   int32_t num_buckets) {
  if (num_rows < 0 || num_col_parts <= 0 || num_buckets <= 0) return 0;
  return carve(nullptr, num_rows, num_col_parts, num_buckets).bytes;
}

int stir_column_part_hyb_device_sizes(int32_t num_rows, int32_t num_cols, const int32_t* d_indptr,
                                      const int32_t* d_indices, int32_t num_col_parts,
                                      const int32_t* buckets, int32_t num_buckets, void* d_workspace,
                                      int64_t* nrows, void* stream) {
  const char* who = "ColumnPartHyb(device)";
  if (check_args(who, num_rows, num_cols, num_col_parts, buckets, num_buckets)) return -1;
  STIR_REQUIRE(nrows, "%s: nrows is null", who);
  const int P = num_col_parts, NB = num_buckets, m = num_rows;
  std::fill(nrows, nrows + size_t(P) * NB, int64_t(0));
  if (m == 0) return 0;
  STIR_REQUIRE(d_indptr && d_workspace, "%s: null pointer argument", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  Workspace ws = carve(d_workspace, m, P, NB);
  const int64_t W = stir::ceil_div(m, kWave);
  int32_t ends[2];
  STIR_HIP(hipMemcpyAsync(&ends[0], d_indptr, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipMemcpyAsync(&ends[1], d_indptr + m, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipMemcpyAsync(ws.widths, buckets, sizeof(int32_t) * NB, hipMemcpyHostToDevice, st));
  STIR_HIP(hipMemsetAsync(ws.status, 0, sizeof(int32_t), st));
  STIR_HIP(hipStreamSynchronize(st));
  const int64_t nnz = (int64_t)ends[1] - ends[0];
  STIR_REQUIRE(ends[0] >= 0 && nnz >= 0, "%s: indptr is not a CSR row pointer", who);
  STIR_REQUIRE(nnz == 0 || (d_indices && num_cols > 0), "%s: nonzeros but no columns", who);
  const int psize = num_cols > 0 ? (num_cols + P - 1) / P : 1;
  if (nnz > 0) {
    hipLaunchKernelGGL(validate_kernel, dim3((unsigned)stir::ceil_div(nnz, 256)), dim3(256), 0, st, m,
                       num_cols, nnz, ends[0], d_indptr, d_indices, ws.status);
    STIR_LAUNCH_CHECK();
  }
  dim3 grid((unsigned)stir::ceil_div(m, 256), (unsigned)P);
  hipLaunchKernelGGL(count_kernel, grid, dim3(256), 0, st, m, psize, NB, W, d_indptr, d_indices,
                     ws.widths, ws.lo, ws.hist);
  STIR_LAUNCH_CHECK();
  hipLaunchKernelGGL(scan_kernel, dim3((unsigned)NB, (unsigned)P), dim3(256), 0, st, NB, W, ws.hist,
                     ws.totals);
  STIR_LAUNCH_CHECK();
  int32_t status = 0;
  STIR_HIP(hipMemcpyAsync(&status, ws.status, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipMemcpyAsync(nrows, ws.totals, sizeof(int64_t) * size_t(P) * NB, hipMemcpyDeviceToHost, st));
  STIR_HIP(hipStreamSynchronize(st));
  STIR_REQUIRE(!(status & kStatusRange), "%s: a column index lies outside [0, %d)", who, num_cols);
  STIR_REQUIRE(!(status & kStatusUnsorted),
               "%s: column indices must ascend inside each row (use the host routine for unsorted rows)", who);
  return 0;
}

int stir_column_part_hyb_device_fill(int32_t num_rows, int32_t num_cols, const int32_t* d_indptr,
                                     const int32_t* d_indices, int32_t num_col_parts,
                                     const int32_t* buckets, int32_t num_buckets, void* d_workspace,
                                     int32_t* const* d_row_indices, int32_t* const* d_col_indices,
                                     int32_t* const* d_mask, void* stream) {
  const char* who = "ColumnPartHyb(device)";
  if (check_args(who, num_rows, num_cols, num_col_parts, buckets, num_buckets)) return -1;
  const int P = num_col_parts, NB = num_buckets, m = num_rows;
  if (m == 0) return 0;
  STIR_REQUIRE(d_indptr && d_workspace && d_row_indices && d_col_indices && d_mask, "%s: null pointer argument", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  Workspace ws = carve(d_workspace, m, P, NB);
  const int64_t W = stir::ceil_div(m, kWave);
  int32_t ends[2];
  STIR_HIP(hipMemcpyAsync(&ends[0], d_indptr, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipMemcpyAsync(&ends[1], d_indptr + m, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  const size_t tab = sizeof(void*) * size_t(P) * NB;
  STIR_HIP(hipMemcpyAsync(ws.rows_tab, d_row_indices, tab, hipMemcpyHostToDevice, st));
  STIR_HIP(hipMemcpyAsync(ws.cols_tab, d_col_indices, tab, hipMemcpyHostToDevice, st));
  STIR_HIP(hipMemcpyAsync(ws.mask_tab, d_mask, tab, hipMemcpyHostToDevice, st));
  STIR_HIP(hipStreamSynchronize(st));
  const int64_t nnz = (int64_t)ends[1] - ends[0];
  if (nnz <= 0) return 0;
  const int psize = (num_cols + P - 1) / P;
  dim3 grid((unsigned)stir::ceil_div(m, 256), (unsigned)P);
  hipLaunchKernelGGL(place_rows_kernel, grid, dim3(256), 0, st, m, NB, W, d_indptr, ws.widths, ws.lo,
                     ws.hist, ws.base, ws.rows_tab, ws.cols_tab, ws.mask_tab);
  STIR_LAUNCH_CHECK();
  hipLaunchKernelGGL(place_entries_kernel, dim3((unsigned)stir::ceil_div(nnz, 256)), dim3(256), 0, st, m, P,
                     psize, NB, nnz, ends[0], d_indptr, d_indices, ws.widths, ws.lo, ws.base, ws.cols_tab,
                     ws.mask_tab);
  STIR_LAUNCH_CHECK();
  return 0;
}

int stir_column_part_hyb_device_values(int32_t num_rows, int32_t num_cols, const int32_t* d_indptr,
                                       const int32_t* d_indices, const float* d_values,
                                       int32_t num_col_parts, const int32_t* buckets, int32_t num_buckets,
                                       void* d_workspace, const int64_t* nrows, float* const* d_A,
                                       void* stream) {
  const char* who = "ColumnPartHyb(device values)";
  if (check_args(who, num_rows, num_cols, num_col_parts, buckets, num_buckets)) return -1;
  const int P = num_col_parts, NB = num_buckets, m = num_rows;
  if (m == 0) return 0;
  STIR_REQUIRE(d_indptr && d_workspace && nrows && d_A, "%s: null pointer argument", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  Workspace ws = carve(d_workspace, m, P, NB);
  int32_t ends[2];
  STIR_HIP(hipMemcpyAsync(&ends[0], d_indptr, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipMemcpyAsync(&ends[1], d_indptr + m, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  // the A_k pointer table reuses the slot of the mask table (same size, no longer needed)
  STIR_HIP(hipMemcpyAsync(ws.mask_tab, d_A, sizeof(void*) * size_t(P) * NB, hipMemcpyHostToDevice, st));
  STIR_HIP(hipStreamSynchronize(st));
  for (int k = 0; k < P * NB; ++k) {
    STIR_REQUIRE(nrows[k] >= 0 && (nrows[k] == 0 || d_A[k]), "%s: bucket %d has rows but no array", who, k);
    if (nrows[k] > 0)
      STIR_HIP(hipMemsetAsync(d_A[k], 0, sizeof(float) * size_t(nrows[k]) * buckets[k % NB], st));
  }
  const int64_t nnz = (int64_t)ends[1] - ends[0];
  if (nnz <= 0) return 0;
  STIR_REQUIRE(d_indices && d_values, "%s: null pointer argument", who);
  const int psize = (num_cols + P - 1) / P;
  hipLaunchKernelGGL(place_values_kernel, dim3((unsigned)stir::ceil_div(nnz, 256)), dim3(256), 0, st, m, P, psize,
                     NB, nnz, ends[0], d_indptr, d_indices, d_values, ws.widths, ws.lo, ws.base,
                     reinterpret_cast<float* const*>(ws.mask_tab));
  STIR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
