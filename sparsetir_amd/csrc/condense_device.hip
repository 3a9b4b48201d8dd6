// ConDense on the GPU, bit-exact with the host routine (csrc/format_host.cpp) and the reference's
// per-tile multimap walk (src/sparse/format.cc:353-429), which runs on the CPU only.
//
// A tile of t rows keeps the distinct columns of its nonzeros in ascending order, g per group;
// mask[group][row in tile][slot] marks the nonzeros.  Here every nonzero gets the key
// (tile, column); one stable radix sort (hipCUB) brings equal keys together, an inclusive scan of
// the "first of its key" flags numbers the distinct keys, the distinct keys of a tile give its
// groups, and every sorted nonzero then knows its group and slot.
#include <hipcub/hipcub.hpp>

#include <algorithm>

#include "common.h"
#include "row_lookup.h"
#include "../../include/sparsetir_amd.h"

namespace {

using stir::ceil_div;
using stir::kWave;

enum Flag { kBadEnds = 1, kBadIndptr = 2, kBadColumn = 4 };

struct Workspace {
  int32_t* flags;     // [16]
  int32_t* counts;    // [tiles + 1] groups per tile
  uint64_t* keys_in;  // [nnz]
  uint64_t* keys;     // [nnz] sorted
  int32_t* rows_in;   // [nnz] row of every nonzero
  int32_t* rows;      // [nnz] in sorted order
  int32_t* rank;      // [nnz] inclusive count of distinct keys up to a sorted position
  int64_t* begin;     // [tiles + 1] first sorted position of a tile
  void* tmp;          // sort / scan scratch
  size_t tmp_bytes;
  size_t total_bytes;
};

struct HeadFlag {
  const uint64_t* keys;
  __host__ __device__ int32_t operator()(int64_t p) const { return (p == 0 || keys[p] != keys[p - 1]) ? 1 : 0; }
};
using HeadIter = hipcub::TransformInputIterator<int32_t, HeadFlag, hipcub::CountingInputIterator<int64_t>>;

int bit_length(uint64_t x) {
  int b = 0;
  while (x) ++b, x >>= 1;
  return b;
}

size_t scratch_bytes(int64_t nnz, int64_t tiles) {
  size_t sort_bytes = 0, scan_bytes = 0, tile_scan_bytes = 0;
  (void)hipcub::DeviceRadixSort::SortPairs(nullptr, sort_bytes, (const uint64_t*)nullptr, (uint64_t*)nullptr,
                                           (const int32_t*)nullptr, (int32_t*)nullptr, (int)nnz, 0, 64,
                                           (hipStream_t) nullptr);
  HeadIter it(hipcub::CountingInputIterator<int64_t>(0), HeadFlag{nullptr});
  (void)hipcub::DeviceScan::InclusiveSum(nullptr, scan_bytes, it, (int32_t*)nullptr, (int)nnz, (hipStream_t) nullptr);
  (void)hipcub::DeviceScan::ExclusiveSum(nullptr, tile_scan_bytes, (const int32_t*)nullptr, (int32_t*)nullptr,
                                         (int)(tiles + 1), (hipStream_t) nullptr);
  return std::max(std::max(sort_bytes, scan_bytes), tile_scan_bytes);
}

Workspace layout(void* d_ws, int64_t tiles, int64_t nnz) {
  Workspace w{};
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char* p = d_ws ? static_cast<char*>(d_ws) + off : nullptr;
    off += (bytes + 255) / 256 * 256;
    return p;
  };
  const size_t e = size_t(std::max<int64_t>(nnz, 1));
  w.flags = reinterpret_cast<int32_t*>(take(16 * sizeof(int32_t)));
  w.counts = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * size_t(tiles + 1)));
  w.keys_in = reinterpret_cast<uint64_t*>(take(sizeof(uint64_t) * e));
  w.keys = reinterpret_cast<uint64_t*>(take(sizeof(uint64_t) * e));
  w.rows_in = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * e));
  w.rows = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * e));
  w.rank = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * e));
  w.begin = reinterpret_cast<int64_t*>(take(sizeof(int64_t) * size_t(tiles + 1)));
  w.tmp_bytes = scratch_bytes(nnz, tiles);
  w.tmp = take(w.tmp_bytes);
  w.total_bytes = off;
  return w;
}

__global__ __launch_bounds__(256) void condense_check_kernel(int n, int64_t nnz, const int32_t* __restrict__ indptr,
                                                             int32_t* __restrict__ flags) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int bad = 0;
  if (i == 0 && (indptr[0] != 0 || indptr[n] != nnz)) bad |= kBadEnds;
  if (i < n && indptr[i] > indptr[i + 1]) bad |= kBadIndptr;
  if (bad) atomicOr(flags, bad);
}

constexpr int kPer = 8;  // nonzeros per lane: a wavefront takes 512 consecutive ones
__global__ __launch_bounds__(256) void condense_keys_kernel(int n, int64_t nnz, int t,
                                                            const int32_t* __restrict__ indptr,
                                                            const int32_t* __restrict__ indices,
                                                            uint64_t* __restrict__ keys, int32_t* __restrict__ rows,
                                                            int32_t* __restrict__ flags) {
  __shared__ int32_t win[4][stir::kRowLookupWindow];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t e0 = ((int64_t)blockIdx.x * 4 + wave) * (kPer * kWave);
  if (e0 >= nnz) return;
  const int64_t e_last = min(e0 + kPer * kWave, nnz) - 1;
  stir::for_each_nonzero_row<kPer>(indptr, n, e0, e_last, win[wave], lane, [&](int64_t e, int row, int, bool live) {
    if (!live) return;
    int32_t col = indices[e];
    if (col < 0) {
      atomicOr(flags, (int)kBadColumn);
      col = 0;
    }
    keys[e] = ((uint64_t)(uint32_t)(row / t) << 32) | (uint32_t)col;
    rows[e] = row;
  });
}

// begin[tile] = first sorted position whose key belongs to tile or a later one
__global__ __launch_bounds__(256) void condense_bounds_kernel(int64_t tiles, int64_t nnz,
                                                              const uint64_t* __restrict__ keys,
                                                              int64_t* __restrict__ begin) {
  const int64_t tile = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (tile > tiles) return;
  const uint64_t target = (uint64_t)tile << 32;
  int64_t lo = 0, hi = nnz;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (keys[mid] < target) lo = mid + 1; else hi = mid;
  }
  begin[tile] = lo;
}

__device__ __forceinline__ int64_t distinct_before(const int32_t* __restrict__ rank, int64_t pos) {
  return pos > 0 ? rank[pos - 1] : 0;
}

// groups per tile (one more entry, zero, so that the scan's last output is the total)
__global__ __launch_bounds__(256) void condense_count_kernel(int64_t tiles, int g, const int64_t* __restrict__ begin,
                                                             const int32_t* __restrict__ rank,
                                                             int32_t* __restrict__ counts) {
  const int64_t tile = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (tile > tiles) return;
  int64_t grp = 0;
  if (tile < tiles) {
    const int64_t distinct = distinct_before(rank, begin[tile + 1]) - distinct_before(rank, begin[tile]);
    grp = (distinct + g - 1) / g;
  }
  counts[tile] = (int32_t)grp;  // at most the tile's nonzeros
}

__global__ __launch_bounds__(256) void condense_zero_kernel(int32_t* __restrict__ a, int64_t na,
                                                            int32_t* __restrict__ b, int64_t nb) {
  for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < na + nb; q += (int64_t)gridDim.x * 256) {
    if (q < na) a[q] = 0; else b[q - na] = 0;
  }
}

__global__ __launch_bounds__(256) void condense_place_kernel(int64_t nnz, int t, int g,
                                                             const uint64_t* __restrict__ keys,
                                                             const int32_t* __restrict__ rows,
                                                             const int32_t* __restrict__ rank,
                                                             const int64_t* __restrict__ begin,
                                                             const int32_t* __restrict__ group_indptr,
                                                             int32_t* __restrict__ tile_indices,
                                                             int32_t* __restrict__ mask) {
  const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (p >= nnz) return;
  const uint64_t key = keys[p];
  const int64_t tile = (int64_t)(key >> 32);
  const int32_t col = (int32_t)(uint32_t)key;
  const int64_t u = rank[p] - 1 - distinct_before(rank, begin[tile]);  // index among the tile's distinct columns
  const int64_t grp = group_indptr[tile] + u / g;
  const int slot = (int)(u % g);
  if (p == 0 || keys[p - 1] != key) tile_indices[grp * g + slot] = col;
  mask[(grp * t + (rows[p] - tile * t)) * g + slot] = 1;
}

int check_args(const char* who, int32_t n, int64_t nnz, const void* indptr, const void* indices, int32_t t, int32_t g,
               const void* ws) {
  STIR_REQUIRE(n >= 0 && nnz >= 0 && indptr, "%s: bad CSR arguments", who);
  STIR_REQUIRE(nnz == 0 || indices, "%s: indices is null", who);
  STIR_REQUIRE(nnz < (int64_t(1) << 31), "%s: more than 2^31 nonzeros", who);
  STIR_REQUIRE(t > 0 && g > 0, "%s: t=%d g=%d must be positive", who, t, g);
  STIR_REQUIRE(ws, "%s: workspace is null", who);
  return 0;
}

}  // namespace

extern "C" {

size_t stir_condense_device_workspace_bytes(int32_t n, int64_t nnz, int32_t t) {
  if (n < 0 || nnz < 0 || t <= 0) return 0;
  return layout(nullptr, ceil_div(n, t), nnz).total_bytes;
}

int stir_condense_device_sizes(int32_t n, int64_t nnz, const int32_t* d_indptr, const int32_t* d_indices, int32_t t,
                               int32_t g, void* d_workspace, int32_t* d_group_indptr, int64_t* num_groups,
                               void* stream) {
  const char* who = "ConDense(device)";
  if (check_args(who, n, nnz, d_indptr, d_indices, t, g, d_workspace)) return -1;
  STIR_REQUIRE(d_group_indptr && num_groups, "%s: null output", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t tiles = ceil_div(n, t);
  Workspace w = layout(d_workspace, tiles, nnz);
  STIR_HIP(hipMemsetAsync(w.flags, 0, 16 * sizeof(int32_t), st));
  hipLaunchKernelGGL(condense_check_kernel, dim3((unsigned)ceil_div((int64_t)n + 1, 256)), dim3(256), 0, st, n, nnz,
                     d_indptr, w.flags);
  STIR_LAUNCH_CHECK();
  int32_t h_flags = 0;
  STIR_HIP(hipMemcpyAsync(&h_flags, w.flags, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipStreamSynchronize(st));
  STIR_REQUIRE(!(h_flags & kBadEnds), "%s: indptr must run from 0 to the number of nonzeros", who);
  STIR_REQUIRE(!(h_flags & kBadIndptr), "%s: indptr decreases", who);
  if (nnz > 0) {
    hipLaunchKernelGGL(condense_keys_kernel, dim3((unsigned)ceil_div(nnz, 4 * kPer * kWave)), dim3(256), 0, st, n, nnz,
                       t, d_indptr, d_indices, w.keys_in, w.rows_in, w.flags);
    STIR_LAUNCH_CHECK();
    size_t bytes = w.tmp_bytes;
    STIR_HIP(hipcub::DeviceRadixSort::SortPairs(w.tmp, bytes, (const uint64_t*)w.keys_in, w.keys,
                                                (const int32_t*)w.rows_in, w.rows, (int)nnz, 0,
                                                32 + std::max(1, bit_length((uint64_t)tiles)), st));
    HeadIter it(hipcub::CountingInputIterator<int64_t>(0), HeadFlag{w.keys});
    bytes = w.tmp_bytes;
    STIR_HIP(hipcub::DeviceScan::InclusiveSum(w.tmp, bytes, it, w.rank, (int)nnz, st));
  }
  hipLaunchKernelGGL(condense_bounds_kernel, dim3((unsigned)ceil_div(tiles + 1, 256)), dim3(256), 0, st, tiles, nnz,
                     w.keys, w.begin);
  STIR_LAUNCH_CHECK();
  hipLaunchKernelGGL(condense_count_kernel, dim3((unsigned)ceil_div(tiles + 1, 256)), dim3(256), 0, st, tiles, g,
                     w.begin, w.rank, w.counts);
  STIR_LAUNCH_CHECK();
  {
    size_t bytes = w.tmp_bytes;
    STIR_HIP(hipcub::DeviceScan::ExclusiveSum(w.tmp, bytes, (const int32_t*)w.counts, d_group_indptr, (int)(tiles + 1),
                                              st));
  }
  int32_t h_total = 0;  // the groups cannot outnumber the nonzeros, which fit 31 bits
  STIR_HIP(hipMemcpyAsync(&h_flags, w.flags, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipMemcpyAsync(&h_total, d_group_indptr + tiles, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  STIR_HIP(hipStreamSynchronize(st));
  *num_groups = h_total;
  STIR_REQUIRE(!(h_flags & kBadColumn), "%s: a column index is negative", who);
  return 0;
}

int stir_condense_device_fill(int32_t n, int64_t nnz, const int32_t* d_indptr, const int32_t* d_indices, int32_t t,
                              int32_t g, void* d_workspace, const int32_t* d_group_indptr, int64_t num_groups,
                              int32_t* d_tile_indices, int32_t* d_mask, void* stream) {
  const char* who = "ConDense(device)";
  if (check_args(who, n, nnz, d_indptr, d_indices, t, g, d_workspace)) return -1;
  STIR_REQUIRE(d_group_indptr && num_groups >= 0, "%s: bad group arguments", who);
  STIR_REQUIRE(num_groups == 0 || (d_tile_indices && d_mask), "%s: null output", who);
  if (num_groups == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t tiles = ceil_div(n, t);
  Workspace w = layout(d_workspace, tiles, nnz);
  const int64_t na = num_groups * g, nm = num_groups * t * g;
  hipLaunchKernelGGL(condense_zero_kernel, dim3((unsigned)std::min<int64_t>(ceil_div(na + nm, 256), 65536)), dim3(256),
                     0, st, d_tile_indices, na, d_mask, nm);
  STIR_LAUNCH_CHECK();
  hipLaunchKernelGGL(condense_place_kernel, dim3((unsigned)ceil_div(nnz, 256)), dim3(256), 0, st, nnz, t, g, w.keys,
                     w.rows, w.rank, w.begin, d_group_indptr, d_tile_indices, d_mask);
  STIR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
