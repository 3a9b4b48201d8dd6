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
// Passes: (0) validate (columns in range; descents between neighbouring entries are counted and
// compared with the descents found at row starts by pass 1, so rows ascend iff the counts agree);
// (1) per (row, partition) binary-search lo and build a per-wavefront histogram of rho per
// bucket; (2) exclusive scan of the histograms along the rows for every (partition, bucket),
// which also yields the ELL row counts; (3) per (row, partition) compute base from the scanned
// histogram plus the rank inside the wavefront, write row ids and padding; (4) scatter the
// column ids and the mask, eight consecutive nonzeros per thread.
#include <cstring>
#include <mutex>
#include <vector>

#include <hipcub/hipcub.hpp>

#include "common.h"
#include "row_lookup.h"
#include "../../include/sparsetir_amd.h"

namespace {

using stir::kWave;

struct Workspace {
  int32_t* lo;       // [P][m]   start of the (row, partition) run inside indices
  int64_t* slot0;    // [P][m]   slot of the run's nonzero e is slot0 + e  (= first ELL row * width - lo)
  int32_t* kb;       // [P][m]   bucket of the run
  int32_t* hist;     // [P][NB][W] per-wavefront ELL-row counts, scanned in place
  int64_t* totals;   // [P][NB]
  int64_t* tile_sums;  // [P][NB][ceil(W / kScanTile)] sums, then offsets, of the scan tiles of hist
  int32_t* widths;   // [NB]
  int32_t* coarse;   // [kCoarse] row that owns nonzero first + q * stride, stride = coarse_stride(nnz)
  int32_t* status;   // [1 + 2 * kCountSlots] status bits; descents between neighbours; descents at row starts
  int32_t** rows_tab;  // [P*NB] output pointers
  int32_t** cols_tab;
  int32_t** mask_tab;
  size_t bytes;       // of the regions above
  // Behind them, with several partitions: the nonzeros regrouped by (row, partition) for
  // matrices whose rows are not ordered by partition -- column ids idx2[nnz] and their source
  // positions perm[nnz], see permuted_tail().
};

// The two descent counts are kept as kCountSlots partial sums each (a workgroup adds to the slot
// of its index), since atomics on a single address serialise; the host adds the slots up.
constexpr int kCountSlots = 1024;
constexpr int kStatusInts = 2 + 2 * kCountSlots;  // status bits, 2 x kCountSlots counters, permuted flag
constexpr int kPermutedAt = 1 + 2 * kCountSlots;

// Row lookup for the per-nonzero passes: the row of every stride-th nonzero is recorded while the
// rows are counted, so a thread finds the row of its first nonzero with a binary search over the
// few rows between two recorded ones instead of over all of indptr.
constexpr int kCoarse = 65536;
inline int64_t coarse_stride(int64_t nnz) { return nnz > kCoarse ? (nnz + kCoarse - 1) / kCoarse : 1; }

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
  w.slot0 = reinterpret_cast<int64_t*>(take(sizeof(int64_t) * size_t(P) * size_t(m > 0 ? m : 1)));
  w.kb = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * size_t(P) * size_t(m > 0 ? m : 1)));
  w.hist = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * size_t(P) * size_t(W > 0 ? W : 1) * NB));
  w.totals = reinterpret_cast<int64_t*>(take(sizeof(int64_t) * size_t(P) * NB));
  w.tile_sums = reinterpret_cast<int64_t*>(take(sizeof(int64_t) * size_t(P) * NB * size_t(W / 4096 + 1)));
  w.widths = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * NB));
  w.coarse = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * kCoarse));
  w.status = reinterpret_cast<int32_t*>(take(sizeof(int32_t) * kStatusInts));
  // the three pointer tables are contiguous so that one copy fills them
  w.rows_tab = reinterpret_cast<int32_t**>(take(sizeof(void*) * 3 * size_t(P) * NB));
  w.cols_tab = w.rows_tab ? w.rows_tab + size_t(P) * NB : nullptr;
  w.mask_tab = w.rows_tab ? w.rows_tab + 2 * size_t(P) * NB : nullptr;
  w.bytes = off;
  return w;
}

enum { kStatusRange = 1, kStatusUnsorted = 2, kStatusIndptr = 4 };

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

// (0) every column inside [0, num_cols); counts the positions e whose successor lies in an
// earlier column partition.  Such a descent is legal only where e + 1 opens a row; count_kernel
// counts those, and the rows are ordered by partition -- all the closed form needs -- exactly
// when the two counts agree.  A thread checks kValidatePerThread consecutive
// entries (vector loads when aligned) and the step to its neighbour's first entry.
constexpr int kValidatePerThread = 16;
__global__ __launch_bounds__(256) void validate_kernel(int num_cols, int psize, int64_t nnz, int32_t first,
                                                       const int32_t* __restrict__ indices,
                                                       int32_t* __restrict__ status) {
  constexpr int N = kValidatePerThread;
  const int64_t end = first + nnz;
  const int64_t e0 = first + ((int64_t)blockIdx.x * 256 + threadIdx.x) * N;
  int v[N + 1];
  const bool full = e0 + N <= end;
  if (full && (reinterpret_cast<uintptr_t>(indices + e0) & 15) == 0) {
#pragma unroll
    for (int j = 0; j < N; j += 4) {
      const int4 c = *reinterpret_cast<const int4*>(indices + e0 + j);
      v[j] = c.x, v[j + 1] = c.y, v[j + 2] = c.z, v[j + 3] = c.w;
    }
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) v[j] = e0 + j < end ? indices[e0 + j] : 0;
  }
  // successor of the last entry: the next lane's first one; the wavefront's last lane reads it
  v[N] = __shfl_down(v[0], 1, kWave);
  if ((threadIdx.x & 63) == 63 && e0 + N < end) v[N] = indices[e0 + N];
  int descents = 0;
  bool bad = false;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    if (e0 + j < end) {
      bad |= v[j] < 0 || v[j] >= num_cols;
      if (e0 + j + 1 < end && v[j + 1] / psize < v[j] / psize) ++descents;
    }
  }
  __shared__ int block_descents;
  if (threadIdx.x == 0) block_descents = 0;
  __syncthreads();
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) descents += __shfl_xor(descents, off, kWave);
  if ((threadIdx.x & 63) == 0 && descents) atomicAdd(&block_descents, descents);
  __syncthreads();
  if (threadIdx.x == 0 && block_descents) atomicAdd(status + 1 + (blockIdx.x % kCountSlots), block_descents);
  if (bad) atomicOr(status, kStatusRange);
}

// (1) lo per (row, partition) and per-wavefront histogram.  grid (ceil(m/256), P).
__global__ __launch_bounds__(256) void count_kernel(int m, int psize, int NB, int64_t W, int first, int64_t end,
                                                    int64_t stride, int32_t* __restrict__ coarse,
                                                    const int32_t* __restrict__ indptr,
                                                    const int32_t* __restrict__ indices,
                                                    const int32_t* __restrict__ widths,
                                                    int32_t* __restrict__ lo_out, int32_t* __restrict__ hist,
                                                    int32_t* __restrict__ status) {
  const int p = blockIdx.y;
  const int P = gridDim.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  int d = 0;
  bool boundary_descent = false;
  if (i < m) {
    int rs = indptr[i], re = indptr[i + 1];
    if (re < rs || rs < first || re > end) {
      if (p == 0) atomicOr(status, kStatusIndptr);
      rs = re = first;
    }
    // a non-empty row that is not the last: does the next stored entry hold a smaller column?
    if (p == 0 && re > rs && re < end) boundary_descent = indices[re] / psize < indices[re - 1] / psize;
    if (p == 0)
      for (int64_t q = (rs - first + stride - 1) / stride; first + q * stride < re; ++q) coarse[q] = i;
    const int lo = p == 0 ? rs : lower_bound_dev(indices, rs, re, (int64_t)p * psize);
    const int hi = p == P - 1 ? re : lower_bound_dev(indices, lo, re, (int64_t)(p + 1) * psize);
    lo_out[(int64_t)p * m + i] = lo;
    d = hi - lo;
  }
  if (wave >= W) return;
  if (p == 0) {
    const unsigned long long bd = __ballot(boundary_descent);
    if (lane == 0 && bd) atomicAdd(status + 1 + kCountSlots + (wave % kCountSlots), __popcll(bd));
  }
  const int beta = bucket_of_dev(widths, NB, d);
  const int w = widths[beta];
  const int rho = d == 0 ? 0 : (d + w - 1) / w;
  int32_t* h = hist + (int64_t)p * NB * W + wave;  // [b][W]
  for (int b = 0; b < NB - 1; ++b) {
    const unsigned long long bal = __ballot(d > 0 && beta == b);
    if (lane == 0) h[b * W] = __popcll(bal);
  }
  int tot = beta == NB - 1 ? rho : 0;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) tot += __shfl_xor(tot, off, kWave);
  if (lane == 0) h[(NB - 1) * W] = tot;
}

// (2) exclusive scan of hist[p][b][.] along the wavefront axis, in three launches: sums of tiles
// of kScanTile entries, an exclusive scan of the tile sums of every (p, b) row by one workgroup,
// and the scan inside every tile started from its offset.
constexpr int kScanTile = 4096;  // 256 threads x 16 consecutive entries
constexpr int kScanPer = kScanTile / 256;

__device__ __forceinline__ int64_t block_sum_256(int64_t v, int64_t* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  if (lane == 0) red[wave] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

// grid (tiles, P * NB)
__global__ __launch_bounds__(256) void scan_tile_sums_kernel(int64_t W, int64_t tiles,
                                                             const int32_t* __restrict__ hist,
                                                             int64_t* __restrict__ tile_sums) {
  __shared__ int64_t red[4];
  const int32_t* h = hist + (int64_t)blockIdx.y * W;
  const int64_t w0 = (int64_t)blockIdx.x * kScanTile;
  int64_t sum = 0;
#pragma unroll
  for (int k = 0; k < kScanPer; ++k) {
    const int64_t w = w0 + threadIdx.x + 256 * k;
    if (w < W) sum += h[w];
  }
  sum = block_sum_256(sum, red);
  if (threadIdx.x == 0) tile_sums[(int64_t)blockIdx.y * tiles + blockIdx.x] = sum;
}

// grid (P * NB), 256 threads: tile sums -> exclusive offsets, row total
__global__ __launch_bounds__(256) void scan_tile_offsets_kernel(int64_t tiles, int64_t* __restrict__ tile_sums,
                                                                int64_t* __restrict__ totals) {
  __shared__ int64_t part[256];
  int64_t* ts = tile_sums + (int64_t)blockIdx.x * tiles;
  int64_t carry = 0;
  for (int64_t t0 = 0; t0 < tiles; t0 += 256) {
    const int64_t t = t0 + threadIdx.x;
    const int64_t v = t < tiles ? ts[t] : 0;
    part[threadIdx.x] = v;
    __syncthreads();
    // Hillis-Steele inclusive scan of 256 values
    for (int off = 1; off < 256; off <<= 1) {
      const int64_t up = (int)threadIdx.x >= off ? part[threadIdx.x - off] : 0;
      __syncthreads();
      part[threadIdx.x] += up;
      __syncthreads();
    }
    if (t < tiles) ts[t] = carry + part[threadIdx.x] - v;
    carry += part[255];
    __syncthreads();
  }
  if (threadIdx.x == 0) totals[blockIdx.x] = carry;
}

// grid (tiles, P * NB): exclusive scan inside the tile; a thread owns kScanPer consecutive entries,
// moved through LDS so that global accesses stay coalesced
__global__ __launch_bounds__(256) void scan_apply_kernel(int64_t W, int64_t tiles, int32_t* __restrict__ hist,
                                                         const int64_t* __restrict__ tile_sums) {
  __shared__ int32_t tile[256][kScanPer + 1];
  __shared__ int64_t part[256];
  int32_t* h = hist + (int64_t)blockIdx.y * W;
  const int64_t w0 = (int64_t)blockIdx.x * kScanTile;
#pragma unroll
  for (int k = 0; k < kScanPer; ++k) {
    const int e = threadIdx.x + 256 * k;
    const int64_t w = w0 + e;
    tile[e / kScanPer][e % kScanPer] = w < W ? h[w] : 0;
  }
  __syncthreads();
  int32_t v[kScanPer];
  int64_t sum = 0;
#pragma unroll
  for (int k = 0; k < kScanPer; ++k) {
    v[k] = tile[threadIdx.x][k];
    sum += v[k];
  }
  part[threadIdx.x] = sum;
  __syncthreads();
  for (int off = 1; off < 256; off <<= 1) {
    const int64_t up = (int)threadIdx.x >= off ? part[threadIdx.x - off] : 0;
    __syncthreads();
    part[threadIdx.x] += up;
    __syncthreads();
  }
  int64_t run = tile_sums[(int64_t)blockIdx.y * tiles + blockIdx.x] + part[threadIdx.x] - sum;
#pragma unroll
  for (int k = 0; k < kScanPer; ++k) {
    tile[threadIdx.x][k] = (int32_t)run;
    run += v[k];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kScanPer; ++k) {
    const int e = threadIdx.x + 256 * k;
    const int64_t w = w0 + e;
    if (w < W) h[w] = tile[e / kScanPer][e % kScanPer];
  }
}

// Spreads the items (lane, off), off < count[lane], evenly over the lanes: item number t (in lane
// order, then off) goes to lane t % 64.  In every round all 64 lanes call f(owner, off, active)
// together, so f may read other lanes' registers with __shfl(x, owner); lanes without an item in
// the last round pass active = false (and owner 0) and must not store.
template <class F>
__device__ __forceinline__ void wave_fill(int count, int lane, F f) {
  int incl = count;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int up = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += up;
  }
  const int excl = incl - count;
  const int total = __shfl(incl, kWave - 1, kWave);
  for (int t0 = 0; t0 < total; t0 += kWave) {
    const int t = t0 + lane;
    // owner: last lane whose exclusive prefix is <= t (lanes with count 0 share their prefix with
    // the next lane and are never the last)
    int lo = 0, hi = kWave - 1;
#pragma unroll
    for (int step = 0; step < 6; ++step) {
      const int mid = (lo + hi + 1) >> 1;
      if (__shfl(excl, mid, kWave) <= t) lo = mid; else hi = mid - 1;
    }
    const int start = __shfl(excl, lo, kWave);
    const bool active = t < total;
    f(active ? lo : 0, active ? t - start : 0, active);
  }
}

// (3) base per (row, partition); row ids and padding slots.  grid (ceil(m/256), P).
__global__ __launch_bounds__(256) void place_rows_kernel(int m, int NB, int64_t W,
                                                         const int32_t* __restrict__ indptr,
                                                         const int32_t* __restrict__ widths,
                                                         const int32_t* __restrict__ lo_in,
                                                         const int32_t* __restrict__ hist,
                                                         int64_t* __restrict__ slot0_out,
                                                         int32_t* __restrict__ kb_out,
                                                         int32_t* const* __restrict__ rows_tab,
                                                         int32_t* const* __restrict__ cols_tab,
                                                         int32_t* const* __restrict__ mask_tab) {
  const int p = blockIdx.y;
  const int P = gridDim.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wave >= W) return;
  int d = 0, lo = 0;
  if (i < m) {
    lo = lo_in[(int64_t)p * m + i];
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
  const bool live = i < m && d > 0;
  int64_t base = 0;
  if (live) {
    base = (int64_t)hist[((int64_t)p * NB + beta) * W + wave] + rank;
  }
  if (i < m) {
    slot0_out[(int64_t)p * m + i] = base * w - lo;
    kb_out[(int64_t)p * m + i] = beta;
  }
  const int k = p * NB + beta;
  // Row ids (rho per lane) and padding slots (rho * w - d per lane) are written by the whole
  // wavefront: item t of the concatenated per-lane ranges goes to lane t % 64, which finds the
  // owning lane by binary search over the exclusive prefix sums.  A row of the widest bucket with
  // hundreds of ELL rows, or a wide row with hundreds of padding slots, costs its share of
  // coalesced stores instead of a serial loop in one lane.
  wave_fill(live ? rho : 0, lane, [&](int owner, int off, bool active) {
    const int kk = __shfl(k, owner, kWave);
    const int64_t b0 = __shfl(base, owner, kWave);
    const int row = __shfl(i, owner, kWave);
    if (active) rows_tab[kk][b0 + off] = row;
  });
  if (P == 1) return;  // one partition: the entry pass writes the padding with the entries
  const int64_t pad0 = base * w + d;
  wave_fill(live ? rho * w - d : 0, lane, [&](int owner, int off, bool active) {
    const int kk = __shfl(k, owner, kWave);
    const int64_t s = __shfl(pad0, owner, kWave) + off;
    if (active) {
      cols_tab[kk][s] = 0;
      mask_tab[kk][s] = 0;
    }
  });
}

// (4) entry placement, two phases per wavefront over 512 consecutive nonzeros.  First a lane owns
// kEntriesPerThread consecutive nonzeros: a binary search finds the row of the first, the others
// follow by walking the row pointer; the slot of an entry is base * width + (position inside its
// (row, partition) run), and the run's parameters are looked up again only when the row or the
// partition changes.  The row pointers the wavefront needs -- the rows between the recorded rows
// around its nonzeros -- are fetched into LDS with one coalesced load when they fit the window,
// so the search and the walk touch no global memory.  The (bucket, slot) pairs go to the
// wavefront's piece of LDS.  Then the lanes take the nonzeros in lane-strided order, so that
// neighbouring lanes hold neighbouring nonzeros and -- inside a run -- neighbouring slots: the
// scattered stores of a run coalesce.  f(k, slot, e) is called once for every nonzero e, k being
// the (partition, bucket) index.
constexpr int kEntriesPerThread = 8;
constexpr int kStageStride = 72;  // LDS words between the j-th entries of lanes 0 and 64: 2-way conflicts at most
constexpr int kRowWindow = 256;   // row pointers held in LDS per wavefront (plus one)
constexpr int64_t kMaxSlots = int64_t(1) << 40;  // slot numbers are staged as 8 + 32 bits
struct alignas(16) EntryStage {
  int32_t kh[kEntriesPerThread * kStageStride];       // k * 256 + (slot >> 32), -1: no entry
  uint32_t slot_lo[kEntriesPerThread * kStageStride];
  int32_t ptr[kRowWindow + 1 + 3];
};
// One column partition: everything an entry needs is a function of its row, so the wavefront
// tabulates it for the rows of its window instead.
struct alignas(16) RowStage {
  int32_t ptr[kRowWindow + 1 + 3];
  int32_t k[kRowWindow];           // bucket of the row
  uint32_t slot0_lo[kRowWindow];   // slot of entry e of the row is slot0 + e
  int32_t slot0_hi[kRowWindow];
  int32_t pad[kRowWindow];         // padding slots after the row's last entry
};

constexpr int kGeneralTile = kWave * kEntriesPerThread;  // nonzeros per wavefront, general path
constexpr int kSingleTile = kGeneralTile;

// Output pointers of the first kLdsTable (partition, bucket) pairs, copied to LDS when a kernel
// starts.  The memory counter of a wavefront retires loads and stores in order, so a pointer
// fetched from global memory between two stores would wait for the first store to complete;
// from LDS it does not.
constexpr int kLdsTable = 256;
template <class T>
struct PtrTable {
  T* lds[kLdsTable];
  T* const* global;
  int count;
  __device__ __forceinline__ void load(T* const* tab, int n) {  // all threads of the workgroup
    global = tab;
    count = n;
    for (int k = threadIdx.x; k < n && k < kLdsTable; k += blockDim.x) lds[k] = tab[k];
  }
  __device__ __forceinline__ T* at(int k) const { return k < kLdsTable ? lds[k] : global[k]; }
};

struct EntryArgs {
  int m, P, psize, NB;
  int64_t nnz;
  int32_t first;
  const int32_t* __restrict__ indptr;
  const int32_t* __restrict__ indices;
  const int32_t* __restrict__ widths;
  const int64_t* __restrict__ slot0_in;
  const int32_t* __restrict__ kb_in;
  const int32_t* __restrict__ coarse;
  int64_t stride;
  // several partitions: flag (device) saying that the rows were not ordered by partition, and
  // then the regrouped column ids and their source positions, indexed like `indices`
  const int32_t* permuted;
  const int32_t* idx2;
  const int32_t* perm;
};

// The view of the matrix the placement kernels walk: the caller's arrays, or the regrouped ones.
__device__ __forceinline__ EntryArgs effective(EntryArgs g) {
  if (g.permuted && *g.permuted)
    g.indices = g.idx2;
  else
    g.perm = nullptr;
  return g;
}

// Rows that can own the nonzeros [e_first, e_last]: between the recorded rows around them.
__device__ __forceinline__ void row_range(const EntryArgs& g, int64_t e_first, int64_t e_last, int& ra, int& rb) {
  const int64_t qa = (e_first - g.first) / g.stride, qb = (e_last - g.first) / g.stride;
  ra = g.coarse[qa];
  rb = (qb + 1) * g.stride < g.nnz ? g.coarse[qb + 1] : g.m - 1;
}

// General path for the kGeneralTile nonzeros from tile_e0 on.
template <bool SINGLE, class L, class F, class Z>
__device__ __forceinline__ void place_general(const EntryArgs& g, EntryStage& st, int64_t tile_e0, int lane, L load,
                                              F f, Z zero) {
  const int m = g.m, NB = g.NB;
  const int64_t end = g.first + g.nnz;
  if (tile_e0 >= end) return;
  const int64_t tile_last = min(end, tile_e0 + kGeneralTile) - 1;
  int ra, rb;
  row_range(g, tile_e0, tile_last, ra, rb);
  const bool windowed = rb - ra < kRowWindow;  // uniform
  __builtin_amdgcn_wave_barrier();
  if (windowed) {
#pragma unroll
    for (int t = 0; t * kWave < kRowWindow + 1; ++t) {
      const int r = ra + t * kWave + lane;
      if (t * kWave + lane <= kRowWindow && r <= rb + 1) st.ptr[t * kWave + lane] = g.indptr[r];
    }
  }
  __builtin_amdgcn_wave_barrier();
  auto ptr_at = [&](int r) -> int64_t { return windowed ? st.ptr[r - ra] : g.indptr[r]; };
  const int64_t e0 = tile_e0 + lane * kEntriesPerThread;
  if (e0 < end) {
    int col[kEntriesPerThread];
    if (e0 + kEntriesPerThread <= end && (reinterpret_cast<uintptr_t>(g.indices + e0) & 15) == 0) {
      const int4 c0 = *reinterpret_cast<const int4*>(g.indices + e0);
      const int4 c1 = *reinterpret_cast<const int4*>(g.indices + e0 + 4);
      col[0] = c0.x, col[1] = c0.y, col[2] = c0.z, col[3] = c0.w;
      col[4] = c1.x, col[5] = c1.y, col[6] = c1.z, col[7] = c1.w;
    } else {
#pragma unroll
      for (int j = 0; j < kEntriesPerThread; ++j) col[j] = e0 + j < end ? g.indices[e0 + j] : 0;
    }
    // row that owns e0: last r in [ra, rb] with indptr[r] <= e0 (rows before it with the same
    // offset are empty)
    int a = ra, b = rb;
    while (a < b) {
      const int mid = a + ((b - a + 1) >> 1);
      if (ptr_at(mid) <= e0) a = mid; else b = mid - 1;
    }
    int r = a;
    int64_t row_end = ptr_at(r + 1);
    int cur_p = -1, k = 0;
    int64_t slot0 = 0;  // slot of entry e is slot0 + e
#pragma unroll
    for (int j = 0; j < kEntriesPerThread; ++j) {
      const int64_t e = e0 + j;
      const int at = j * kStageStride + lane;
      if (e >= end) {
        st.kh[at] = -1;
        continue;
      }
      while (e >= row_end) {
        ++r;
        row_end = ptr_at(r + 1);
        cur_p = -1;
      }
      const int p = col[j] / g.psize;
      if (p != cur_p) {
        cur_p = p;
        k = p * NB + g.kb_in[(int64_t)p * m + r];
        slot0 = g.slot0_in[(int64_t)p * m + r];
      }
      const int64_t slot = slot0 + e;
      st.kh[at] = k * 256 + (int32_t)(slot >> 32);
      st.slot_lo[at] = (uint32_t)slot;
      if (SINGLE && e + 1 == row_end) {
        // one partition: the padding behind a row's last entry is written here (rare path:
        // more rows around the wavefront's nonzeros than the window holds)
        const int w = g.widths[k];
        const int64_t stop = (slot + w) / w * w;
        for (int64_t z = slot + 1; z < stop; ++z) zero(k, z);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < kEntriesPerThread; ++j) st.kh[j * kStageStride + lane] = -1;
  }
  __builtin_amdgcn_wave_barrier();
  int khs[kEntriesPerThread], src[kEntriesPerThread];
  uint32_t lows[kEntriesPerThread];
#pragma unroll
  for (int t = 0; t < kEntriesPerThread; ++t) {
    const int n = t * kWave + lane;  // n-th nonzero of the tile: entry n % 8 of lane n / 8
    const int at = (n % kEntriesPerThread) * kStageStride + n / kEntriesPerThread;
    khs[t] = st.kh[at];
    lows[t] = st.slot_lo[at];
    src[t] = khs[t] >= 0 ? load(tile_e0 + n) : 0;  // every load of the tile precedes its stores
  }
#pragma unroll
  for (int t = 0; t < kEntriesPerThread; ++t)
    if (khs[t] >= 0) f(khs[t] >> 8, ((int64_t)(khs[t] & 255) << 32) | lows[t], src[t]);
}

// One partition, rows [ra, rb] fit the window: fetch what the tile's nonzeros carry (lane-strided),
// tabulate bucket and first slot per row, place the nonzeros, then zero the padding behind every
// row whose last entry lies in the tile (so that a row's slots reach memory together).  All global
// loads come before the first store.
template <class L, class F, class Z>
__device__ __forceinline__ void place_single(const EntryArgs& g, RowStage& rs, int64_t tile_e0, int64_t tile_last,
                                             int ra, int rb, int lane, L load, F f, Z zero) {
  const int nr = rb - ra + 1;
  int src[kEntriesPerThread];
#pragma unroll
  for (int t = 0; t < kEntriesPerThread; ++t) {
    const int64_t e = tile_e0 + t * kWave + lane;
    src[t] = e <= tile_last ? load(e) : 0;
  }
#pragma unroll
  for (int t = 0; t * kWave < kRowWindow; ++t) {
    const int x = t * kWave + lane;
    if (x < nr) {
      const int lo = g.indptr[ra + x], hi = g.indptr[ra + x + 1];
      const int beta = g.kb_in[ra + x];
      const int64_t slot0 = g.slot0_in[ra + x];
      const int d = hi - lo;
      const int w = g.widths[beta];
      rs.ptr[x] = lo;
      if (x == nr - 1) rs.ptr[nr] = hi;
      rs.k[x] = beta;
      rs.slot0_lo[x] = (uint32_t)slot0;
      rs.slot0_hi[x] = (int32_t)(slot0 >> 32);
      const bool mine = d > 0 && hi - 1 >= tile_e0 && hi - 1 <= tile_last;
      rs.pad[x] = mine ? (d + w - 1) / w * w - d : 0;
    }
  }
  __builtin_amdgcn_wave_barrier();
  int steps = 0;
  while ((1 << steps) < nr) ++steps;
  // window row of each of the lane's nonzeros: last x with ptr[x] <= e; the searches advance
  // together so that their LDS reads overlap
  int a[kEntriesPerThread], b[kEntriesPerThread];
#pragma unroll
  for (int t = 0; t < kEntriesPerThread; ++t) a[t] = 0, b[t] = nr - 1;
  for (int it = 0; it < steps; ++it) {
#pragma unroll
    for (int t = 0; t < kEntriesPerThread; ++t) {
      const int mid = (a[t] + b[t] + 1) >> 1;
      if (rs.ptr[mid] <= tile_e0 + t * kWave + lane) a[t] = mid; else b[t] = mid - 1;
    }
  }
#pragma unroll
  for (int t = 0; t < kEntriesPerThread; ++t) {
    const int64_t e = tile_e0 + t * kWave + lane;
    if (e <= tile_last) {
      const int64_t slot0 = ((int64_t)rs.slot0_hi[a[t]] << 32) | rs.slot0_lo[a[t]];
      f(rs.k[a[t]], slot0 + e, src[t]);
    }
  }
  for (int c = 0; c < nr; c += kWave) {
    const int x = c + lane;
    wave_fill(x < nr ? rs.pad[x] : 0, lane, [&](int owner, int off, bool active) {
      const int xo = c + owner;
      const int64_t slot0 = ((int64_t)rs.slot0_hi[xo] << 32) | rs.slot0_lo[xo];
      if (active) zero(rs.k[xo], slot0 + rs.ptr[xo + 1] + off);
    });
  }
}

// load(e) fetches what nonzero e carries (an int: its column, or the bits of its value),
// f(k, slot, carried) stores it, zero(k, slot) clears a padding slot (one partition only).
template <bool SINGLE, class L, class F, class Z>
__device__ __forceinline__ void for_each_entry_slot(const EntryArgs& g, L load, F f, Z zero) {
  // one piece of LDS per wavefront, viewed as either staging layout (the wavefronts of a
  // workgroup may take different paths, so the pieces must not depend on the view)
  union WaveStage {
    EntryStage entry;
    RowStage row;
  };
  __shared__ WaveStage stage_all[4];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t end = g.first + g.nnz;
  if (SINGLE) {
    const int64_t tile_e0 = g.first + ((int64_t)blockIdx.x * 4 + wave) * kSingleTile;
    if (tile_e0 >= end) return;
    const int64_t tile_last = min(end, tile_e0 + kSingleTile) - 1;
    int ra, rb;
    row_range(g, tile_e0, tile_last, ra, rb);
    if (rb - ra < kRowWindow) {
      place_single(g, stage_all[wave].row, tile_e0, tile_last, ra, rb, lane, load, f, zero);
    } else {
      for (int sub = 0; sub < kSingleTile / kGeneralTile; ++sub)
        place_general<true>(g, stage_all[wave].entry, tile_e0 + (int64_t)sub * kGeneralTile, lane, load, f, zero);
    }
  } else {
    const int64_t tile_e0 = g.first + ((int64_t)blockIdx.x * 4 + wave) * kGeneralTile;
    place_general<false>(g, stage_all[wave].entry, tile_e0, lane, load, f, zero);
  }
}

template <bool SINGLE>
__global__ __launch_bounds__(256) void place_entries_kernel(EntryArgs g_in, int32_t* const* __restrict__ cols_tab,
                                                            int32_t* const* __restrict__ mask_tab) {
  const EntryArgs g = effective(g_in);
  __shared__ PtrTable<int32_t> cols, mask;
  cols.load(cols_tab, g.P * g.NB);
  mask.load(mask_tab, g.P * g.NB);
  __syncthreads();
  for_each_entry_slot<SINGLE>(
      g, [&](int64_t e) { return g.indices[e]; },
      [&](int k, int64_t slot, int col) {
        cols.at(k)[slot] = col;
        mask.at(k)[slot] = 1;
      },
      [&](int k, int64_t slot) {
        cols.at(k)[slot] = 0;
        mask.at(k)[slot] = 0;
      });
}

// Value rewrite: A_k[slot] = values[e] for every nonzero, zero in the padding slots, the
// placement computed exactly as in place_entries_kernel.  (With several partitions the padding
// is cleared beforehand instead.)
template <bool SINGLE>
__global__ __launch_bounds__(256) void place_values_kernel(EntryArgs g_in, const float* __restrict__ values,
                                                           float* const* __restrict__ a_tab) {
  const EntryArgs g = effective(g_in);
  __shared__ PtrTable<float> out;
  out.load(a_tab, g.P * g.NB);
  __syncthreads();
  for_each_entry_slot<SINGLE>(
      g, [&](int64_t e) { return __float_as_int(values[g.perm ? g.perm[e] : e]); },
      [&](int k, int64_t slot, int bits) { out.at(k)[slot] = __int_as_float(bits); },
      [&](int k, int64_t slot) { out.at(k)[slot] = 0.f; });
}

// indptr[0] and indptr[m] as read by the sizing call, remembered per (workspace, indptr) so that
// the fill calls for the same matrix need no device round trip of their own.
struct EndsEntry {
  const void* workspace;
  const void* indptr;
  int32_t num_rows;
  int32_t ends[2];
};
std::mutex g_ends_mutex;
EndsEntry g_ends[8];
int g_ends_next = 0;

void remember_ends(const void* ws, const void* indptr, int32_t m, const int32_t (&ends)[2]) {
  std::lock_guard<std::mutex> lock(g_ends_mutex);
  for (EndsEntry& e : g_ends)
    if (e.workspace == ws) e.workspace = nullptr;  // the workspace now describes another matrix
  g_ends[g_ends_next] = EndsEntry{ws, indptr, m, {ends[0], ends[1]}};
  g_ends_next = (g_ends_next + 1) % 8;
}

bool recall_ends(const void* ws, const void* indptr, int32_t m, int32_t (&ends)[2]) {
  std::lock_guard<std::mutex> lock(g_ends_mutex);
  for (const EndsEntry& e : g_ends)
    if (e.workspace == ws && e.indptr == indptr && e.num_rows == m) {
      ends[0] = e.ends[0], ends[1] = e.ends[1];
      return true;
    }
  return false;
}

// ---- rows that are not ordered by partition: regroup the nonzeros by (row, partition), stably
size_t tail_bytes(int32_t P, int64_t nnz) { return P > 1 && nnz > 0 ? 2 * align_up(sizeof(int32_t) * size_t(nnz)) : 0; }

struct PermutedTail {
  int32_t* idx2;
  int32_t* perm;
};
PermutedTail permuted_tail(void* workspace, const Workspace& ws, int64_t nnz) {
  char* base = static_cast<char*>(workspace) + ws.bytes;
  return PermutedTail{reinterpret_cast<int32_t*>(base),
                      reinterpret_cast<int32_t*>(base + align_up(sizeof(int32_t) * size_t(nnz)))};
}

__global__ __launch_bounds__(256) void perm_keys_kernel(int m, int P, int psize, int64_t nnz, int32_t first,
                                                        const int32_t* __restrict__ indptr,
                                                        const int32_t* __restrict__ indices,
                                                        uint32_t* __restrict__ keys, int32_t* __restrict__ vals) {
  __shared__ int32_t win_all[4][stir::kRowLookupWindow];
  const int lane = threadIdx.x & 63;
  const int64_t end = first + nnz;
  const int64_t e0 = first + ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * (kWave * 8);
  if (e0 >= end) return;
  const int64_t e_last = min(end, e0 + kWave * 8) - 1;
  stir::for_each_nonzero_row<8>(indptr, m, e0, e_last, win_all[threadIdx.x >> 6], lane,
                                [&](int64_t e, int row, int, bool live) {
    if (!live) return;
    keys[e - first] = (uint32_t)row * (uint32_t)P + (uint32_t)(indices[e] / psize);
    vals[e - first] = (int32_t)e;
  });
}

__global__ __launch_bounds__(256) void perm_gather_kernel(int64_t nnz, const int32_t* __restrict__ indices,
                                                          const int32_t* __restrict__ perm,
                                                          int32_t* __restrict__ idx2) {
  const int64_t s = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (s < nnz) idx2[s] = indices[perm[s]];
}

// Fills tail.perm (source position of the s-th nonzero in the regrouped order) and tail.idx2 (its
// column).  Scratch for the keys and the sort is allocated and freed here: this is the slow path.
int build_permutation(const char* who, int m, int P, int psize, int64_t nnz, int32_t first,
                      const int32_t* d_indptr, const int32_t* d_indices, const PermutedTail& tail,
                      hipStream_t st) {
  STIR_REQUIRE((int64_t)m * P < (int64_t(1) << 32), "%s: %d rows x %d partitions is too large for unsorted rows",
               who, m, P);
  STIR_REQUIRE(nnz < (int64_t(1) << 31), "%s: too many nonzeros for unsorted rows", who);
  int end_bit = 1;
  while (end_bit < 32 && (int64_t(1) << end_bit) < (int64_t)m * P) ++end_bit;
  size_t sort_bytes = 0;
  hipError_t err = hipcub::DeviceRadixSort::SortPairs(nullptr, sort_bytes, (const uint32_t*)nullptr,
                                                      (uint32_t*)nullptr, (const int32_t*)nullptr,
                                                      (int32_t*)nullptr, (int)nnz, 0, end_bit, st);
  uint32_t* keys = nullptr;  // keys, sorted keys, source positions
  void* d_sort = nullptr;
  if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void**>(&keys), sizeof(uint32_t) * 3 * size_t(nnz));
  if (err == hipSuccess) err = hipMalloc(&d_sort, sort_bytes ? sort_bytes : 16);
  if (err == hipSuccess) {
    uint32_t* keys_sorted = keys + nnz;
    int32_t* vals = reinterpret_cast<int32_t*>(keys + 2 * nnz);
    hipLaunchKernelGGL(perm_keys_kernel, dim3((unsigned)stir::ceil_div(nnz, 4 * kWave * 8)), dim3(256), 0, st, m, P,
                       psize, nnz, first, d_indptr, d_indices, keys, vals);
    err = hipGetLastError();
    if (err == hipSuccess)
      err = hipcub::DeviceRadixSort::SortPairs(d_sort, sort_bytes, (const uint32_t*)keys, keys_sorted,
                                               (const int32_t*)vals, tail.perm, (int)nnz, 0, end_bit, st);
    if (err == hipSuccess) {
      hipLaunchKernelGGL(perm_gather_kernel, dim3((unsigned)stir::ceil_div(nnz, 256)), dim3(256), 0, st, nnz,
                         d_indices, tail.perm, tail.idx2);
      err = hipGetLastError();
    }
    if (err == hipSuccess) err = hipStreamSynchronize(st);
  }
  if (keys) (void)hipFree(keys);
  if (d_sort) (void)hipFree(d_sort);
  STIR_REQUIRE(err == hipSuccess, "%s: regrouping unsorted rows failed: %s", who, hipGetErrorString(err));
  return 0;
}

int check_args(const char* who, int32_t num_rows, int32_t num_cols, int32_t parts, const int32_t* buckets,
               int32_t nb) {
  STIR_REQUIRE(num_rows >= 0 && num_cols >= 0, "%s: bad matrix shape %d x %d", who, num_rows, num_cols);
  STIR_REQUIRE(parts > 0 && parts <= 65535, "%s: num_col_parts=%d", who, parts);
  STIR_REQUIRE(nb > 0 && nb <= 65535 && buckets, "%s: empty bucket list", who);
  STIR_REQUIRE((int64_t)parts * nb < (int64_t(1) << 22), "%s: %d partitions x %d buckets is too many", who, parts, nb);
  for (int b = 0; b < nb; ++b) STIR_REQUIRE(buckets[b] > 0, "%s: bucket width %d is not positive", who, buckets[b]);
  for (int b = 1; b < nb; ++b) STIR_REQUIRE(buckets[b - 1] <= buckets[b], "%s: bucket widths must ascend", who);
  return 0;
}

// Scans hist in place (exclusive, per (partition, bucket) row) and leaves the row totals in
// ws.totals.
int scan_hist(const Workspace& ws, int P, int NB, int64_t W, hipStream_t st) {
  const int64_t tiles = stir::ceil_div(W, kScanTile);
  STIR_REQUIRE(tiles < (int64_t(1) << 31), "ColumnPartHyb(device): too many rows for the scan");
  const dim3 grid((unsigned)tiles, (unsigned)(P * NB));
  hipLaunchKernelGGL(scan_tile_sums_kernel, grid, dim3(256), 0, st, W, tiles, ws.hist, ws.tile_sums);
  STIR_LAUNCH_CHECK();
  hipLaunchKernelGGL(scan_tile_offsets_kernel, dim3((unsigned)(P * NB)), dim3(256), 0, st, tiles, ws.tile_sums,
                     ws.totals);
  STIR_LAUNCH_CHECK();
  hipLaunchKernelGGL(scan_apply_kernel, grid, dim3(256), 0, st, W, tiles, ws.hist, ws.tile_sums);
  STIR_LAUNCH_CHECK();
  return 0;
}

}  // namespace

extern "C" {

size_t stir_column_part_hyb_device_workspace_bytes(int32_t num_rows, int32_t num_col_parts,
                                                   int32_t num_buckets, int64_t nnz) {
  if (num_rows < 0 || num_col_parts <= 0 || num_buckets <= 0 || nnz < 0) return 0;
  return carve(nullptr, num_rows, num_col_parts, num_buckets).bytes + tail_bytes(num_col_parts, nnz);
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
  STIR_HIP(hipMemsetAsync(ws.status, 0, sizeof(int32_t) * kStatusInts, st));
  STIR_HIP(hipStreamSynchronize(st));
  const int64_t nnz = (int64_t)ends[1] - ends[0];
  STIR_REQUIRE(ends[0] >= 0 && nnz >= 0, "%s: indptr is not a CSR row pointer", who);
  STIR_REQUIRE(nnz == 0 || (d_indices && num_cols > 0), "%s: nonzeros but no columns", who);
  const int psize = num_cols > 0 ? (num_cols + P - 1) / P : 1;
  if (nnz > 0) {
    hipLaunchKernelGGL(validate_kernel, dim3((unsigned)stir::ceil_div(nnz, 256 * kValidatePerThread)), dim3(256), 0, st, num_cols,
                       psize, nnz, ends[0], d_indices, ws.status);
    STIR_LAUNCH_CHECK();
  }
  dim3 grid((unsigned)stir::ceil_div(m, 256), (unsigned)P);
  hipLaunchKernelGGL(count_kernel, grid, dim3(256), 0, st, m, psize, NB, W, ends[0], (int64_t)ends[1],
                     coarse_stride(nnz), ws.coarse, d_indptr,
                     d_indices, ws.widths, ws.lo, ws.hist, ws.status);
  STIR_LAUNCH_CHECK();
  if (scan_hist(ws, P, NB, W, st)) return -1;
  std::vector<int32_t> counts(kStatusInts, 0);
  STIR_HIP(hipMemcpyAsync(counts.data(), ws.status, sizeof(int32_t) * kStatusInts, hipMemcpyDeviceToHost, st));
  STIR_HIP(hipMemcpyAsync(nrows, ws.totals, sizeof(int64_t) * size_t(P) * NB, hipMemcpyDeviceToHost, st));
  STIR_HIP(hipStreamSynchronize(st));
  const int32_t status = counts[0];
  int64_t descents = 0, row_start_descents = 0;
  for (int k = 0; k < kCountSlots; ++k) {
    descents += counts[1 + k];
    row_start_descents += counts[1 + kCountSlots + k];
  }
  STIR_REQUIRE(!(status & kStatusIndptr), "%s: indptr is not a CSR row pointer (it decreases)", who);
  STIR_REQUIRE(!(status & kStatusRange), "%s: a column index lies outside [0, %d)", who, num_cols);
  // With one partition a run is the whole row whatever the order of its columns.  With several,
  // rows that are not ordered by partition are regrouped by (row, partition) -- stably, so every
  // run keeps the CSR order of its entries as in the sequential routine -- and counted again.
  if (P > 1 && descents != row_start_descents) {
    const PermutedTail tail = permuted_tail(d_workspace, ws, nnz);
    if (build_permutation(who, m, P, psize, nnz, ends[0], d_indptr, d_indices, tail, st)) return -1;
    const int32_t one = 1;
    STIR_HIP(hipMemcpyAsync(ws.status + kPermutedAt, &one, sizeof(one), hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL(count_kernel, grid, dim3(256), 0, st, m, psize, NB, W, ends[0], (int64_t)ends[1],
                       coarse_stride(nnz), ws.coarse, d_indptr, tail.idx2 - ends[0], ws.widths, ws.lo, ws.hist,
                       ws.status);
    STIR_LAUNCH_CHECK();
    if (scan_hist(ws, P, NB, W, st)) return -1;
    STIR_HIP(hipMemcpyAsync(nrows, ws.totals, sizeof(int64_t) * size_t(P) * NB, hipMemcpyDeviceToHost, st));
    STIR_HIP(hipStreamSynchronize(st));
  }
  for (int k = 0; k < P * NB; ++k)
    STIR_REQUIRE(nrows[k] < kMaxSlots / buckets[k % NB], "%s: bucket %d holds too many slots", who, k);
  remember_ends(d_workspace, d_indptr, m, ends);
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
  const bool known = recall_ends(d_workspace, d_indptr, m, ends);
  if (!known) {
    STIR_HIP(hipMemcpyAsync(&ends[0], d_indptr, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    STIR_HIP(hipMemcpyAsync(&ends[1], d_indptr + m, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  }
  const size_t pnb = size_t(P) * NB;
  std::vector<int32_t*> tabs(3 * pnb);
  std::copy(d_row_indices, d_row_indices + pnb, tabs.begin());
  std::copy(d_col_indices, d_col_indices + pnb, tabs.begin() + pnb);
  std::copy(d_mask, d_mask + pnb, tabs.begin() + 2 * pnb);
  STIR_HIP(hipMemcpyAsync(ws.rows_tab, tabs.data(), sizeof(void*) * 3 * pnb, hipMemcpyHostToDevice, st));
  STIR_HIP(hipStreamSynchronize(st));  // `tabs` and `ends` are host stack/heap of this call
  const int64_t nnz = (int64_t)ends[1] - ends[0];
  if (nnz <= 0) return 0;
  const int psize = (num_cols + P - 1) / P;
  dim3 grid((unsigned)stir::ceil_div(m, 256), (unsigned)P);
  hipLaunchKernelGGL(place_rows_kernel, grid, dim3(256), 0, st, m, NB, W, d_indptr, ws.widths, ws.lo,
                     ws.hist, ws.slot0, ws.kb, ws.rows_tab, ws.cols_tab, ws.mask_tab);
  STIR_LAUNCH_CHECK();
  const PermutedTail tail = permuted_tail(d_workspace, ws, nnz);
  const EntryArgs ea{m, P, psize, NB, nnz, ends[0], d_indptr, d_indices, ws.widths, ws.slot0, ws.kb, ws.coarse,
                     coarse_stride(nnz), P > 1 ? ws.status + kPermutedAt : nullptr,
                     P > 1 ? tail.idx2 - ends[0] : nullptr, P > 1 ? tail.perm - ends[0] : nullptr};
  if (P == 1)
    hipLaunchKernelGGL(place_entries_kernel<true>, dim3((unsigned)stir::ceil_div(nnz, 4 * kSingleTile)), dim3(256), 0,
                       st, ea, ws.cols_tab, ws.mask_tab);
  else
    hipLaunchKernelGGL(place_entries_kernel<false>, dim3((unsigned)stir::ceil_div(nnz, 4 * kGeneralTile)), dim3(256),
                       0, st, ea, ws.cols_tab, ws.mask_tab);
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
  if (!recall_ends(d_workspace, d_indptr, m, ends)) {
    STIR_HIP(hipMemcpyAsync(&ends[0], d_indptr, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    STIR_HIP(hipMemcpyAsync(&ends[1], d_indptr + m, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  }
  // the A_k pointer table reuses the slot of the mask table (same size, no longer needed)
  STIR_HIP(hipMemcpyAsync(ws.mask_tab, d_A, sizeof(void*) * size_t(P) * NB, hipMemcpyHostToDevice, st));
  STIR_HIP(hipStreamSynchronize(st));
  for (int k = 0; k < P * NB; ++k) {
    STIR_REQUIRE(nrows[k] >= 0 && (nrows[k] == 0 || d_A[k]), "%s: bucket %d has rows but no array", who, k);
    // several partitions: padding slots are cleared here; with one the entry pass writes them
    if (nrows[k] > 0 && P > 1)
      STIR_HIP(hipMemsetAsync(d_A[k], 0, sizeof(float) * size_t(nrows[k]) * buckets[k % NB], st));
  }
  const int64_t nnz = (int64_t)ends[1] - ends[0];
  if (nnz <= 0) return 0;
  STIR_REQUIRE(d_indices && d_values, "%s: null pointer argument", who);
  const int psize = (num_cols + P - 1) / P;
  float* const* a_tab = reinterpret_cast<float* const*>(ws.mask_tab);
  const PermutedTail tail = permuted_tail(d_workspace, ws, nnz);
  const EntryArgs ea{m, P, psize, NB, nnz, ends[0], d_indptr, d_indices, ws.widths, ws.slot0, ws.kb, ws.coarse,
                     coarse_stride(nnz), P > 1 ? ws.status + kPermutedAt : nullptr,
                     P > 1 ? tail.idx2 - ends[0] : nullptr, P > 1 ? tail.perm - ends[0] : nullptr};
  if (P == 1)
    hipLaunchKernelGGL(place_values_kernel<true>, dim3((unsigned)stir::ceil_div(nnz, 4 * kSingleTile)), dim3(256), 0,
                       st, ea, d_values, a_tab);
  else
    hipLaunchKernelGGL(place_values_kernel<false>, dim3((unsigned)stir::ceil_div(nnz, 4 * kGeneralTile)), dim3(256),
                       0, st, ea, d_values, a_tab);
  STIR_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
