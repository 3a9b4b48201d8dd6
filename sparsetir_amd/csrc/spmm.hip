// CSR row-split SpMM and hyb (bucketed ELL) SpMM for gfx950, fp32.
//
// Both kernels are gathers of dense feature rows: per nonzero one row of B (feat*4 bytes)
// is read, scaled and summed.  The feature row is spread over a "lane group" of G lanes,
// each lane owning float4 chunks, so one wavefront (64 lanes) serves 64/G nonzeros per
// step with fully coalesced 16-byte loads.  Column indices and values are fetched once per
// wavefront with one coalesced load (lane l holds slot l of the 64-slot tile) and handed to
// the lane groups through cross-lane reads, so no lane issues a redundant index load.
#include <hipcub/hipcub.hpp>

#include <algorithm>
#include <mutex>
#include <vector>

#include "common.h"
#include "row_lookup.h"
#include "../../include/sparsetir_amd.h"

// Device memory of stir_hyb_spmm_f32_noalloc: room for the two descriptor tables of an operator
// with up to kStaticBuckets non-empty buckets (64 bytes per descriptor and table).  One copy per
// GPU, held until the process ends.  Host code reaches it through the per-device address that
// static_scratch() returns, never through this name.
constexpr int kStaticBuckets = 1024;
static __device__ __align__(256) unsigned char scratch[2 * kStaticBuckets * 64];

namespace {

using stir::kWave;

struct alignas(16) HybBucket {
  const float* A;
  const int32_t* rows;
  const int32_t* cols;
  int64_t nrows;
  int64_t tile_begin;  // first wave tile of this bucket in the fused launch
  int32_t width;
  int32_t log2w;   // log2(width) when the bucket runs in slot-tile mode, else -1
  int32_t atomic;  // 0: store the row, 1: add it with atomics, 2: add it with a plain read-modify-write
  int32_t chunks;  // row mode: wave tiles per ELL row (each covers kRowChunk slots)
};

// Row mode splits an ELL row of an accumulating bucket into chunks of this many slots, one
// wavefront each, so that a hub row does not serialise on a single wavefront.
constexpr int kRowChunk = 256;

__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }

__device__ __forceinline__ void fma4(float4& acc, float a, const float4& x) {
  acc.x = fmaf(a, x.x, acc.x);
  acc.y = fmaf(a, x.y, acc.y);
  acc.z = fmaf(a, x.z, acc.z);
  acc.w = fmaf(a, x.w, acc.w);
}

// Sum `acc` over the lane groups whose group index differs in the bits [G, limit).
template <int G, int REP>
__device__ __forceinline__ void reduce_groups(float4 (&acc)[REP], int limit) {
#pragma unroll
  for (int off = G; off < kWave; off <<= 1) {
    if (off < limit) {
#pragma unroll
      for (int r = 0; r < REP; ++r) {
        acc[r].x += __shfl_xor(acc[r].x, off, kWave);
        acc[r].y += __shfl_xor(acc[r].y, off, kWave);
        acc[r].z += __shfl_xor(acc[r].z, off, kWave);
        acc[r].w += __shfl_xor(acc[r].w, off, kWave);
      }
    }
  }
}

// Store, or accumulate with atomics, the 4*G*REP features a lane group holds for output row
// `row`.  A lane owns 4 consecutive floats, so issuing the atomics straight from the registers
// would make every atomic instruction touch G addresses 16 bytes apart (4 cache lines per 32
// lanes, 4 times over).  Instead the group's floats go through the wavefront's piece of LDS
// (`stage`, 256*REP floats) and come back with lane l holding float k*G + l, so each atomic
// instruction covers G consecutive floats.  LDS instructions of one wavefront execute in order,
// no workgroup barrier is involved.
template <int G, int REP>
__device__ __forceinline__ void write_row(float* C, int64_t row, int feat, int lane,
                                          const float4 (&acc)[REP], int atomic, float* stage) {
  const int g = lane / G, gl = lane % G;
  if (atomic == 2) {
    // the only writer of this row in this launch: no atomics needed to add
    float* base = C + row * feat + gl * 4;
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      if (gl * 4 + r * G * 4 >= feat) continue;
      float* q = base + r * G * 4;
      const float o0 = q[0], o1 = q[1], o2 = q[2], o3 = q[3];
      q[0] = o0 + acc[r].x, q[1] = o1 + acc[r].y, q[2] = o2 + acc[r].z, q[3] = o3 + acc[r].w;
    }
    return;
  }
  if (!atomic) {
    float* base = C + row * feat + gl * 4;
#pragma unroll
    for (int r = 0; r < REP; ++r) {
      if (gl * 4 + r * G * 4 >= feat) continue;  // feat below 4*G*REP: this lane's float4 is padding
      float* q = base + r * G * 4;
      __builtin_nontemporal_store(acc[r].x, q);
      __builtin_nontemporal_store(acc[r].y, q + 1);
      __builtin_nontemporal_store(acc[r].z, q + 2);
      __builtin_nontemporal_store(acc[r].w, q + 3);
    }
    return;
  }
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int r = 0; r < REP; ++r) *reinterpret_cast<float4*>(stage + (r * kWave + lane) * 4) = acc[r];
  __builtin_amdgcn_wave_barrier();
  float* base = C + row * feat + gl;
#pragma unroll
  for (int r = 0; r < REP; ++r) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float v = stage[(r * kWave + g * G) * 4 + k * G + gl];
      if (r * G * 4 + k * G + gl < feat)
        __hip_atomic_fetch_add(base + r * G * 4 + k * G, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// ----------------------------------------------------------------------------- CSR SpMM
// Partial sum of A[p] * B[indices[p], :] over p in [start, end) for one wavefront: the 64/G lane
// groups take the nonzeros round-robin; the caller combines the groups.
// INDIRECT: A is an array of addresses of the values (the merged rows of a hyb plan, whose values
// stay in the caller's bucket arrays), and nonzeros whose value is 0 -- ELL padding -- fetch no row.
template <int G, int REP, bool INDIRECT = false>
__device__ __forceinline__ void csr_accumulate(float4 (&acc)[REP], int start, int end, int feat,
                                               const float* __restrict__ A, const float* __restrict__ B,
                                               const int32_t* __restrict__ indices, int lane) {
  constexpr int NG = kWave / G;
  constexpr int UNROLL = 4;
  const int g = lane / G, gl = lane % G;
  for (int base = start; base < end; base += kWave) {
    const int p = base + lane;
    const int my_col = p < end ? __builtin_nontemporal_load(indices + p) : 0;
    float my_val = 0.f;
    if (p < end) {
      if constexpr (INDIRECT)
        my_val = *__builtin_nontemporal_load(reinterpret_cast<const float* const*>(A) + p);
      else
        my_val = __builtin_nontemporal_load(A + p);
    }
    const int cnt = min(kWave, end - base);
    for (int j0 = 0; j0 < cnt; j0 += NG * UNROLL) {
      float4 x[UNROLL][REP];
      float v[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int j = j0 + u * NG + g;  // < 64 because NG*UNROLL divides 64
        const int col = __shfl(my_col, j, kWave);
        v[u] = __shfl(my_val, j, kWave);
        const float* bp = B + (int64_t)col * feat + gl * 4;
#pragma unroll
        for (int r = 0; r < REP; ++r)
          x[u][r] = (j < cnt && gl * 4 + r * G * 4 < feat && (!INDIRECT || v[u] != 0.f)) ? ld4(bp + r * G * 4)
                                                                                          : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u)
#pragma unroll
        for (int r = 0; r < REP; ++r) fma4(acc[r], v[u], x[u][r]);
    }
  }
}

// Rows with more nonzeros than this are not left to a single wavefront (a 17k-entry hub row
// costs one wavefront milliseconds): the row kernel only clears them and csr_long_rows_kernel,
// launched after it, adds them up in pieces of kLongPiece nonzeros.  64 rather than 256: the
// piece kernel keeps every lane busy whatever the row, a wavefront on a row of its own does not
// (169 k-node power-law graph, half of its nonzeros in rows above 256: 46 -> 41 us at 32 features,
// 223 -> 203 us at 256; 2.45 M-node graph, 128 features: 5.05 -> 5.01 ms; 32 is slower again).
constexpr int kLongRow = 64;
constexpr int kLongPiece = 256;

// One wavefront per row.  With split_long the rows above kLongRow are zero-filled here.
template <int G, int REP, bool INDIRECT = false>
__global__ __launch_bounds__(256) void csr_spmm_kernel(int m, int feat, int split_long,
                                                       const float* __restrict__ A,
                                                       const float* __restrict__ B,
                                                       float* __restrict__ C,
                                                       const int32_t* __restrict__ indptr,
                                                       const int32_t* __restrict__ indices) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= m) return;
  const int g = lane / G;
  const int start = indptr[row], end = indptr[row + 1];
  float4 acc[REP];
#pragma unroll
  for (int r = 0; r < REP; ++r) acc[r] = make_float4(0.f, 0.f, 0.f, 0.f);
  if (!(split_long && end - start > kLongRow))
    csr_accumulate<G, REP, INDIRECT>(acc, start, end, feat, A, B, indices, lane);
  reduce_groups<G, REP>(acc, kWave);
  if constexpr (INDIRECT) {
    // merged rows of a hyb plan: the operator adds to C, as its buckets do; this wavefront is the
    // row's only writer in this launch, long rows are left to csr_long_rows_kernel altogether
    if (end - start > kLongRow) return;
    if (g == 0) write_row<G, REP>(C, row, feat, lane, acc, 2, nullptr);
  } else {
    if (g == 0) write_row<G, REP>(C, row, feat, lane, acc, 0, nullptr);
  }
}

// Feature rows narrower than a wavefront (G < 64 lanes): a wavefront owns 64 / G consecutive rows
// of the matrix, one per lane group.  A group walks its own row -- G nonzeros per index load, up
// to eight gathers in flight per lane -- and stores it without any exchange between lanes; the
// wavefront writes 64 / G consecutive rows of C.  With one wavefront per row (the kernel above) a
// row of seven nonzeros at 32 features keeps one lane group in eight busy for one step and still
// pays the index round trip, the cross-lane sum and the store.  Rows of more than 2 * G nonzeros
// would hold the other groups up: the wavefront takes those one by one afterwards, all groups
// sharing the row as in the kernel above (and leaves rows above kLongRow zero-filled for
// csr_long_rows_kernel when split_long is set).
template <int G>
__global__ __launch_bounds__(256) void csr_spmm_rows_kernel(int m, int feat, int split_long,
                                                            const float* __restrict__ A,
                                                            const float* __restrict__ B,
                                                            float* __restrict__ C,
                                                            const int32_t* __restrict__ indptr,
                                                            const int32_t* __restrict__ indices) {
  constexpr int NG = kWave / G;
  constexpr int CH = G < 8 ? G : 8;  // gathers in flight per lane
  constexpr int kGroupRow = 2 * G;   // longest row a lane group takes alone (1 to 4 * G measure the same)
  const int lane = threadIdx.x & 63;
  const int g = lane / G, gl = lane % G;
  const int64_t row0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * NG;
  if (row0 >= m) return;
  const int64_t row = row0 + g;
  int start = 0, end = 0;
  if (row < m) start = indptr[row], end = indptr[row + 1];
  const bool alone = end - start <= kGroupRow;
  const int my_end = alone ? end : start;
  const bool chunk_live = gl * 4 < feat;
  const float* Bl = B + gl * 4;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int base = start; base < my_end; base += G) {
    const int p = base + gl;
    const int my_col = p < my_end ? __builtin_nontemporal_load(indices + p) : 0;
    const float my_val = p < my_end ? __builtin_nontemporal_load(A + p) : 0.f;
    const int cnt = min(G, my_end - base);
#pragma unroll 1
    for (int c = 0; c < cnt; c += CH) {
      float4 x[CH];
      float v[CH];
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        const int sl = g * G + c + u;  // a lane of this group: it is in this loop as well
        const int col = __shfl(my_col, sl, kWave);
        v[u] = __shfl(my_val, sl, kWave);
        x[u] = (c + u < cnt && chunk_live) ? ld4(Bl + (int64_t)col * feat) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < CH; ++u) fma4(acc, v[u], x[u]);
    }
  }
  if (row < m && alone && chunk_live) {
    float* q = C + row * feat + gl * 4;
    __builtin_nontemporal_store(acc.x, q);
    __builtin_nontemporal_store(acc.y, q + 1);
    __builtin_nontemporal_store(acc.z, q + 2);
    __builtin_nontemporal_store(acc.w, q + 3);
  }
  // the longer rows, one after the other, by the whole wavefront
  uint64_t todo = __ballot(row < m && !alone && gl == 0);
  while (todo) {
    const int src = __ffsll((long long)todo) - 1;
    todo &= todo - 1;
    const int s = __shfl(start, src, kWave), e = __shfl(end, src, kWave);
    float4 sum[1] = {make_float4(0.f, 0.f, 0.f, 0.f)};
    if (!(split_long && e - s > kLongRow)) csr_accumulate<G, 1>(sum, s, e, feat, A, B, indices, lane);
    reduce_groups<G, 1>(sum, kWave);
    if (g == 0) write_row<G, 1>(C, row0 + src / G, feat, lane, sum, 0, nullptr);
  }
}

// One wavefront per kLongPiece consecutive nonzeros: the parts of rows longer than kLongRow that
// fall into the piece are summed and added to C (cleared by csr_spmm_kernel) with atomics.
// Pieces that touch no long row -- nearly all of them -- end after looking at their rows.
template <int G, int REP, bool INDIRECT = false>
__global__ __launch_bounds__(256) void csr_long_rows_kernel(int m, int feat, int64_t first, int64_t nnz,
                                                            const float* __restrict__ A,
                                                            const float* __restrict__ B,
                                                            float* __restrict__ C,
                                                            const int32_t* __restrict__ indptr,
                                                            const int32_t* __restrict__ indices) {
  __shared__ float stage_all[4][kWave * 4 * REP];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t p0 = first + ((int64_t)blockIdx.x * 4 + wave) * kLongPiece;
  const int64_t end_all = first + nnz;
  if (p0 >= end_all) return;
  const int64_t p1 = min(end_all, p0 + kLongPiece);
  const int ra = stir::wave_last_row(indptr, m, p0, lane);
  const int rb = stir::wave_last_row(indptr, m, p1 - 1, lane);
  const int g = lane / G;
  for (int r0 = ra; r0 <= rb; r0 += kWave) {
    const int r = r0 + lane;
    int rs = 0, re = 0;
    if (r <= rb && r < m) rs = indptr[r], re = indptr[r + 1];
    uint64_t todo = __ballot(re - rs > kLongRow);
    while (todo) {
      const int src = __ffsll((long long)todo) - 1;
      todo &= todo - 1;
      const int row = r0 + src;
      const int64_t s = max((int64_t)__shfl(rs, src, kWave), p0);
      const int64_t e = min((int64_t)__shfl(re, src, kWave), p1);
      float4 acc[REP];
#pragma unroll
      for (int q = 0; q < REP; ++q) acc[q] = make_float4(0.f, 0.f, 0.f, 0.f);
      csr_accumulate<G, REP, INDIRECT>(acc, (int)s, (int)e, feat, A, B, indices, lane);
      reduce_groups<G, REP>(acc, kWave);
      if (g == 0) write_row<G, REP>(C, row, feat, lane, acc, true, stage_all[wave]);
    }
  }
}

// Any feature width: one wavefront per row, lane l owns features l, l+64, ...
__global__ __launch_bounds__(256) void csr_spmm_generic_kernel(int m, int feat, const float* __restrict__ A,
                                                               const float* __restrict__ B,
                                                               float* __restrict__ C,
                                                               const int32_t* __restrict__ indptr,
                                                               const int32_t* __restrict__ indices) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= m) return;
  const int start = indptr[row], end = indptr[row + 1];
  for (int f = lane; f < feat; f += kWave) {
    float acc = 0.f;
    for (int p = start; p < end; ++p) acc = fmaf(A[p], B[(int64_t)indices[p] * feat + f], acc);
    C[(int64_t)row * feat + f] = acc;
  }
}

// ----------------------------------------------------------------------------- hyb SpMM
// Slot-tile mode (power-of-two width <= 64): a wavefront owns 64 consecutive ELL slots,
// i.e. 64/width whole ELL rows.  Lane group g owns slots [g*G, g*G+G) of the tile.
template <int G, int REP, int LOG2W>
__device__ __forceinline__ void hyb_slot_tile(const HybBucket& bk, int64_t t, int feat,
                                              const float* __restrict__ B, float* __restrict__ C,
                                              int lane, float* stage) {
  constexpr int W = 1 << LOG2W;
  constexpr int CH = G < 8 ? G : 8;  // gathers in flight per lane
  const int g = lane / G, gl = lane % G;
  const int64_t slot0 = t * kWave;
  const int64_t nslots = bk.nrows << LOG2W;
  const int64_t s = slot0 + lane;
  // index and weight arrays are read once: non-temporal, so they do not displace rows of B
  const int my_col = s < nslots ? __builtin_nontemporal_load(bk.cols + s) : 0;
  const float my_val = s < nslots ? __builtin_nontemporal_load(bk.A + s) : 0.f;
  constexpr int ROWS = kWave >> LOG2W;  // ELL rows per tile
  const int64_t row0 = slot0 >> LOG2W;
  int my_row = -1;
  if (lane < ROWS && row0 + lane < bk.nrows) my_row = bk.rows[row0 + lane];
  const int atomic = bk.atomic;

  float4 acc[REP];
#pragma unroll
  for (int r = 0; r < REP; ++r) acc[r] = make_float4(0.f, 0.f, 0.f, 0.f);

  // The chunk loop stays rolled so that only CH gathers (not all G) are live at once.
#pragma unroll 1
  for (int c = 0; c < G; c += CH) {
    float4 x[CH][REP];
    float v[CH];
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      const int sl = g * G + c + u;
      const int col = __shfl(my_col, sl, kWave);
      v[u] = __shfl(my_val, sl, kWave);
      const float* bp = B + (int64_t)col * feat + gl * 4;
      // a slot of weight zero (padding) adds nothing: its row of B is not fetched
#pragma unroll
      for (int r = 0; r < REP; ++r)
        x[u][r] = (v[u] != 0.f && gl * 4 + r * G * 4 < feat) ? ld4(bp + r * G * 4)
                                                             : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < CH; ++u) {
#pragma unroll
      for (int r = 0; r < REP; ++r) fma4(acc[r], v[u], x[u][r]);
      if constexpr (W <= G) {
        // end of an ELL row inside this lane group; for W <= CH this folds to a constant
        if (((c + u + 1) & (W - 1)) == 0) {
          const int out_row = __shfl(my_row, (g * G + c + u) >> LOG2W, kWave);
          if (out_row >= 0) write_row<G, REP>(C, out_row, feat, lane, acc, atomic, stage);
#pragma unroll
          for (int r = 0; r < REP; ++r) acc[r] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
    }
  }
  if constexpr (W > G) {
    // an ELL row spans W/G lane groups: combine them, the first group of the row writes
    reduce_groups<G, REP>(acc, W);
    const int out_row = __shfl(my_row, (g * G) >> LOG2W, kWave);
    if (((g * G) & (W - 1)) == 0 && out_row >= 0)
      write_row<G, REP>(C, out_row, feat, lane, acc, atomic, stage);
  }
}

// Row mode (any width): a wavefront owns one ELL row, or one kRowChunk-slot piece of it when
// the bucket accumulates, and walks it 64 slots at a time.
template <int G, int REP>
__device__ __forceinline__ void hyb_row_tile(const HybBucket& bk, int64_t t, int feat,
                                             const float* __restrict__ B, float* __restrict__ C,
                                             int lane, float* stage) {
  constexpr int CH = G < 8 ? G : 8;
  const int g = lane / G, gl = lane % G;
  const int w = bk.width;
  const int64_t row = bk.chunks > 1 ? t / bk.chunks : t;
  const int s_begin = bk.chunks > 1 ? (int)(t % bk.chunks) * kRowChunk : 0;
  const int s_end = bk.chunks > 1 ? min(w, s_begin + kRowChunk) : w;
  const int32_t* cols = bk.cols + row * w;
  const float* vals = bk.A + row * w;
  float4 acc[REP];
#pragma unroll
  for (int r = 0; r < REP; ++r) acc[r] = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int c0 = s_begin; c0 < s_end; c0 += kWave) {
    const int s = c0 + lane;
    const int my_col = s < s_end ? __builtin_nontemporal_load(cols + s) : 0;
    const float my_val = s < s_end ? __builtin_nontemporal_load(vals + s) : 0.f;
#pragma unroll 1
    for (int c = 0; c < G; c += CH) {
      float4 x[CH][REP];
      float v[CH];
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        const int sl = g * G + c + u;
        const int col = __shfl(my_col, sl, kWave);
        v[u] = __shfl(my_val, sl, kWave);  // zero beyond s_end and on padding
        const float* bp = B + (int64_t)col * feat + gl * 4;
#pragma unroll
        for (int r = 0; r < REP; ++r)
          x[u][r] = (v[u] != 0.f && gl * 4 + r * G * 4 < feat) ? ld4(bp + r * G * 4)
                                                             : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < CH; ++u)
#pragma unroll
        for (int r = 0; r < REP; ++r) fma4(acc[r], v[u], x[u][r]);
    }
  }
  reduce_groups<G, REP>(acc, kWave);
  if (g == 0) write_row<G, REP>(C, bk.rows[row], feat, lane, acc, bk.atomic, stage);
}

__device__ __forceinline__ int find_bucket(const HybBucket* __restrict__ table, int nb,
                                           int64_t tile) {
  int lo = 0, hi = nb - 1;  // largest k with tile_begin[k] <= tile
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[mid].tile_begin <= tile)
      lo = mid;
    else
      hi = mid - 1;
  }
  return lo;
}

template <int G, int REP>
__global__ __launch_bounds__(256) void hyb_spmm_kernel(const HybBucket* __restrict__ table, int nb,
                                                       int64_t tile_base, int64_t tile_end, int feat,
                                                       const float* __restrict__ B,
                                                       float* __restrict__ C) {
  __shared__ float stage_all[4][kWave * 4 * REP];  // per-wavefront staging for atomic rows
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  float* stage = stage_all[wave];
  const int64_t tile = tile_base + (int64_t)blockIdx.x * 4 + wave;
  if (tile >= tile_end) return;
  const int k = find_bucket(table, nb, tile);
  const HybBucket bk = table[k];
  const int64_t t = tile - bk.tile_begin;
  switch (bk.log2w) {
    case 0: hyb_slot_tile<G, REP, 0>(bk, t, feat, B, C, lane, stage); break;
    case 1: hyb_slot_tile<G, REP, 1>(bk, t, feat, B, C, lane, stage); break;
    case 2: hyb_slot_tile<G, REP, 2>(bk, t, feat, B, C, lane, stage); break;
    case 3: hyb_slot_tile<G, REP, 3>(bk, t, feat, B, C, lane, stage); break;
    case 4: hyb_slot_tile<G, REP, 4>(bk, t, feat, B, C, lane, stage); break;
    case 5: hyb_slot_tile<G, REP, 5>(bk, t, feat, B, C, lane, stage); break;
    case 6: hyb_slot_tile<G, REP, 6>(bk, t, feat, B, C, lane, stage); break;
    default: hyb_row_tile<G, REP>(bk, t, feat, B, C, lane, stage); break;
  }
}

// Any feature width: one wavefront per ELL row, lane l owns features l, l+64, ...
__global__ __launch_bounds__(256) void hyb_spmm_generic_kernel(const HybBucket* __restrict__ table,
                                                               int nb, int64_t total_rows, int feat,
                                                               const float* __restrict__ B,
                                                               float* __restrict__ C) {
  const int lane = threadIdx.x & 63;
  const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tile >= total_rows) return;
  const int k = find_bucket(table, nb, tile);
  const HybBucket bk = table[k];
  const int64_t t = tile - bk.tile_begin;
  const int w = bk.width;
  const int64_t out_row = bk.rows[t];
  for (int f = lane; f < feat; f += kWave) {
    float acc = 0.f;
    for (int s = 0; s < w; ++s)
      acc = fmaf(bk.A[t * w + s], B[(int64_t)bk.cols[t * w + s] * feat + f], acc);
    float* dst = C + out_row * feat + f;
    if (bk.atomic)
      __hip_atomic_fetch_add(dst, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
      *dst = acc;
  }
}

// Marks (mark = 1) or looks up (mark = 0) the output rows of one bucket in a bitmap with one bit
// per output row.  flags[0] is raised when a row is met that is already marked, flags[1] when a
// row id lies outside [0, m).
__global__ __launch_bounds__(256) void hyb_mark_rows_kernel(const int32_t* __restrict__ rows, int64_t nrows,
                                                            int32_t m, uint32_t* __restrict__ bitmap, int mark,
                                                            int32_t* __restrict__ flags) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nrows) return;
  const int32_t r = rows[i];
  if (r < 0 || r >= m) {
    flags[1] = 1;
    return;
  }
  const uint32_t bit = 1u << (r & 31);
  const uint32_t seen = mark ? atomicOr(bitmap + (r >> 5), bit) : bitmap[r >> 5];
  if (seen & bit) flags[0] = 1;
}

// ---- merged rows (plans with more column partitions than run as phases)
// With p column partitions an output row is the sum of up to p ELL rows, each in another bucket:
// added with atomics that is p read-modify-writes of the row through the L2 atomic units
// (config 3 with the reference's 16 partitions: 39 M ELL rows of mostly one or two slots, 20 GB of
// atomic traffic).  Such a plan lists, once, the slots of every output row one after the other --
// their column ids and the addresses of their values, which stay in the caller's arrays -- and
// its launches run the CSR row kernels over that list: every row is read and written once (the
// operator adds to C, like its buckets would).

// count[r] += width for the output row r of every ELL row of one bucket; flags[1] when a row id
// lies outside [0, m)
__global__ __launch_bounds__(256) void hyb_count_slots_kernel(const int32_t* __restrict__ rows, int64_t nrows,
                                                              int32_t width, int32_t m, int32_t* __restrict__ count,
                                                              int32_t* __restrict__ flags) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nrows) return;
  const int32_t r = rows[i];
  if (r < 0 || r >= m) {
    flags[1] = 1;
    return;
  }
  atomicAdd(count + r, width);
}

// The slots of ELL row i of one bucket go to the next `width` places of its output row's list
// (cursor[r] starts at the row's first place).
__global__ __launch_bounds__(256) void hyb_place_slots_kernel(const int32_t* __restrict__ rows,
                                                              const int32_t* __restrict__ cols,
                                                              const float* __restrict__ A, int64_t nrows,
                                                              int32_t width, int32_t* __restrict__ cursor,
                                                              int32_t* __restrict__ merged_cols,
                                                              const float** __restrict__ merged_vals) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nrows) return;
  const int32_t r = rows[i];  // in range: hyb_count_slots_kernel has looked at it
  const int32_t at = atomicAdd(cursor + r, width);
  const int64_t first = i * width;
  for (int32_t j = 0; j < width; ++j) {
    merged_cols[at + j] = cols[first + j];
    merged_vals[at + j] = A + first + j;
  }
}

// Copies `count` bucket descriptors, handed over as a kernel argument, to dst[first ...]: how the
// entry point that allocates nothing gets its descriptor tables into device memory without a
// host-to-device copy.
constexpr int kTableChunk = 32;
struct HybTableChunk {
  HybBucket b[kTableChunk];
};
__global__ __launch_bounds__(256) void hyb_table_fill_kernel(HybTableChunk chunk, int count,
                                                             HybBucket* __restrict__ dst) {
  constexpr int kWords = sizeof(HybBucket) / 4;
  const uint32_t* src = reinterpret_cast<const uint32_t*>(&chunk);
  uint32_t* out = reinterpret_cast<uint32_t*>(dst);
  for (int i = threadIdx.x; i < count * kWords; i += 256) out[i] = src[i];
}

// 0..5: lane groups of 4, 8, 16, 32, 64 lanes and 64 lanes x 2 float4 cover feat; -1: generic kernel
int vector_class(int feat) {
  if (feat % 4 != 0 || feat > 512) return -1;
  int c = 0;
  while ((16 << c) < feat) ++c;
  return c;
}

int log2_exact(int64_t x) {
  int l = 0;
  while ((int64_t(1) << l) < x) ++l;
  return l;
}

// Whether the partitions may run one after the other with plain read-modify-write adds in all but
// their last bucket: inside every partition an output row must belong to one ELL row of one
// non-last bucket, or to ELL rows of the last bucket only.  ColumnPartHyb output always does;
// arrays built by other means may not, and the reference adds those atomically
// (examples/spmm/bench_spmm.py:170-177).  Reads the row arrays as they are now (after a device
// synchronisation).  *ok = 0 when some row is shared; an error when a row id is out of range.
int phases_have_single_writers(int32_t m, int num_col_parts, int num_buckets, const int64_t* nrows,
                               const int32_t* const* d_rows, bool* ok) {
  *ok = true;
  if (m == 0) return 0;
  const size_t words = ((size_t)m + 31) / 32;
  uint32_t* d_bitmap = nullptr;
  for (int k = 0; k < num_col_parts * num_buckets; ++k)
    STIR_REQUIRE(stir::ceil_div(nrows[k], 256) < (int64_t(1) << 31), "hyb_plan_create: bucket %d too large", k);
  STIR_HIP(hipDeviceSynchronize());
  STIR_HIP(hipMalloc(reinterpret_cast<void**>(&d_bitmap), (words + 2) * sizeof(uint32_t)));
  int32_t* d_flags = reinterpret_cast<int32_t*>(d_bitmap + words);
  hipError_t e = hipMemset(d_bitmap, 0, (words + 2) * sizeof(uint32_t));
  for (int p = 0; p < num_col_parts && e == hipSuccess; ++p) {
    bool any = false;
    for (int b = 0; b < num_buckets; ++b) {
      const int k = p * num_buckets + b;
      if (nrows[k] == 0) continue;
      hipLaunchKernelGGL(hyb_mark_rows_kernel, dim3((unsigned)stir::ceil_div(nrows[k], 256)), dim3(256), 0, 0,
                         d_rows[k], nrows[k], m, d_bitmap, b != num_buckets - 1 ? 1 : 0, d_flags);
      any = true;
    }
    if (any && p + 1 < num_col_parts) e = hipMemsetAsync(d_bitmap, 0, words * sizeof(uint32_t), 0);
  }
  int32_t flags[2] = {0, 0};
  if (e == hipSuccess) e = hipGetLastError();
  if (e == hipSuccess) e = hipMemcpy(flags, d_flags, sizeof(flags), hipMemcpyDeviceToHost);
  (void)hipFree(d_bitmap);
  if (e != hipSuccess) return stir::fail("hyb_plan_create: %s", hipGetErrorString(e));
  STIR_REQUIRE(flags[1] == 0, "hyb_plan_create: a row index lies outside [0, %d)", m);
  *ok = flags[0] == 0;
  return 0;
}

}  // namespace

constexpr int kMaxPhases = 4;
// With 2 to kMaxPhases partitions a plan holds both forms and the launch picks by feature width:
// phases below this width, merged rows from it on.  Measured on the 169k-node graph with two
// partitions (CSR row-split 39 / 64 / 112 / 203 us at 32 / 64 / 128 / 256 features): phases
// 44 / 60 / 119 / 254 us, merged rows 81 / 98 / 136 / 235 us -- a phase reads and writes C once
// more, which at 256 features (173 MB each way) costs more than the merged list's indirect loads.
constexpr int kMergedFromFeat = 256;
constexpr size_t kMergedOptionalBytes = size_t(1) << 30;  // ... when the slot list stays below this

namespace {

// Host image of a hyb operator: the bucket descriptors in launch order, once with tile_begin
// counted in wave tiles (vectorised kernel) and once in ELL rows (generic kernel).
struct HybTables {
  std::vector<HybBucket> tiles, rows;
  int64_t total_tiles = 0, total_rows = 0;
  // first table entry / first wave tile of every launch of the vectorised kernel, and the ends
  std::vector<int> phase_bucket;
  std::vector<int64_t> phase_tile;
};

int check_hyb_arguments(const char* who, int32_t m, int32_t n, int32_t num_col_parts, int32_t num_buckets,
                        const int32_t* bucket_widths, const int64_t* nrows, const float* const* d_A,
                        const int32_t* const* d_rows, const int32_t* const* d_cols) {
  STIR_REQUIRE(m >= 0 && n >= 0 && num_col_parts > 0 && num_buckets > 0, "%s: bad sizes", who);
  STIR_REQUIRE(bucket_widths && nrows && d_A && d_rows && d_cols, "%s: null pointer argument", who);
  for (int b = 0; b < num_buckets; ++b)
    STIR_REQUIRE(bucket_widths[b] > 0, "%s: bucket width %d is not positive", who, bucket_widths[b]);
  const int total = num_col_parts * num_buckets;
  for (int k = 0; k < total; ++k) {
    STIR_REQUIRE(nrows[k] >= 0, "%s: nrows[%d] is negative", who, k);
    STIR_REQUIRE(nrows[k] == 0 || (d_A[k] && d_rows[k] && d_cols[k]), "%s: bucket %d has rows but a null array",
                 who, k);
  }
  return 0;
}

// phased: the partitions run one after the other (one launch each) and all but the last bucket of
// a partition add with a plain read-modify-write.
void make_hyb_tables(int32_t num_col_parts, int32_t num_buckets, const int32_t* bucket_widths,
                     const int64_t* nrows, const float* const* d_A, const int32_t* const* d_rows,
                     const int32_t* const* d_cols, bool phased, HybTables* out) {
  const int total = num_col_parts * num_buckets;
  // Widest buckets first: their wavefronts run longest, so they are dispatched first and the
  // launch does not end on a tail of hub rows.
  std::vector<int> order;
  for (int k = 0; k < total; ++k)
    if (nrows[k] > 0) order.push_back(k);
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) {
    if (phased && a / num_buckets != b / num_buckets) return a / num_buckets < b / num_buckets;
    return bucket_widths[a % num_buckets] > bucket_widths[b % num_buckets];
  });
  const int nk = (int)order.size();
  out->tiles.resize(nk);
  out->rows.resize(nk);
  int64_t tiles = 0, rows = 0;
  for (int q = 0; q < nk; ++q) {
    const int k = order[q];
    const int b = k % num_buckets;
    const int w = bucket_widths[b];
    HybBucket e;
    e.A = d_A[k];
    e.rows = d_rows[k];
    e.cols = d_cols[k];
    e.nrows = nrows[k];
    e.width = w;
    const int fused_mode = (num_col_parts > 1 || b == num_buckets - 1) ? 1 : 0;
    e.atomic = (phased && b != num_buckets - 1) ? 2 : fused_mode;
    const bool slot_mode = stir::is_pow2(w) && w <= kWave;
    e.log2w = slot_mode ? log2_exact(w) : -1;
    e.chunks = (!slot_mode && e.atomic == 1 && w > kRowChunk) ? (int)stir::ceil_div(w, kRowChunk) : 1;
    e.tile_begin = tiles;
    out->tiles[q] = e;
    if (phased && (q == 0 || k / num_buckets != order[q - 1] / num_buckets)) {
      out->phase_bucket.push_back(q);
      out->phase_tile.push_back(tiles);
    }
    tiles += slot_mode ? stir::ceil_div(nrows[k] * w, kWave) : nrows[k] * e.chunks;
    e.tile_begin = rows;
    e.chunks = 1;
    e.atomic = fused_mode;  // the generic kernel runs all partitions in one launch
    out->rows[q] = e;
    rows += nrows[k];
  }
  if (!phased) out->phase_bucket.push_back(0), out->phase_tile.push_back(0);
  out->phase_bucket.push_back(nk);
  out->phase_tile.push_back(tiles);
  out->total_tiles = tiles;
  out->total_rows = rows;
}

// The merged rows of a plan (see hyb_count_slots_kernel): CSR over all slots of the operator.
struct MergedRows {
  int32_t* slot_ptr = nullptr;       // m + 1
  int32_t* cols = nullptr;           // slots
  const float** vals = nullptr;      // slots: addresses inside the caller's value arrays
  int64_t slots = 0;
  void release() {
    if (slot_ptr) (void)hipFree(slot_ptr);
    if (cols) (void)hipFree(cols);
    if (vals) (void)hipFree(vals);
    slot_ptr = cols = nullptr;
    vals = nullptr;
    slots = 0;
  }
};

// Builds the merged rows from the bucket arrays as they are now (synchronises the device).
// *built = false, and nothing allocated, when the list would not fit 31-bit offsets or a quarter
// of the free device memory.
int build_merged_rows(int32_t m, int total_buckets, int num_buckets, const int32_t* bucket_widths,
                      const int64_t* nrows, const float* const* d_A, const int32_t* const* d_rows,
                      const int32_t* const* d_cols, MergedRows* out, bool* built) {
  *built = false;
  int64_t slots = 0;
  for (int k = 0; k < total_buckets; ++k) {
    STIR_REQUIRE(stir::ceil_div(nrows[k], 256) < (int64_t(1) << 31), "hyb_plan_create: bucket %d too large", k);
    slots += nrows[k] * bucket_widths[k % num_buckets];
  }
  if (m == 0 || slots == 0 || slots >= (int64_t(1) << 31)) return 0;
  size_t free_bytes = 0, total_bytes = 0;
  STIR_HIP(hipMemGetInfo(&free_bytes, &total_bytes));
  const size_t need = size_t(slots) * 12 + size_t(m + 1) * 12;
  if (need > free_bytes / 4) return 0;
  STIR_HIP(hipDeviceSynchronize());
  MergedRows mr;
  int32_t *count = nullptr, *flags = nullptr;
  void* tmp = nullptr;
  size_t tmp_bytes = 0;
  auto cleanup = [&]() {
    if (count) (void)hipFree(count);
    if (tmp) (void)hipFree(tmp);
  };
  hipError_t e = hipMalloc(reinterpret_cast<void**>(&count), sizeof(int32_t) * (size_t(m) + 3));
  if (e == hipSuccess) e = hipMemset(count, 0, sizeof(int32_t) * (size_t(m) + 3));
  if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&mr.slot_ptr), sizeof(int32_t) * (size_t(m) + 1));
  if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&mr.cols), sizeof(int32_t) * size_t(slots));
  if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&mr.vals), sizeof(float*) * size_t(slots));
  if (e == hipSuccess)
    e = hipcub::DeviceScan::ExclusiveSum(nullptr, tmp_bytes, (const int32_t*)nullptr, (int32_t*)nullptr, m + 1, 0);
  if (e == hipSuccess) e = hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 16);
  if (e != hipSuccess) {
    cleanup();
    mr.release();
    return stir::fail("hyb_plan_create: %s", hipGetErrorString(e));
  }
  flags = count + m + 1;  // count[m] stays 0: the scan turns it into the number of slots
  for (int k = 0; k < total_buckets; ++k)
    if (nrows[k] > 0)
      hipLaunchKernelGGL(hyb_count_slots_kernel, dim3((unsigned)stir::ceil_div(nrows[k], 256)), dim3(256), 0, 0,
                         d_rows[k], nrows[k], bucket_widths[k % num_buckets], m, count, flags);
  int32_t h_flags[2] = {0, 0};
  e = hipGetLastError();
  if (e == hipSuccess) e = hipMemcpy(h_flags, flags, sizeof(h_flags), hipMemcpyDeviceToHost);
  if (e == hipSuccess && h_flags[1] == 0) {
    e = hipcub::DeviceScan::ExclusiveSum(tmp, tmp_bytes, (const int32_t*)count, mr.slot_ptr, m + 1, 0);
    // the counts become the cursors of the placement
    if (e == hipSuccess)
      e = hipMemcpyAsync(count, mr.slot_ptr, sizeof(int32_t) * size_t(m), hipMemcpyDeviceToDevice, 0);
    for (int k = 0; k < total_buckets && e == hipSuccess; ++k)
      if (nrows[k] > 0)
        hipLaunchKernelGGL(hyb_place_slots_kernel, dim3((unsigned)stir::ceil_div(nrows[k], 256)), dim3(256), 0, 0,
                           d_rows[k], d_cols[k], d_A[k], nrows[k], bucket_widths[k % num_buckets], count, mr.cols,
                           mr.vals);
    if (e == hipSuccess) e = hipGetLastError();
    if (e == hipSuccess) e = hipDeviceSynchronize();
  }
  cleanup();
  if (e != hipSuccess || h_flags[1] != 0) {
    mr.release();
    if (e != hipSuccess) return stir::fail("hyb_plan_create: %s", hipGetErrorString(e));
    return stir::fail("hyb_plan_create: a row index lies outside [0, %d)", m);
  }
  mr.slots = slots;
  *out = mr;
  *built = true;
  return 0;
}

// Launches the CSR row kernels over the merged rows.  feat must have a vector class.
int launch_merged(const MergedRows& mr, int32_t m, int32_t feat, const float* d_B, float* d_C, hipStream_t st) {
  dim3 grid((unsigned)stir::ceil_div(m, 4)), block(256);
  dim3 pieces((unsigned)stir::ceil_div(stir::ceil_div(mr.slots, kLongPiece), 4));
  const float* vals = reinterpret_cast<const float*>(mr.vals);
#define STIR_MERGED(G, REP)                                                                                   \
  {                                                                                                           \
    hipLaunchKernelGGL((csr_spmm_kernel<G, REP, true>), grid, block, 0, st, m, feat, 1, vals, d_B, d_C,       \
                       mr.slot_ptr, mr.cols);                                                                 \
    hipLaunchKernelGGL((csr_long_rows_kernel<G, REP, true>), pieces, block, 0, st, m, feat, (int64_t)0, mr.slots, \
                       vals, d_B, d_C, mr.slot_ptr, mr.cols);                                                 \
  }
  switch (vector_class(feat)) {
    case 0: STIR_MERGED(4, 1); break;
    case 1: STIR_MERGED(8, 1); break;
    case 2: STIR_MERGED(16, 1); break;
    case 3: STIR_MERGED(32, 1); break;
    case 4: STIR_MERGED(64, 1); break;
    case 5: STIR_MERGED(64, 2); break;
    default: return stir::fail("hyb_spmm: feat=%d has no vectorised kernel", feat);
  }
#undef STIR_MERGED
  STIR_LAUNCH_CHECK();
  return 0;
}

// Launches the kernels of a hyb operator whose descriptor tables are at d_tiles / d_rows.
int launch_hyb(const HybTables& t, const HybBucket* d_tiles, const HybBucket* d_rows, int32_t feat,
               const float* d_B, float* d_C, hipStream_t st) {
  const int nk = (int)t.tiles.size();
  dim3 block(256);
  STIR_REQUIRE(stir::ceil_div(t.total_tiles, 4) < (int64_t(1) << 31), "hyb_spmm: %lld tiles exceed one launch",
               (long long)t.total_tiles);
  // one launch per phase (a single one unless the partitions run one after the other)
#define STIR_HYB(G, REP)                                                                                    \
  for (size_t ph = 0; ph + 1 < t.phase_bucket.size(); ++ph) {                                               \
    const int64_t t0 = t.phase_tile[ph], t1 = t.phase_tile[ph + 1];                                          \
    if (t1 == t0) continue;                                                                                 \
    hipLaunchKernelGGL((hyb_spmm_kernel<G, REP>), dim3((unsigned)stir::ceil_div(t1 - t0, 4)), block, 0, st,  \
                       d_tiles + t.phase_bucket[ph], t.phase_bucket[ph + 1] - t.phase_bucket[ph], t0, t1,   \
                       feat, d_B, d_C);                                                                     \
  }
  switch (vector_class(feat)) {
    case 0: STIR_HYB(4, 1); break;
    case 1: STIR_HYB(8, 1); break;
    case 2: STIR_HYB(16, 1); break;
    case 3: STIR_HYB(32, 1); break;
    case 4: STIR_HYB(64, 1); break;
    case 5: STIR_HYB(64, 2); break;
    default: {
      const int64_t rb = stir::ceil_div(t.total_rows, 4);
      STIR_REQUIRE(rb < (int64_t(1) << 31), "hyb_spmm: %lld rows exceed one launch", (long long)t.total_rows);
      hipLaunchKernelGGL(hyb_spmm_generic_kernel, dim3((unsigned)rb), block, 0, st, d_rows, nk, t.total_rows,
                         feat, d_B, d_C);
    }
  }
#undef STIR_HYB
  STIR_LAUNCH_CHECK();
  return 0;
}

// Address of `scratch` on the current device, asked from the runtime once per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int static_scratch(HybBucket** out) {
  int dev = -1;
  STIR_HIP(hipGetDevice(&dev));
  STIR_REQUIRE(dev >= 0 && dev < kMaxDevices, "hyb_spmm_noalloc: device %d is not supported", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    STIR_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    STIR_REQUIRE(ptr, "hyb_spmm_noalloc: the scratch array has no address on device %d", dev);
    g_scratch_ptr[dev] = ptr;
  }
  *out = static_cast<HybBucket*>(g_scratch_ptr[dev]);
  return 0;
}

}  // namespace

struct stir_hyb_plan {
  int32_t m, n, num_col_parts, num_buckets;
  int device;
  HybTables tables;
  HybBucket* d_tables;  // tables.tiles followed by tables.rows
  bool merged;          // more partitions than run as phases: launches go over `rows`
  MergedRows rows;
};

extern "C" {

int stir_csr_spmm_f32(int32_t m, int32_t n, int32_t feat, int64_t nnz, const float* d_A,
                      const float* d_B, float* d_C, const int32_t* d_indptr,
                      const int32_t* d_indices, void* stream) {
  STIR_REQUIRE(m >= 0 && n >= 0 && feat > 0 && nnz >= 0, "csr_spmm: bad sizes m=%d n=%d feat=%d", m, n, feat);
  if (m == 0) return 0;
  STIR_REQUIRE(d_B && d_C && d_indptr && (nnz == 0 || (d_A && d_indices)), "csr_spmm: null pointer argument");
  hipStream_t st = static_cast<hipStream_t>(stream);
  dim3 grid((unsigned)stir::ceil_div(m, 4)), block(256);
  // Hub rows are split over many wavefronts by a second launch; a matrix this small cannot hold
  // a row long enough to matter against the extra launch.
  const int split_long = nnz >= (int64_t(1) << 18) ? 1 : 0;
  dim3 pieces((unsigned)stir::ceil_div(stir::ceil_div(nnz, kLongPiece), 4));
#define STIR_CSR(G, REP)                                                                                   \
  {                                                                                                        \
    hipLaunchKernelGGL((csr_spmm_kernel<G, REP>), grid, block, 0, st, m, feat, split_long, d_A, d_B, d_C,  \
                       d_indptr, d_indices);                                                               \
    if (split_long)                                                                                        \
      hipLaunchKernelGGL((csr_long_rows_kernel<G, REP>), pieces, block, 0, st, m, feat, (int64_t)0, nnz, d_A,   \
                         d_B, d_C, d_indptr, d_indices);                                                   \
  }
  // feature widths that are a multiple of 4 take the vectorised kernel with the smallest lane
  // group that covers them (lanes beyond feat / 4 idle); anything else the generic one
  // lane groups narrower than the wavefront: a lane group per row (csr_spmm_rows_kernel)
#define STIR_CSR_ROWS(G)                                                                                   \
  {                                                                                                        \
    const dim3 row_grid((unsigned)stir::ceil_div(m, 4 * (kWave / G)));                                     \
    hipLaunchKernelGGL((csr_spmm_rows_kernel<G>), row_grid, block, 0, st, m, feat, split_long, d_A, d_B,   \
                       d_C, d_indptr, d_indices);                                                          \
    if (split_long)                                                                                        \
      hipLaunchKernelGGL((csr_long_rows_kernel<G, 1>), pieces, block, 0, st, m, feat, (int64_t)0, nnz, d_A, \
                         d_B, d_C, d_indptr, d_indices);                                                   \
  }
  switch (vector_class(feat)) {
    case 0: STIR_CSR_ROWS(4); break;
    case 1: STIR_CSR_ROWS(8); break;
    case 2: STIR_CSR_ROWS(16); break;
    case 3:
      // two rows per wavefront pay when rows are short: config 2 (7 nonzeros per row) 125 -> 119 us,
      // config 3 (25 per row) 5.06 -> 5.14 ms
      if (nnz < 16 * (int64_t)m) STIR_CSR_ROWS(32) else STIR_CSR(32, 1);
      break;
    case 4: STIR_CSR(64, 1); break;
    case 5: STIR_CSR(64, 2); break;
    default:
      hipLaunchKernelGGL(csr_spmm_generic_kernel, grid, block, 0, st, m, feat, d_A, d_B, d_C, d_indptr, d_indices);
  }
#undef STIR_CSR_ROWS
#undef STIR_CSR
  STIR_LAUNCH_CHECK();
  return 0;
}

int stir_hyb_plan_create(stir_hyb_plan** plan, int32_t m, int32_t n, int32_t num_col_parts,
                         int32_t num_buckets, const int32_t* bucket_widths, const int64_t* nrows,
                         const float* const* d_A, const int32_t* const* d_rows,
                         const int32_t* const* d_cols) {
  return stir_hyb_plan_create_ex(plan, m, n, num_col_parts, num_buckets, bucket_widths, nrows, d_A, d_rows, d_cols, 0);
}

int stir_hyb_plan_create_ex(stir_hyb_plan** plan, int32_t m, int32_t n, int32_t num_col_parts,
                            int32_t num_buckets, const int32_t* bucket_widths, const int64_t* nrows,
                            const float* const* d_A, const int32_t* const* d_rows,
                            const int32_t* const* d_cols, uint32_t flags) {
  STIR_REQUIRE(plan, "hyb_plan_create: plan is null");
  STIR_REQUIRE((flags & ~uint32_t(STIR_PLAN_ADDRESSES_ONLY)) == 0, "hyb_plan_create: unknown flags 0x%x", flags);
  if (check_hyb_arguments("hyb_plan_create", m, n, num_col_parts, num_buckets, bucket_widths, nrows, d_A, d_rows,
                          d_cols) != 0)
    return -1;
  // nothing of the plan may depend on what the arrays hold: one launch, atomics in every adding
  // bucket (the reference's rule), no list of slots per output row
  const bool addresses_only = (flags & STIR_PLAN_ADDRESSES_ONLY) != 0;
  bool phased = !addresses_only && num_col_parts > 1 && num_col_parts <= kMaxPhases;
  if (phased && phases_have_single_writers(m, num_col_parts, num_buckets, nrows, d_rows, &phased) != 0) return -1;
  stir_hyb_plan* p = new stir_hyb_plan();
  p->m = m;
  p->n = n;
  p->num_col_parts = num_col_parts;
  p->num_buckets = num_buckets;
  p->d_tables = nullptr;
  p->merged = false;
  bool want_merged = !addresses_only && num_col_parts > kMaxPhases;
  if (!addresses_only && num_col_parts > 1 && num_col_parts <= kMaxPhases) {
    size_t slots = 0;
    for (int k = 0; k < num_col_parts * num_buckets; ++k) slots += size_t(nrows[k]) * size_t(bucket_widths[k % num_buckets]);
    want_merged = slots * 12 <= kMergedOptionalBytes;
  }
  if (want_merged &&
      build_merged_rows(m, num_col_parts * num_buckets, num_buckets, bucket_widths, nrows, d_A, d_rows, d_cols,
                        &p->rows, &p->merged) != 0) {
    delete p;
    return -1;
  }
  make_hyb_tables(num_col_parts, num_buckets, bucket_widths, nrows, d_A, d_rows, d_cols, phased, &p->tables);
  const size_t nk = p->tables.tiles.size();
  hipError_t e = hipGetDevice(&p->device);
  if (e == hipSuccess && nk > 0) {
    e = hipMalloc(reinterpret_cast<void**>(&p->d_tables), sizeof(HybBucket) * 2 * nk);
    if (e == hipSuccess)
      e = hipMemcpy(p->d_tables, p->tables.tiles.data(), sizeof(HybBucket) * nk, hipMemcpyHostToDevice);
    if (e == hipSuccess)
      e = hipMemcpy(p->d_tables + nk, p->tables.rows.data(), sizeof(HybBucket) * nk, hipMemcpyHostToDevice);
  }
  if (e != hipSuccess) {
    if (p->d_tables) (void)hipFree(p->d_tables);
    p->rows.release();
    delete p;
    return stir::fail("hyb_plan_create: %s", hipGetErrorString(e));
  }
  *plan = p;
  return 0;
}

int stir_hyb_spmm_f32(const stir_hyb_plan* plan, int32_t feat, const float* d_B, float* d_C,
                      void* stream) {
  STIR_REQUIRE(plan, "hyb_spmm: plan is null");
  STIR_REQUIRE(feat > 0, "hyb_spmm: feat=%d", feat);
  const size_t nk = plan->tables.tiles.size();
  if (nk == 0) return 0;
  STIR_REQUIRE(d_B && d_C, "hyb_spmm: null pointer argument");
  if (plan->merged && vector_class(feat) >= 0 && (plan->num_col_parts > kMaxPhases || feat >= kMergedFromFeat))
    return launch_merged(plan->rows, plan->m, feat, d_B, d_C, static_cast<hipStream_t>(stream));
  return launch_hyb(plan->tables, plan->d_tables, plan->d_tables + nk, feat, d_B, d_C,
                    static_cast<hipStream_t>(stream));
}

int stir_hyb_spmm_f32_noalloc(int32_t m, int32_t n, int32_t num_col_parts, int32_t num_buckets,
                              const int32_t* bucket_widths, const int64_t* nrows, const float* const* d_A,
                              const int32_t* const* d_rows, const int32_t* const* d_cols, int32_t feat,
                              const float* d_B, float* d_C, void* stream) {
  static_assert(sizeof(HybBucket) == 64, "descriptor size the scratch array is laid out for");
  if (check_hyb_arguments("hyb_spmm_noalloc", m, n, num_col_parts, num_buckets, bucket_widths, nrows, d_A, d_rows,
                          d_cols) != 0)
    return -1;
  STIR_REQUIRE(feat > 0, "hyb_spmm_noalloc: feat=%d", feat);
  HybTables tables;
  // one launch, every bucket adds with atomics when there are several partitions
  // (examples/spmm/bench_spmm.py:170 of the reference): nothing is known about the row arrays here
  make_hyb_tables(num_col_parts, num_buckets, bucket_widths, nrows, d_A, d_rows, d_cols, false, &tables);
  const int nk = (int)tables.tiles.size();
  if (nk == 0) return 0;
  STIR_REQUIRE(nk <= kStaticBuckets, "hyb_spmm_noalloc: %d non-empty buckets, at most %d are supported", nk,
               kStaticBuckets);
  STIR_REQUIRE(d_B && d_C, "hyb_spmm_noalloc: null pointer argument");
  HybBucket* d_tables = nullptr;
  if (static_scratch(&d_tables) != 0) return -1;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // only the table the kernel for this feature width reads is written
  const bool generic = vector_class(feat) < 0;
  const std::vector<HybBucket>& src = generic ? tables.rows : tables.tiles;
  HybBucket* dst = generic ? d_tables + kStaticBuckets : d_tables;
  for (int first = 0; first < nk; first += kTableChunk) {
    HybTableChunk chunk = {};
    const int count = std::min(kTableChunk, nk - first);
    std::copy(src.begin() + first, src.begin() + first + count, chunk.b);
    hipLaunchKernelGGL(hyb_table_fill_kernel, dim3(1), dim3(256), 0, st, chunk, count, dst + first);
  }
  STIR_LAUNCH_CHECK();
  return launch_hyb(tables, d_tables, d_tables + kStaticBuckets, feat, d_B, d_C, st);
}

int stir_hyb_plan_destroy(stir_hyb_plan* plan) {
  if (!plan) return 0;
  if (plan->d_tables) (void)hipFree(plan->d_tables);
  plan->rows.release();
  delete plan;
  return 0;
}

}  // extern "C"
