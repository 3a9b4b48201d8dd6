// Row lookup for kernels that walk the nonzeros of a CSR matrix: which row owns nonzero e,
// i.e. the last r with indptr[r] <= e.
//
// A per-nonzero binary search over all of indptr costs ~log2(m) dependent loads.  Here a
// wavefront owns a tile of consecutive nonzeros; the rows of the tile's first and last nonzero are
// found by the whole wavefront (64 probes of indptr per step narrow the range 64-fold), the row
// pointers in between go to LDS with one coalesced load, and every nonzero is located there.  A
// tile that spans more rows than the window holds (long runs of empty rows) falls back to a
// per-nonzero search between the two rows.
#pragma once
#include "common.h"

namespace stir {

// last r in [0, m] with indptr[r] <= q; all lanes pass the same q and get the same answer
__device__ __forceinline__ int wave_last_row(const int32_t* __restrict__ indptr, int m, int64_t q, int lane) {
  int lo = 0, hi = m;  // indptr[lo] <= q, the answer lies in [lo, hi]
  while (hi > lo) {
    const int span = hi - lo;
    const int pos = lo + (int)(((int64_t)span * (lane + 1) + kWave - 1) / kWave);  // in (lo, hi], ascending
    const int cnt = __popcll(__ballot((int64_t)indptr[pos] <= q));  // true for the first cnt lanes
    const int new_lo = cnt ? __shfl(pos, cnt - 1, kWave) : lo;
    const int new_hi = cnt < kWave ? __shfl(pos, cnt, kWave) - 1 : hi;
    lo = new_lo;
    hi = new_hi;
  }
  return lo;
}

constexpr int kRowLookupWindow = 512;  // row pointers held in LDS per wavefront

// Calls f(e, row, t, live) for e = e0 + t * 64 + lane, t < PER: `live` says whether e <= e_last,
// and `row` is then the row that owns e (0 otherwise).  All 64 lanes make every call together, so
// f may use cross-lane operations.  `win` is the wavefront's own LDS piece of kRowLookupWindow
// ints.  Every lane of the wavefront must call this with the same e0 and e_last.
template <int PER, class F>
__device__ __forceinline__ void for_each_nonzero_row(const int32_t* __restrict__ indptr, int m, int64_t e0,
                                                     int64_t e_last, int32_t* win, int lane, F f) {
  const int ra = wave_last_row(indptr, m, e0, lane);
  const int rb = wave_last_row(indptr, m, e_last, lane);
  const int nr = rb - ra + 1;
  if (nr <= kRowLookupWindow) {
    __builtin_amdgcn_wave_barrier();
    for (int x = lane; x < nr; x += kWave) win[x] = indptr[ra + x];
    __builtin_amdgcn_wave_barrier();
    int steps = 0;
    while ((1 << steps) < nr) ++steps;
    // the searches advance together so that their LDS reads overlap
    int a[PER], b[PER];
#pragma unroll
    for (int t = 0; t < PER; ++t) a[t] = 0, b[t] = nr - 1;
    for (int it = 0; it < steps; ++it) {
#pragma unroll
      for (int t = 0; t < PER; ++t) {
        const int c = (a[t] + b[t] + 1) >> 1;
        if ((int64_t)win[c] <= e0 + t * kWave + lane) a[t] = c; else b[t] = c - 1;
      }
    }
#pragma unroll
    for (int t = 0; t < PER; ++t) {
      const int64_t e = e0 + t * kWave + lane;
      const bool live = e <= e_last;
      f(e, live ? ra + a[t] : 0, t, live);
    }
  } else {
#pragma unroll 1
    for (int t = 0; t < PER; ++t) {
      const int64_t e = e0 + t * kWave + lane;
      const bool live = e <= e_last;
      int a = ra, b = live ? rb : ra;
      while (a < b) {
        const int c = a + ((b - a + 1) >> 1);
        if ((int64_t)indptr[c] <= e) a = c; else b = c - 1;
      }
      f(e, live ? a : 0, t, live);
    }
  }
}

}  // namespace stir
