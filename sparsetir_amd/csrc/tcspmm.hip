// SpMM on the gfx950 matrix cores over the condensed format of ConDense: the rows of the
// sparse matrix are cut into tiles of t rows (t = 8, 16 -- the two sizes the reference's
// examples/spmm/bench_tc_spmm.py:584-585,670 condenses with -- or 32); inside a tile the distinct
// columns are gathered g = 16 at a time into dense t x 16 blocks A[jo] (zero where the row has no
// entry):
//   C[io*t + ii, f] = sum over groups jo of tile io, ji < 16:  A[jo, ii, ji] * B[indices[jo, ji], f]
// fp16 inputs, fp32 accumulation, fp16 or fp32 output.
//
// Same tiling as the BSR kernel: a workgroup of four wavefronts owns (row tile, 128 features),
// a wavefront t rows x 32 features.  A step covers two groups (32 gathered rows of B): A[jo] is
// already in MFMA A-operand order (a lane's 8 k values are contiguous), the 32 gathered rows of
// B go through LDS, interleaved into (k, k+1) pairs on the way, double-buffered, with the next
// step's gathers in flight during the multiply.  Tiles of 32 rows multiply with two
// v_mfma_f32_32x32x16_f16 per step (one per group); tiles of 16 rows with v_mfma_f32_16x16x32_f16,
// whose k extent of 32 is the step's two groups, once per 16 features; tiles of 8 rows are the
// upper half of a 16-row operand whose other rows are zero.
//
// A row tile that touches thousands of distinct columns (a hub row of a power-law graph) would be
// one long serial chain in one workgroup.  With fp32 output such tiles are cut into up to kSplit
// units of at least kUnitSteps steps that add their results with atomics; a first launch clears the rows
// of those tiles.  With fp16 output partial sums would be rounded once per unit; there, tiles of
// more than kLongSteps steps are left to a second launch (tcspmm_long_kernel) whose workgroups
// have 16 wavefronts that split the steps of the tile among them and add their fp32 partial sums
// through LDS before the one write of the tile.  (For fp32 output that launch is the slower of the
// two ways: the launches run in turn.  Running them side by side on two streams was tried for
// fp16 output and lost: workgroups of 16 wavefronts wait for room beside the other launch, and
// the hub tile's chain runs slower on a shared compute unit than the overlap gains.)
// With a plan (stir_tc_plan: the long tiles listed once, longest first, in pieces of at most
// kPieceSteps steps) the second launch has a workgroup per piece and the hub tiles are spread
// over many compute units; fp32 partial tiles in the plan's memory, one rounding at the end.
#include <algorithm>
#include <vector>

#include "common.h"
#include "../../include/sparsetir_amd.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileF = 128;
constexpr int kGroup = 16;  // g
constexpr int kUnitSteps = 16;  // steps (of two groups) per unit of a long tile
constexpr int kSplit = 16;      // most units per tile (second grid dimension of the split launch)
constexpr int kLongSteps = 16;  // fp16 output: tiles with more steps go to the second launch
constexpr int kLongScan = 8;    // ... each workgroup of which looks at this many row tiles
constexpr int kLongNT = 2;      // ... whose workgroups own 32 * kLongNT features and have 32 / kLongNT * 4 wavefronts

__device__ __forceinline__ int tile_steps(const int32_t* __restrict__ indptr, int64_t io) {
  const int64_t rows_total = (int64_t)(indptr[io + 1] - indptr[io]) * kGroup;
  return (int)((rows_total + 31) / 32);
}

// ---- what differs between the row-tile sizes: the accumulators of a wavefront for (T rows) x
// (32 features), the A operand of a step, and the multiply of a step out of the staged rows of B.
// WIDE = 32-row tiles on the 32x32x16 instruction; otherwise 16-row operands on 16x16x32.
template <bool WIDE>
struct TcAcc;
template <>
struct TcAcc<true> {
  static constexpr int kRegs = 16;
  f32x16 r;
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int v = 0; v < 16; ++v) r[v] = 0.f;
  }
  __device__ __forceinline__ float get(int v) const { return r[v]; }
  // register v of lane l is this row / feature of the wavefront's tile
  static __device__ __forceinline__ int row(int v, int l) { return (v & 3) + 4 * (l >> 5) + 8 * (v >> 2); }
  static __device__ __forceinline__ int col(int v, int l) { return l & 31; }
};
template <>
struct TcAcc<false> {
  static constexpr int kRegs = 8;  // two 16x16 tiles side by side
  f32x4 r[2];
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int v = 0; v < 8; ++v) r[v >> 2][v & 3] = 0.f;
  }
  __device__ __forceinline__ float get(int v) const { return r[v >> 2][v & 3]; }
  static __device__ __forceinline__ int row(int v, int l) { return 4 * (l >> 4) + (v & 3); }
  static __device__ __forceinline__ int col(int v, int l) { return 16 * (v >> 2) + (l & 15); }
};

// A[jo] and A[jo + 1] as the A operand(s) of a step (zero past the tile's last group).
// T = 32: lane (n = l % 32, h = l / 32) holds A[jo + d][n][8h .. 8h+7] in a[d].
// T <= 16: lane (i = l % 16, q = l / 16) holds k = 8q .. 8q+7 of the step's 32, i.e.
// A[jo + q/2][i][8(q%2) ..], in a[0]; rows i >= T of the operand are zero.
template <int T>
__device__ __forceinline__ void tc_load_a(u32x4 (&a)[2], const uint16_t* __restrict__ A, int64_t jo, int64_t g_end,
                                          int lane) {
  a[0] = a[1] = u32x4{0, 0, 0, 0};
  if constexpr (T == 32) {
    const int n = lane & 31, h = lane >> 5;
    a[0] = *reinterpret_cast<const u32x4*>(A + (jo * 32 + n) * kGroup + 8 * h);
    if (jo + 1 < g_end) a[1] = *reinterpret_cast<const u32x4*>(A + ((jo + 1) * 32 + n) * kGroup + 8 * h);
  } else {
    const int i = lane & 15, q = lane >> 4;
    const int64_t grp = jo + (q >> 1);
    if (i < T && grp < g_end) a[0] = *reinterpret_cast<const u32x4*>(A + (grp * T + i) * kGroup + 8 * (q & 1));
  }
}

// Where 16-byte-aligned feature offset `col` of k pair `kp` lives inside its staged row of STRIDE
// words (a power of two).  The 16-row multiply reads rows 4q .. 4q+3 for q = l / 16 at 16
// consecutive features: rotating a row by 16 (kp / 4) words puts the four q on different banks.
template <int T, int STRIDE>
__device__ __forceinline__ int tc_stage_col(int kp, int col) {
  if constexpr (T == 32) return col;
  else return (col + 16 * (kp >> 2)) & (STRIDE - 1);
}

// acc += A-operand(s) x the 32 staged rows of B, features col0 .. col0+31 of the staged rows
// xs[16 k pairs][STRIDE]
template <int T, int STRIDE>
__device__ __forceinline__ void tc_multiply(TcAcc<T == 32>& acc, const u32x4 (&a)[2], const uint32_t* xs, int col0,
                                            int lane) {
  if constexpr (T == 32) {
    const int n = lane & 31, h = lane >> 5;
    u32x4 b0, b1;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      b0[d] = xs[(4 * h + d) * STRIDE + col0 + n];      // rows 8h .. 8h+7 of the first group
      b1[d] = xs[(8 + 4 * h + d) * STRIDE + col0 + n];  // rows 8h .. 8h+7 of the second group
    }
    acc.r = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[0]), __builtin_bit_cast(f16x8, b0),
                                                  acc.r, 0, 0, 0);
    acc.r = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[1]), __builtin_bit_cast(f16x8, b1),
                                                  acc.r, 0, 0, 0);
  } else {
    const int n = lane & 15, q = lane >> 4;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int c = tc_stage_col<T, STRIDE>(4 * q, col0 + 16 * nt) + n;
      u32x4 b;
#pragma unroll
      for (int d = 0; d < 4; ++d) b[d] = xs[(4 * q + d) * STRIDE + c];  // rows 8q .. 8q+7 of the step
      acc.r[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a[0]),
                                                        __builtin_bit_cast(f16x8, b), acc.r[nt], 0, 0, 0);
    }
  }
}

// Clears the fp32 rows of the tiles that the split launch accumulates into.  grid (mb * f_tiles)
__global__ __launch_bounds__(256) void tcspmm_clear_long_kernel(int tile, int feat, int64_t mb, int f_tiles,
                                                                float* __restrict__ C,
                                                                const int32_t* __restrict__ indptr) {
  const int f_tile = (int)(blockIdx.x % f_tiles);
  const int64_t io = blockIdx.x / f_tiles;
  if (io >= mb || tile_steps(indptr, io) <= kUnitSteps) return;
  const int f0 = f_tile * kTileF;
  for (int e = threadIdx.x; e < tile * kTileF; e += 256) {
    const int row = e / kTileF, f = f0 + e % kTileF;
    if (f < feat) C[(io * tile + row) * feat + f] = 0.f;
  }
}

// OUT: 0 = fp16 output, 1 = fp32 output.  SPLIT: grid is (mb * f_tiles, kSplit); the units of a
// long tile take equal shares of its steps and add with atomics, unit 0 of a short tile stores.
template <int T, int OUT, bool SPLIT, bool SKIP_LONG = (OUT == 0)>
__global__ __launch_bounds__(256) void tcspmm_kernel(int feat, int64_t mb, int f_tiles,
                                                     const uint16_t* __restrict__ A,
                                                     const uint16_t* __restrict__ B, void* __restrict__ C,
                                                     const int32_t* __restrict__ indptr,
                                                     const int32_t* __restrict__ indices) {
  __shared__ __attribute__((aligned(16))) uint32_t xs[2][16 * kTileF];  // [buffer][k pair][feature]
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int f_tile = (int)(blockIdx.x % f_tiles);
  const int64_t io = blockIdx.x / f_tiles;
  if (io >= mb) return;
  const int f0 = f_tile * kTileF;
  const int kp = tid >> 4, fc = tid & 15;  // staging role: k pair, 8-feature chunk
  const bool stage_live = f0 + fc * 8 < feat;
  const int stage_at = kp * kTileF + tc_stage_col<T, kTileF>(kp, fc * 8);

  TcAcc<T == 32> acc;
  acc.clear();

  const int64_t g_begin = indptr[io], g_end = indptr[io + 1];
  const int64_t rows_total = (g_end - g_begin) * kGroup;  // gathered rows of B for this tile
  const int steps = (int)((rows_total + 31) / 32);
  const int32_t* rowlist = indices + g_begin * kGroup;
  if constexpr (SKIP_LONG) {
    if (steps > kLongSteps) return;  // left to the launch for long tiles; uniform over the workgroup
  }
  int it_begin = 0, it_end = steps;
  bool add = false;
  if constexpr (SPLIT) {
    const int u = blockIdx.y;
    if (steps > kUnitSteps) {
      add = true;
      const int len = max(kUnitSteps, (steps + kSplit - 1) / kSplit);  // even shares beyond kSplit units
      it_begin = u * len;
      it_end = min(steps, it_begin + len);
      if (it_begin >= it_end) return;  // uniform over the workgroup
    } else if (u > 0) {
      return;
    }
  }

  // The row ids of a step are requested one step before its rows of B, so that a step costs one
  // memory round trip, not two in a row.
  int row_a = 0, row_b = 0;
  auto fetch_ids = [&](int it) {
    const int64_t k = (int64_t)it * 32 + 2 * kp;
    row_a = row_b = 0;
    if (k < rows_total) row_a = rowlist[k], row_b = rowlist[k + 1];  // the same group: both exist
  };
  u32x4 r0, r1, a_next[2];
  auto fetch = [&](int it) {
    tc_load_a<T>(a_next, A, g_begin + 2 * it, g_end, lane);
    r0 = r1 = u32x4{0, 0, 0, 0};
    const int64_t k = (int64_t)it * 32 + 2 * kp;
    if (stage_live && k < rows_total) {
      r0 = *reinterpret_cast<const u32x4*>(B + (int64_t)row_a * feat + f0 + fc * 8);
      r1 = *reinterpret_cast<const u32x4*>(B + (int64_t)row_b * feat + f0 + fc * 8);
    }
    if (it + 1 < it_end) fetch_ids(it + 1);
  };

  if (it_begin < it_end) {
    fetch_ids(it_begin);
    fetch(it_begin);
  }
  for (int it = it_begin; it < it_end; ++it) {
    const int buf = it & 1;
    const u32x4 a_now[2] = {a_next[0], a_next[1]};
    u32x4 lo, hi;
#pragma unroll
    for (int d = 0; d < 2; ++d) {
      lo[2 * d] = __builtin_amdgcn_perm(r1[d], r0[d], 0x05040100);
      lo[2 * d + 1] = __builtin_amdgcn_perm(r1[d], r0[d], 0x07060302);
      hi[2 * d] = __builtin_amdgcn_perm(r1[d + 2], r0[d + 2], 0x05040100);
      hi[2 * d + 1] = __builtin_amdgcn_perm(r1[d + 2], r0[d + 2], 0x07060302);
    }
    *reinterpret_cast<u32x4*>(&xs[buf][stage_at]) = lo;
    *reinterpret_cast<u32x4*>(&xs[buf][stage_at + 4]) = hi;
    if (it + 1 < it_end) fetch(it + 1);
    __syncthreads();
    tc_multiply<T, kTileF>(acc, a_now, xs[buf], wave * 32, lane);
  }
  const int fcol = f0 + wave * 32;
  if (fcol >= feat) return;
#pragma unroll
  for (int v = 0; v < TcAcc<T == 32>::kRegs; ++v) {
    const int row = TcAcc<T == 32>::row(v, lane);
    if (T < 16 && row >= T) continue;
    const int64_t off = (io * T + row) * feat + fcol + TcAcc<T == 32>::col(v, lane);
    if constexpr (OUT == 1) {
      if (add)
        __hip_atomic_fetch_add(static_cast<float*>(C) + off, acc.get(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else
        static_cast<float*>(C)[off] = acc.get(v);
    } else {
      const _Float16 hv = (_Float16)acc.get(v);
      static_cast<uint16_t*>(C)[off] = __builtin_bit_cast(uint16_t, hv);
    }
  }
}

// The steps [s_begin, s_end) of row tile io for the features [f0, f0 + 32 * NTL), by a workgroup of
// 32 / NTL wavefronts: 8 with all four 32-feature accumulators of a 128-feature slice, or (what is
// launched) 16 with two -- 64 features; half the accumulators and half the staged bytes per
// wavefront, so that 16 fit the register file.  Wavefront w takes steps s_begin + w, + WAVES, ...,
// gathers the step's 32 rows of B itself (lane: k pairs kp, kp + KP, ... and 8-feature chunk
// fc) into its own piece of LDS -- no workgroup barrier in the loop, the LDS operations of one
// wavefront execute in order -- and the partial results are added through LDS, one 32-feature
// tile at a time; store(row in tile, feature, sum) receives every sum once.  The steps are a chain
// per wavefront (a step is a round trip to memory): more wavefronts per tile shorten it.
// lds: WAVES * 16 * 32 * NTL words (64 KB either way).  Ends with LDS reads: a caller that goes on
// to another tile puts a workgroup barrier in between.
template <int T, int NTL, class Store>
__device__ __forceinline__ void tcspmm_long_steps(uint32_t* __restrict__ lds, int feat, int64_t io, int f0,
                                                  int s_begin, int s_end, const uint16_t* __restrict__ A,
                                                  const uint16_t* __restrict__ B,
                                                  const int32_t* __restrict__ indptr,
                                                  const int32_t* __restrict__ indices, Store store) {
  using Acc = TcAcc<T == 32>;
  constexpr int WAVES = 32 / NTL;  // wavefronts per workgroup
  constexpr int TF = 32 * NTL;     // features per workgroup
  constexpr int CH = TF / 8;       // 8-feature chunks of a staged row
  constexpr int KP = 64 / CH;      // k pairs a wavefront stages at once
  constexpr int Q = 16 / KP;       // ... times Q = the 16 k pairs of a step
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kp = lane / CH, fc = lane % CH;
  const bool stage_live = f0 + fc * 8 < feat;
  uint32_t* xs = lds + wave * (16 * TF);  // [k pair][feature]
  const int64_t g_begin = indptr[io], g_end = indptr[io + 1];
  const int64_t rows_total = (g_end - g_begin) * kGroup;
  const int32_t* rowlist = indices + g_begin * kGroup;

  Acc acc[NTL];
#pragma unroll
  for (int t = 0; t < NTL; ++t) acc[t].clear();

  // row ids one step (of this wavefront) before the rows of B, as in the kernel above
  int row_a[Q], row_b[Q];
  auto fetch_ids = [&](int it) {
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      const int64_t k = (int64_t)it * 32 + 2 * (kp + KP * q);
      row_a[q] = row_b[q] = 0;
      if (k < rows_total) row_a[q] = rowlist[k], row_b[q] = rowlist[k + 1];
    }
  };
  u32x4 r0[Q], r1[Q], a_next[2];
  auto fetch = [&](int it) {
    tc_load_a<T>(a_next, A, g_begin + 2 * it, g_end, lane);
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      r0[q] = r1[q] = u32x4{0, 0, 0, 0};
      const int64_t k = (int64_t)it * 32 + 2 * (kp + KP * q);
      if (stage_live && k < rows_total) {
        r0[q] = *reinterpret_cast<const u32x4*>(B + (int64_t)row_a[q] * feat + f0 + fc * 8);
        r1[q] = *reinterpret_cast<const u32x4*>(B + (int64_t)row_b[q] * feat + f0 + fc * 8);
      }
    }
    if (it + WAVES < s_end) fetch_ids(it + WAVES);
  };

  // a wavefront without a step (fewer steps than wavefronts) only takes part in the sums
  if (s_begin + wave < s_end) {
    fetch_ids(s_begin + wave);
    fetch(s_begin + wave);
  }
  for (int it = s_begin + wave; it < s_end; it += WAVES) {
    const u32x4 a_now[2] = {a_next[0], a_next[1]};
#pragma unroll
    for (int q = 0; q < Q; ++q) {
      u32x4 lo, hi;
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        lo[2 * d] = __builtin_amdgcn_perm(r1[q][d], r0[q][d], 0x05040100);
        lo[2 * d + 1] = __builtin_amdgcn_perm(r1[q][d], r0[q][d], 0x07060302);
        hi[2 * d] = __builtin_amdgcn_perm(r1[q][d + 2], r0[q][d + 2], 0x05040100);
        hi[2 * d + 1] = __builtin_amdgcn_perm(r1[q][d + 2], r0[q][d + 2], 0x07060302);
      }
      const int at = (kp + KP * q) * TF + tc_stage_col<T, TF>(kp + KP * q, fc * 8);
      *reinterpret_cast<u32x4*>(xs + at) = lo;
      *reinterpret_cast<u32x4*>(xs + at + 4) = hi;
    }
    if (it + WAVES < s_end) fetch(it + WAVES);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int t = 0; t < NTL; ++t) tc_multiply<T, TF>(acc[t], a_now, xs, t * 32, lane);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();  // the next step's stores come after these reads
  }

  // ---- the partial tiles, one 32-feature tile at a time: a thread sums register v of lane l
  // over the wavefronts
  constexpr int REGS = Acc::kRegs;
  float* red = reinterpret_cast<float*>(lds);  // [wavefront][register][lane], at most 4 KB per wavefront
#pragma unroll
  for (int t = 0; t < NTL; ++t) {
    __syncthreads();  // staging pieces (t = 0) or the sums of the tile before are done with
#pragma unroll
    for (int v = 0; v < REGS; ++v) red[(wave * REGS + v) * 64 + lane] = acc[t].get(v);
    __syncthreads();
    for (int e = tid; e < REGS * 64; e += 64 * WAVES) {
      const int v = e >> 6, l = e & 63;
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) sum += red[(w * REGS + v) * 64 + l];
      const int row = Acc::row(v, l);
      const int fcol = f0 + t * 32 + Acc::col(v, l);
      if (fcol < feat && row < T) store(row, fcol, sum);
    }
  }
}

// fp16 output without a plan: the tiles the kernel above skips (more than kLongSteps steps).
template <int T, int NTL>
__global__ __launch_bounds__(64 * (32 / NTL)) void tcspmm_long_kernel(int feat, int64_t mb, int f_tiles,
                                                                      const uint16_t* __restrict__ A,
                                                                      const uint16_t* __restrict__ B,
                                                                      void* __restrict__ C,
                                                                      const int32_t* __restrict__ indptr,
                                                                      const int32_t* __restrict__ indices) {
  extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
  const int lane = threadIdx.x & 63;
  const int f0 = (int)(blockIdx.x % f_tiles) * (32 * NTL);
  // A workgroup looks at kLongScan row tiles and works on the long ones among them (most have
  // none): a workgroup per tile would start tens of thousands that only find out that their tile
  // is short, each holding 64 KB of LDS while it does.  Its tiles lie a whole grid apart -- long
  // tiles come in runs (the hub rows of a graph sorted by degree) and would otherwise queue up in
  // one workgroup.
  const int64_t io_stride = gridDim.x / f_tiles;
  // which of them are long: lane k asks for the group range of the k-th tile, all at once
  uint64_t todo;
  {
    const int64_t io = blockIdx.x / f_tiles + (int64_t)lane * io_stride;
    int64_t groups = 0;
    if (lane < kLongScan && io < mb) groups = indptr[io + 1] - indptr[io];
    todo = __ballot((groups * kGroup + 31) / 32 > kLongSteps);
  }
  bool used_lds = false;
  while (todo) {
    const int k_tile = __ffsll((long long)todo) - 1;
    todo &= todo - 1;
    const int64_t io = blockIdx.x / f_tiles + (int64_t)k_tile * io_stride;
    if (used_lds) __syncthreads();  // the sums of the tile before have been read
    used_lds = true;
    tcspmm_long_steps<T, NTL>(lds, feat, io, f0, 0, tile_steps(indptr, io), A, B, indptr, indices,
                              [&](int row, int fcol, float sum) {
                                const _Float16 hv = (_Float16)sum;
                                static_cast<uint16_t*>(C)[(io * T + row) * feat + fcol] = __builtin_bit_cast(uint16_t, hv);
                              });
  }
}

// ---- fp16 output with a plan (stir_tc_plan): the long tiles are listed once, longest first, and
// cut into pieces of at most kPieceSteps steps, a workgroup of 16 wavefronts each, so that the
// hub tiles of a power-law graph are spread over many compute units from the start of the launch
// and no workgroup is started only to find its tile short.  A tile that is one piece is written
// as fp16 by its workgroup; the pieces of a longer tile leave fp32 partial tiles in the plan's
// scratch memory, and the workgroup that finishes last among the pieces of a tile (per feature
// tile: a counter in device memory, which that workgroup sets back to zero) adds them up in piece
// order and rounds once -- no launch of its own for the sums, and the same bits whichever
// workgroup comes last.  The partial tiles are written and read with device-coherent accesses
// (they pass the XCD's L2), so that no workgroup has to write back or invalidate a whole L2 --
// which a release or acquire at device scope does, and which costs more than the extra launch.
constexpr int kPieceSteps = 128;

struct TcPiece {
  int32_t tile, step_begin, step_end;
  int32_t slot;        // partial tile in the scratch memory, or -1: the piece is the whole tile
  int32_t first_slot;  // of the tile's pieces
  int32_t pieces;      // of the tile
  int32_t multi;       // number of the tile among the tiles of several pieces
  int32_t pad;
};

__device__ __forceinline__ void coherent_store(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float coherent_load(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int T, int NTL, int OUT>
__global__ __launch_bounds__(64 * (32 / NTL)) void tcspmm_pieces_kernel(int feat, int f_tiles,
                                                                        const TcPiece* __restrict__ pieces,
                                                                        const uint16_t* __restrict__ A,
                                                                        const uint16_t* __restrict__ B,
                                                                        void* __restrict__ C,
                                                                        float* scratch, uint32_t* arrived,
                                                                        const int32_t* __restrict__ indptr,
                                                                        const int32_t* __restrict__ indices) {
  extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
  __shared__ int last_of_tile;
  constexpr int TF = 32 * NTL;
  const TcPiece pc = pieces[blockIdx.x / f_tiles];
  const int f_tile = (int)(blockIdx.x % f_tiles);
  const int f0 = f_tile * TF;
  const int64_t io = pc.tile;
  // a plan made from other contents of indptr: stay inside the tile as it is now
  const int s_end = min(pc.step_end, tile_steps(indptr, io));
  if (pc.slot < 0) {
    tcspmm_long_steps<T, NTL>(lds, feat, io, f0, pc.step_begin, s_end, A, B, indptr, indices,
                              [&](int row, int fcol, float sum) {
                                const int64_t off = (io * T + row) * feat + fcol;
                                if constexpr (OUT == 1) {
                                  static_cast<float*>(C)[off] = sum;
                                } else {
                                  const _Float16 hv = (_Float16)sum;
                                  static_cast<uint16_t*>(C)[off] = __builtin_bit_cast(uint16_t, hv);
                                }
                              });
    return;
  }
  const int64_t elems = (int64_t)T * feat;
  float* part = scratch + (int64_t)pc.slot * elems;
  tcspmm_long_steps<T, NTL>(lds, feat, io, f0, pc.step_begin, s_end, A, B, indptr, indices,
                            [&](int row, int fcol, float sum) { coherent_store(part + (int64_t)row * feat + fcol, sum); });
  // Every wavefront waits until its stores have arrived, then one thread counts the workgroup
  // in: whoever counts last finds the partial tiles of all the others in memory.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t* counter = arrived + (int64_t)pc.multi * f_tiles + f_tile;
    const uint32_t before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool last = before + 1 == (uint32_t)pc.pieces;
    if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    last_of_tile = last;
  }
  __syncthreads();
  if (!last_of_tile) return;
  // C[tile, f0 .. f0 + TF) = the partial tiles added in piece order, rounded once; four
  // consecutive features per thread (feat is a multiple of 32)
  const float* first = scratch + (int64_t)pc.first_slot * elems;
  for (int w = threadIdx.x; w < T * (TF / 4); w += 64 * (32 / NTL)) {
    const int row = w / (TF / 4), fcol = f0 + (w % (TF / 4)) * 4;
    if (fcol >= feat) continue;
    const int64_t e = (int64_t)row * feat + fcol;
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int p0 = 0; p0 < pc.pieces; p0 += 4) {
      float4 x[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        x[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (p0 + u < pc.pieces) {
          const float* at = first + (p0 + u) * elems + e;
          x[u] = make_float4(coherent_load(at), coherent_load(at + 1), coherent_load(at + 2), coherent_load(at + 3));
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) sum.x += x[u].x, sum.y += x[u].y, sum.z += x[u].z, sum.w += x[u].w;
    }
    if constexpr (OUT == 1) {
      *reinterpret_cast<float4*>(static_cast<float*>(C) + io * elems + e) = sum;
    } else {
      const _Float16 h0 = (_Float16)sum.x, h1 = (_Float16)sum.y, h2 = (_Float16)sum.z, h3 = (_Float16)sum.w;
      uint2 out;
      out.x = (uint32_t)__builtin_bit_cast(uint16_t, h0) | ((uint32_t)__builtin_bit_cast(uint16_t, h1) << 16);
      out.y = (uint32_t)__builtin_bit_cast(uint16_t, h2) | ((uint32_t)__builtin_bit_cast(uint16_t, h3) << 16);
      *reinterpret_cast<uint2*>(static_cast<uint16_t*>(C) + io * elems + e) = out;
    }
  }
}

constexpr int kLongTF = 32 * kLongNT, kLongWaves = 32 / kLongNT;
constexpr size_t kLongLds = size_t(kLongWaves) * 16 * kLongTF * sizeof(uint32_t);

int check_args(int32_t out_dtype, int32_t mb, int32_t tile_size, int32_t group_size, int32_t feat, int64_t nnzb,
               const void* d_A, const void* d_B, void* d_C, const int32_t* d_indptr, const int32_t* d_indices) {
  STIR_REQUIRE(out_dtype == STIR_F16 || out_dtype == STIR_F32, "tc_spmm: out_dtype must be STIR_F16 or STIR_F32");
  STIR_REQUIRE((tile_size == 8 || tile_size == 16 || tile_size == 32) && group_size == kGroup,
               "tc_spmm: tile_size=%d group_size=%d; the MFMA path needs t in {8, 16, 32} and g=16", tile_size,
               group_size);
  STIR_REQUIRE(mb >= 0 && nnzb >= 0, "tc_spmm: bad sizes");
  STIR_REQUIRE(feat > 0 && feat % 32 == 0, "tc_spmm: feat=%d must be a multiple of 32", feat);
  STIR_REQUIRE(mb == 0 || (d_B && d_C && d_indptr && (nnzb == 0 || (d_A && d_indices))),
               "tc_spmm: null pointer argument");
  return 0;
}

template <int T>
int launch_unplanned(bool out32, int32_t mb, int32_t feat, const uint16_t* A, const uint16_t* B, void* d_C,
                     const int32_t* d_indptr, const int32_t* d_indices, hipStream_t st) {
  const int f_tiles = (int)stir::ceil_div(feat, kTileF);
  const int64_t blocks = (int64_t)mb * f_tiles;
  STIR_REQUIRE(blocks < (int64_t(1) << 31), "tc_spmm: too many tiles for one launch");
  if (out32) {
    hipLaunchKernelGGL(tcspmm_clear_long_kernel, dim3((unsigned)blocks), dim3(256), 0, st, T, feat, (int64_t)mb,
                       f_tiles, static_cast<float*>(d_C), d_indptr);
    STIR_LAUNCH_CHECK();
    hipLaunchKernelGGL((tcspmm_kernel<T, 1, true>), dim3((unsigned)blocks, kSplit), dim3(256), 0, st, feat,
                       (int64_t)mb, f_tiles, A, B, d_C, d_indptr, d_indices);
  } else {
    // the two launches write different row tiles
    const int long_f_tiles = (int)stir::ceil_div(feat, kLongTF);
    const int64_t long_blocks = stir::ceil_div((int64_t)mb, kLongScan) * long_f_tiles;
    STIR_REQUIRE(long_blocks < (int64_t(1) << 31), "tc_spmm: too many tiles for one launch");
    hipLaunchKernelGGL((tcspmm_kernel<T, 0, false>), dim3((unsigned)blocks), dim3(256), 0, st, feat, (int64_t)mb,
                       f_tiles, A, B, d_C, d_indptr, d_indices);
    STIR_LAUNCH_CHECK();
    hipLaunchKernelGGL((tcspmm_long_kernel<T, kLongNT>), dim3((unsigned)long_blocks), dim3(64 * kLongWaves), kLongLds,
                       st, feat, (int64_t)mb, long_f_tiles, A, B, d_C, d_indptr, d_indices);
  }
  STIR_LAUNCH_CHECK();
  return 0;
}

template <int T>
int launch_planned(bool out32, int32_t mb, int32_t feat, int64_t n_pieces, const TcPiece* d_pieces, float* d_scratch,
                   uint32_t* d_arrived, const uint16_t* A, const uint16_t* B, void* d_C, const int32_t* d_indptr,
                   const int32_t* d_indices, hipStream_t st) {
  const int f_tiles = (int)stir::ceil_div(feat, kTileF);
  const int64_t blocks = (int64_t)mb * f_tiles;
  STIR_REQUIRE(blocks < (int64_t(1) << 31), "tc_spmm: too many tiles for one launch");
  // the tiles of up to kLongSteps steps
  if (out32)
    hipLaunchKernelGGL((tcspmm_kernel<T, 1, false, true>), dim3((unsigned)blocks), dim3(256), 0, st, feat,
                       (int64_t)mb, f_tiles, A, B, d_C, d_indptr, d_indices);
  else
    hipLaunchKernelGGL((tcspmm_kernel<T, 0, false, true>), dim3((unsigned)blocks), dim3(256), 0, st, feat,
                       (int64_t)mb, f_tiles, A, B, d_C, d_indptr, d_indices);
  STIR_LAUNCH_CHECK();
  if (n_pieces == 0) return 0;
  const int long_f_tiles = (int)stir::ceil_div(feat, kLongTF);
  const int64_t long_blocks = n_pieces * long_f_tiles;
  STIR_REQUIRE(long_blocks < (int64_t(1) << 31), "tc_spmm: too many pieces for one launch");
  if (out32)
    hipLaunchKernelGGL((tcspmm_pieces_kernel<T, kLongNT, 1>), dim3((unsigned)long_blocks), dim3(64 * kLongWaves),
                       kLongLds, st, feat, long_f_tiles, d_pieces, A, B, d_C, d_scratch, d_arrived, d_indptr,
                       d_indices);
  else
    hipLaunchKernelGGL((tcspmm_pieces_kernel<T, kLongNT, 0>), dim3((unsigned)long_blocks), dim3(64 * kLongWaves),
                       kLongLds, st, feat, long_f_tiles, d_pieces, A, B, d_C, d_scratch, d_arrived, d_indptr,
                       d_indices);
  STIR_LAUNCH_CHECK();
  return 0;
}

}  // namespace

extern "C" int stir_tc_spmm_f16(int32_t out_dtype, int32_t mb, int32_t tile_size, int32_t group_size,
                                int32_t feat, int64_t nnzb, const void* d_A, const void* d_B, void* d_C,
                                const int32_t* d_indptr, const int32_t* d_indices, void* stream) {
  if (check_args(out_dtype, mb, tile_size, group_size, feat, nnzb, d_A, d_B, d_C, d_indptr, d_indices)) return -1;
  if (mb == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint16_t* A = static_cast<const uint16_t*>(d_A);
  const uint16_t* B = static_cast<const uint16_t*>(d_B);
  const bool out32 = out_dtype == STIR_F32;
  switch (tile_size) {
    case 8: return launch_unplanned<8>(out32, mb, feat, A, B, d_C, d_indptr, d_indices, st);
    case 16: return launch_unplanned<16>(out32, mb, feat, A, B, d_C, d_indptr, d_indices, st);
    default: return launch_unplanned<32>(out32, mb, feat, A, B, d_C, d_indptr, d_indices, st);
  }
}

struct stir_tc_plan {
  int32_t mb = 0;
  int device = 0;
  int64_t n_pieces = 0, n_multi = 0, slots = 0;
  TcPiece* d_pieces = nullptr;
  float* d_scratch = nullptr;  // slots x 32 x feat floats, grown by the launch that needs more
  size_t scratch_bytes = 0;
  // per tile of several pieces and feature tile: the pieces that have finished in the running
  // launch; zero between launches (the workgroup that counts last clears its counter)
  uint32_t* d_arrived = nullptr;
  size_t arrived_count = 0;
};

extern "C" int stir_tc_plan_destroy(stir_tc_plan* plan) {
  if (!plan) return 0;
  if (plan->d_pieces) (void)hipFree(plan->d_pieces);
  if (plan->d_arrived) (void)hipFree(plan->d_arrived);
  if (plan->d_scratch) (void)hipFree(plan->d_scratch);
  delete plan;
  return 0;
}

extern "C" int stir_tc_plan_create(stir_tc_plan** plan, int32_t mb, const int32_t* d_indptr, void* stream) {
  STIR_REQUIRE(plan, "tc_plan_create: plan is null");
  STIR_REQUIRE(mb >= 0 && (mb == 0 || d_indptr), "tc_plan_create: bad arguments");
  hipStream_t st = static_cast<hipStream_t>(stream);
  std::vector<int32_t> ptr(size_t(mb) + 1, 0);
  if (mb > 0) {
    STIR_HIP(hipMemcpyAsync(ptr.data(), d_indptr, sizeof(int32_t) * ptr.size(), hipMemcpyDeviceToHost, st));
    STIR_HIP(hipStreamSynchronize(st));
  }
  // the long tiles, longest first (ties in tile order)
  std::vector<std::pair<int32_t, int32_t>> longs;  // (steps, tile)
  for (int32_t io = 0; io < mb; ++io) {
    STIR_REQUIRE(ptr[io] <= ptr[io + 1], "tc_plan_create: indptr decreases at tile %d", io);
    const int64_t steps = ((int64_t)(ptr[io + 1] - ptr[io]) * kGroup + 31) / 32;
    if (steps > kLongSteps) longs.emplace_back((int32_t)steps, io);
  }
  std::stable_sort(longs.begin(), longs.end(),
                   [](const std::pair<int32_t, int32_t>& a, const std::pair<int32_t, int32_t>& b) { return a.first > b.first; });
  std::vector<TcPiece> pieces;
  int64_t slots = 0, n_multi = 0;
  for (const auto& lt : longs) {
    const int32_t steps = lt.first, io = lt.second;
    const int32_t n = (steps + kPieceSteps - 1) / kPieceSteps;  // pieces of equal length
    const int32_t len = (steps + n - 1) / n;
    STIR_REQUIRE(slots + n < (int64_t(1) << 31), "tc_plan_create: too many pieces");
    for (int32_t p = 0; p < n; ++p)
      pieces.push_back(TcPiece{io, p * len, std::min(steps, (p + 1) * len), n > 1 ? (int32_t)(slots + p) : -1,
                               (int32_t)slots, n, (int32_t)n_multi, 0});
    if (n > 1) slots += n, ++n_multi;
  }
  stir_tc_plan* p = new stir_tc_plan();
  p->mb = mb;
  p->n_pieces = (int64_t)pieces.size();
  p->n_multi = n_multi;
  p->slots = slots;
  hipError_t e = hipGetDevice(&p->device);
  if (e == hipSuccess && !pieces.empty()) {
    e = hipMalloc(reinterpret_cast<void**>(&p->d_pieces), sizeof(TcPiece) * pieces.size());
    if (e == hipSuccess)
      e = hipMemcpyAsync(p->d_pieces, pieces.data(), sizeof(TcPiece) * pieces.size(), hipMemcpyHostToDevice, st);
  }
  if (e == hipSuccess) e = hipStreamSynchronize(st);  // the host vectors go away
  if (e != hipSuccess) {
    stir_tc_plan_destroy(p);
    return stir::fail("tc_plan_create: %s", hipGetErrorString(e));
  }
  *plan = p;
  return 0;
}

extern "C" int stir_tc_spmm_f16_planned(stir_tc_plan* plan, int32_t out_dtype, int32_t mb, int32_t tile_size,
                                        int32_t group_size, int32_t feat, int64_t nnzb, const void* d_A,
                                        const void* d_B, void* d_C, const int32_t* d_indptr,
                                        const int32_t* d_indices, void* stream) {
  STIR_REQUIRE(plan, "tc_spmm_planned: plan is null");
  if (check_args(out_dtype, mb, tile_size, group_size, feat, nnzb, d_A, d_B, d_C, d_indptr, d_indices)) return -1;
  STIR_REQUIRE(plan->mb == mb, "tc_spmm_planned: the plan was made for %d row tiles, not %d", plan->mb, mb);
  int device = 0;
  STIR_HIP(hipGetDevice(&device));
  STIR_REQUIRE(device == plan->device, "tc_spmm_planned: the plan lives on device %d, the current device is %d",
               plan->device, device);
  if (mb == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint16_t* A = static_cast<const uint16_t*>(d_A);
  const uint16_t* B = static_cast<const uint16_t*>(d_B);
  // the sums of the partial tiles leave four to a thread, as one 8- or 16-byte store
  const bool out32 = out_dtype == STIR_F32;
  STIR_REQUIRE(plan->n_multi == 0 || reinterpret_cast<uintptr_t>(d_C) % (out32 ? 16 : 8) == 0,
               "tc_spmm: C must be %d-byte aligned", out32 ? 16 : 8);
  // the partial tiles of this tile size and feature width
  const size_t need = size_t(plan->slots) * size_t(tile_size) * size_t(feat) * sizeof(float);
  if (need > plan->scratch_bytes) {
    if (plan->d_scratch) STIR_HIP(hipFree(plan->d_scratch));
    plan->d_scratch = nullptr;
    plan->scratch_bytes = 0;
    STIR_HIP(hipMalloc(reinterpret_cast<void**>(&plan->d_scratch), need));
    plan->scratch_bytes = need;
  }
  const size_t counters = size_t(plan->n_multi) * size_t(stir::ceil_div(feat, kLongTF));
  if (counters > plan->arrived_count) {
    if (plan->d_arrived) STIR_HIP(hipFree(plan->d_arrived));
    plan->d_arrived = nullptr;
    plan->arrived_count = 0;
    STIR_HIP(hipMalloc(reinterpret_cast<void**>(&plan->d_arrived), counters * sizeof(uint32_t)));
    STIR_HIP(hipMemsetAsync(plan->d_arrived, 0, counters * sizeof(uint32_t), st));
    plan->arrived_count = counters;
  }
  switch (tile_size) {
    case 8:
      return launch_planned<8>(out32, mb, feat, plan->n_pieces, plan->d_pieces, plan->d_scratch, plan->d_arrived, A, B,
                               d_C, d_indptr, d_indices, st);
    case 16:
      return launch_planned<16>(out32, mb, feat, plan->n_pieces, plan->d_pieces, plan->d_scratch, plan->d_arrived, A,
                                B, d_C, d_indptr, d_indices, st);
    default:
      return launch_planned<32>(out32, mb, feat, plan->n_pieces, plan->d_pieces, plan->d_scratch, plan->d_arrived, A,
                                B, d_C, d_indptr, d_indices, st);
  }
}
