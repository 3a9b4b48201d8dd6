// BSR SpMM on the gfx950 matrix cores: Y[i-th block row] = sum over stored blocks p of
// A_p (blk x blk) * X[indices[p]-th block of rows], 16-bit inputs, fp32 accumulation.
//
// A workgroup of four wavefronts owns 32 or 64 rows of a block row and a 128*NT-wide slice of the
// feature axis; a wavefront owns NT 32-feature tiles per 32 rows, each a 32x32 fp32 accumulator
// fed by v_mfma_f32_32x32x16_{f16,bf16}.  Both operands go through LDS: the MFMA B operand wants
// 8 consecutive k for one feature per lane while X is feature-contiguous, and the A fragment is
// shared by the four wavefronts (see bsr_tile).  Small launches use bsr_spmm_ksplit_kernel.
#include <hip/hip_fp16.h>

#include <numeric>

#include "common.h"
#include "../../include/sparsetir_amd.h"

namespace {

using stir::kWave;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __fp16 tr16x4 __attribute__((__vector_size__(4 * sizeof(__fp16))));  // result type of the transposing LDS read
#define STIR_LDS __attribute__((address_space(3)))

constexpr int kTileF = 128;  // features per workgroup
constexpr int kTileK = 32;   // k rows staged per step

template <bool BF16>
__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

template <bool BF16>
__device__ __forceinline__ uint16_t to16(float v) {
  if constexpr (BF16) {
    uint32_t u = __float_as_uint(v);
    if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x40);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);                                          // nearest even
    return uint16_t(u >> 16);
  } else {
    _Float16 h = (_Float16)v;
    return __builtin_bit_cast(uint16_t, h);
  }
}

// Workgroup -> (32-row slice, feature tile).  Workgroups are dispatched round-robin over the 8
// XCDs, each with its own L2.  All slices of one feature tile read the same columns of X
// (nb*blk rows x TF features), so when there are at least 8 feature tiles each XCD walks its own
// feature tiles one after the other and that slice of X stays resident in its L2; with fewer
// tiles the tile index is the fastest-varying one, which (for 1, 2 or 4 tiles) also pins a tile
// to an XCD.
__device__ __forceinline__ bool decode_tile(int64_t L, int64_t slices, int f_tiles, int64_t& slice,
                                            int& f_tile) {
  if (f_tiles >= 8) {
    const int xcd = (int)(L & 7);
    const int64_t slot = L >> 3;
    f_tile = xcd + 8 * (int)(slot / slices);
    slice = slot % slices;
    return f_tile < f_tiles;
  }
  f_tile = (int)(L % f_tiles);
  slice = L / f_tiles;
  return slice < slices;
}

// One tile of the output: the 32*RS rows [bi0, bi0 + 32*RS) of stored block row i times the
// features [f0, f0 + 128*NT).  256 threads = 4 wavefronts; wavefront w owns features
// [32*NT*w, 32*NT*(w+1)) of the tile and RS*NT 32x32 accumulators.  RS = 2 (blocks of 64 rows and
// more): two adjacent 32-row slices of a block row, so every X fragment read from LDS feeds two
// MFMAs and the X tile is fetched once for 64 rows.
//
// Per step (one stored block, 32 of its k columns) the workgroup brings a 32 x 128*NT tile of X
// and the 32*RS x 32 piece of the block into LDS -- each thread loads 16-byte chunks, consecutive
// lanes consecutive chunks of a row of X -- while the previous step is multiplied (two LDS
// stages, one barrier per step).  LDS keeps X feature-contiguous, in 16-byte units of 8 features:
// unit (k, c) sits at (k/4)*4*FCN + (k%4)*FCN + (c ^ 4*(k%4)), FCN = units per row.  The MFMA B
// operand (8 consecutive k for one feature per lane) comes out of that image through the
// transposing read ds_read_b64_tr_b16, which hands lane i of a block of 16 lanes four consecutive
// k of column i when the lanes address rows k .. k+3, four features each.  The LDS serves such a
// read 32 lanes at a time from 64 banks: two blocks of 16 lanes, each reading two units in each of
// four rows whose stride is a multiple of all banks, so the XOR has to move the four rows of a
// block to four different groups of four units (c ^ 4*(k%4); with c ^ 2*(k%4) two rows of the two
// blocks met in the same banks and every read took twice its cycles).  The 16-byte stores of a row
// (8 lanes and 8 consecutive units per cycle) stay on distinct banks under either XOR.
// The block piece is fetched once per workgroup (8*RS bytes per thread) and laid out by k chunk so
// that a lane's A operand is one 16-byte read.
// lds: 2 * (64*128*NT + 2048*RS) bytes.
template <bool BF16, int OUT, int NT, int RS>  // OUT: 0 = same 16-bit type as the inputs, 1 = fp32
__device__ __forceinline__ void bsr_tile(char* __restrict__ lds, int blk, int feat, int i, int i_out, int bi0,
                                         int f0, const uint16_t* __restrict__ A,
                                         const uint16_t* __restrict__ X, void* __restrict__ Y,
                                         const int32_t* __restrict__ indptr,
                                         const int32_t* __restrict__ indices) {
  constexpr int TF = kTileF * NT;
  constexpr int FCN = TF / 8;            // 16-byte units per tile row
  constexpr int XB = kTileK * TF * 2;    // bytes of X per stage
  constexpr int SB = XB + 2048 * RS;     // bytes per stage
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;

  // staging role: 2*NT chunks of X per thread
  uint32_t xoff[2 * NT], xdst[2 * NT];
#pragma unroll
  for (int q = 0; q < 2 * NT; ++q) {
    const int idx = 64 * (wave * 2 * NT + q) + lane, c = idx % FCN, k = idx / FCN;
    xoff[q] = (uint32_t)(k * feat + 8 * c);  // in elements, from the tile's first element
    xdst[q] = (uint32_t)(((k >> 2) * 4 * FCN + (k & 3) * FCN + (c ^ (4 * (k & 3)))) * 16);
  }
  // a lane's chunks all lie in the same feature column (FCN divides 64): one test for all of
  // them; feat is a multiple of 32, so chunks are whole.  A lane beyond feat never loads and
  // keeps staging the zeros its registers start with.
  static_assert(64 % FCN == 0, "a lane's chunks share their feature column");
  const bool xlive = f0 + 8 * (lane % FCN) < feat;
  // ... and 8*RS bytes of the block: RS = 1: half of the unit (chunk tid/64, row (tid/2)%32);
  // RS = 2: the unit (slice tid/128, chunk (tid/32)%4, row tid%32)
  uint32_t aoff;
  if constexpr (RS == 1)
    aoff = (uint32_t)(((tid >> 1) & 31) * blk + (tid >> 6) * 8 + (tid & 1) * 4);
  else
    aoff = (uint32_t)((32 * (tid >> 7) + (tid & 31)) * blk + ((tid >> 5) & 3) * 8);
  // operand reads, bytes inside a stage
  const int sl = lane & 15, half16 = (lane >> 4) & 1;
  uint32_t bread[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int kr = sl >> 2, c = (wave * NT + t) * 4 + 2 * half16 + ((sl & 3) >> 1);
    bread[t] = (uint32_t)(((2 * h) * 4 * FCN + kr * FCN + (c ^ (4 * kr))) * 16 + (sl & 1) * 8);
  }
  const uint32_t aread = XB + (h * 32 + n) * 16;

  f32x16 acc[RS][NT];
#pragma unroll
  for (int rs = 0; rs < RS; ++rs)
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[rs][t][v] = 0.f;

  const int p_begin = indptr[i];
  const int nblk = indptr[i + 1] - p_begin;
  const int steps = nblk * (blk / kTileK);

  // The step to fetch next: block pb of the row, k offset k0.  The block column of the block after
  // the current one is requested a whole block ahead, so that no step waits for an index before
  // it can ask for its rows of X.
  int pb = 0, k0 = 0;
  int j_cur = nblk > 0 ? indices[p_begin] : 0;
  int j_nxt = nblk > 1 ? indices[p_begin + 1] : 0;
  u32x4 xr[2 * NT];
#pragma unroll
  for (int q = 0; q < 2 * NT; ++q) xr[q] = u32x4{0, 0, 0, 0};
  u32x4 ar;  // RS = 1 uses the first two words
  auto fetch = [&]() {
    const uint16_t* xb = X + ((int64_t)j_cur * blk + k0) * feat + f0;
    const uint16_t* ab = A + (int64_t)(p_begin + pb) * blk * blk + (int64_t)bi0 * blk + k0;
    if (xlive) {
#pragma unroll
      for (int q = 0; q < 2 * NT; ++q) xr[q] = *reinterpret_cast<const u32x4*>(xb + xoff[q]);
    }
    if constexpr (RS == 1) {
      const u32x2 v = *reinterpret_cast<const u32x2*>(ab + aoff);
      ar[0] = v[0], ar[1] = v[1];
    } else {
      ar = *reinterpret_cast<const u32x4*>(ab + aoff);
    }
    k0 += kTileK;
    if (k0 == blk) {
      k0 = 0;
      ++pb;
      j_cur = j_nxt;
      if (pb + 1 < nblk) j_nxt = indices[p_begin + pb + 1];
    }
  };

  if (steps > 0) fetch();
  for (int it = 0; it < steps; ++it) {
    char* stage = lds + (it & 1) * SB;
#pragma unroll
    for (int q = 0; q < 2 * NT; ++q) *reinterpret_cast<u32x4*>(stage + xdst[q]) = xr[q];
    if constexpr (RS == 1)
      *reinterpret_cast<u32x2*>(stage + XB + tid * 8) = u32x2{ar[0], ar[1]};
    else
      *reinterpret_cast<u32x4*>(stage + XB + tid * 16) = ar;
    if (it + 1 < steps) fetch();
    __syncthreads();  // stage `it` is complete; the other stage's readers passed the previous barrier
    u32x4 a[RS][2];
#pragma unroll
    for (int rs = 0; rs < RS; ++rs)
#pragma unroll
      for (int m = 0; m < 2; ++m) a[rs][m] = *reinterpret_cast<const u32x4*>(stage + aread + rs * 2048 + m * 1024);
#pragma unroll
    for (int m = 0; m < 2; ++m) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const char* bp = stage + bread[t] + (4 * m) * FCN * 64;
        const tr16x4 t0 = __builtin_amdgcn_ds_read_tr16_b64_v4f16((STIR_LDS tr16x4*)(bp));
        const tr16x4 t1 = __builtin_amdgcn_ds_read_tr16_b64_v4f16((STIR_LDS tr16x4*)(bp + FCN * 64));
        const u32x2 lo = __builtin_bit_cast(u32x2, t0), hi = __builtin_bit_cast(u32x2, t1);
        const u32x4 b = {lo[0], lo[1], hi[0], hi[1]};
#pragma unroll
        for (int rs = 0; rs < RS; ++rs) acc[rs][t] = mfma32<BF16>(a[rs][m], b, acc[rs][t]);
      }
    }
  }
  // acc[rs][t][v] is row 32 rs + (v%4) + 4h + 8(v/4), column n of the t-th 32x32 tile.
  // The row stride is made opaque here: when this function is inlined into a loop over tiles,
  // the sixteen row offsets would otherwise be computed once before that loop and held in
  // registers throughout it (60 registers, halving the resident workgroups).
  int row_stride = feat;
  asm volatile("" : "+s"(row_stride));
#pragma unroll
  for (int rs = 0; rs < RS; ++rs) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int fcol = f0 + (wave * NT + t) * 32;
      if (fcol >= feat) continue;
      const int64_t first = ((int64_t)i_out * blk + bi0 + 32 * rs + 4 * h) * row_stride + fcol + n;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t off = first + (int64_t)((v & 3) + 8 * (v >> 2)) * row_stride;
        if constexpr (OUT == 1)
          __builtin_nontemporal_store(acc[rs][t][v], static_cast<float*>(Y) + off);
        else
          __builtin_nontemporal_store(to16<BF16>(acc[rs][t][v]), static_cast<uint16_t*>(Y) + off);
      }
    }
  }
}

// The other order, for tall blocks (by_rows): XCD x owns the block rows i = x, x + 8, ... and
// walks, for each, the slices of the block row inside every feature tile before the next feature
// tile.  The workgroups that are resident together on an XCD then share the blocks of A of their
// block row (fetched into that L2 once instead of once per feature tile) and, between the slices
// of a block row, its tiles of X.
__device__ __forceinline__ bool decode_tile_by_rows(int64_t L, int64_t block_rows, int sub, int f_tiles,
                                                    int64_t& slice, int& f_tile) {
  const int xcd = (int)(L & 7);
  const int64_t t = L >> 3;
  const int64_t i = xcd + 8 * (t / ((int64_t)sub * f_tiles));
  f_tile = (int)((t / sub) % f_tiles);
  slice = i * sub + t % sub;
  return i < block_rows;
}

// One workgroup per tile, 1-D grid (see decode_tile).
template <bool BF16, int OUT, int NT, int RS>
__global__ __launch_bounds__(256) void bsr_spmm_kernel(int blk, int feat, int64_t slices, int f_tiles, int by_rows,
                                                       const uint16_t* __restrict__ A,
                                                       const uint16_t* __restrict__ X, void* __restrict__ Y,
                                                       const int32_t* __restrict__ indptr,
                                                       const int32_t* __restrict__ indices,
                                                       const int32_t* __restrict__ row_ids) {
  constexpr int TF = kTileF * NT;
  __shared__ __attribute__((aligned(16))) char xs[2 * (kTileK * TF * 2 + 2048 * RS)];
  int64_t slice;
  int f_tile;
  const int sub = blk / (32 * RS);  // slices of 32*RS rows per block row
  if (by_rows) {
    if (!decode_tile_by_rows(blockIdx.x, slices / sub, sub, f_tiles, slice, f_tile)) return;
  } else if (!decode_tile(blockIdx.x, slices, f_tiles, slice, f_tile)) {
    return;
  }
  const int i = (int)(slice / sub), bi0 = (int)(slice % sub) * (32 * RS);
  // doubly-compressed form: stored block row i is block row row_ids[i] of the output
  const int i_out = row_ids ? row_ids[i] : i;
  bsr_tile<BF16, OUT, NT, RS>(xs, blk, feat, i, i_out, bi0, f_tile * TF, A, X, Y, indptr, indices);
}

// ------------------------------------------------------------------ large launches, swept in step
// When the X rows of one feature tile (nb*blk rows of 256*NT bytes) exceed a per-XCD L2 (4 MB),
// workgroups that walk their block rows at unrelated times miss L2 on about half of their X
// tiles.  Block columns are ascending inside a block row, so workgroups that start together on
// block rows of equal length move through X together and share a narrow window of it.  This
// kernel arranges that: exactly as many workgroups as are resident at once (gridDim.x = 8 * G,
// workgroup b runs on XCD b % 8, the dispatch order of the hardware), each a loop over tiles; all
// workgroups of an XCD work on the same feature tile, and in round r workgroup w of the XCD takes
// the slice of rank r*G + w when slices are ordered by their number of blocks, longest first.  A
// round's slices have (nearly) the same length, so no workgroup has to wait for another and the
// workgroups still stay in step; nothing here synchronises workgroups, the order only decides
// what L2 holds.  The ranking is computed by every workgroup from indptr before its first tile
// (a stable counting sort in LDS: every workgroup gets the same permutation).
constexpr int kSweepMaxSlices = 8192;  // permutation entries are 16 bits wide and live in LDS
constexpr int kSweepBins = 1024;       // block rows with more blocks than this share the last bin
constexpr int kSweepMaxItems = 128;    // tiles per workgroup and feature tile

// Calls f(value, lanes holding it) once per distinct value among the lanes with valid = true.
template <typename F>
__device__ __forceinline__ void for_each_distinct(int value, bool valid, F f) {
  uint64_t todo = __ballot(valid);
  while (todo) {
    const int src = __ffsll((long long)todo) - 1;
    const int v = __shfl(value, src, kWave);
    const uint64_t same = __ballot(valid && value == v);
    f(v, same);
    todo &= ~same;
  }
}

// Fills items[0 .. count) with the slices this workgroup takes, one per round, for subset
// `part` of `parts`: ranks (r*G + w)*parts + part.  lds: at least 4*kSweepBins + kSweepMaxSlices/2
// words, free again when the call returns.
__device__ __forceinline__ int sweep_my_slices(uint32_t* __restrict__ lds, uint16_t* __restrict__ items,
                                               const int32_t* __restrict__ indptr, int slices, int sub,
                                               int G, int w, int parts, int part) {
  uint32_t* hist = lds;                                                       // [bin][wavefront]
  uint16_t* perm = reinterpret_cast<uint16_t*>(lds + 4 * kSweepBins);         // [rank] -> slice
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  for (int b = tid; b < 4 * kSweepBins; b += 256) hist[b] = 0;
  __syncthreads();
  // wavefront `wave` ranks the contiguous quarter [s_begin, s_end) of the slices
  const int quarter = ((slices + 3) / 4 + kWave - 1) / kWave * kWave;
  const int s_begin = wave * quarter, s_end = min(slices, s_begin + quarter);
  auto bin_of = [&](int s) {
    const int i = s / sub;
    const int len = indptr[i + 1] - indptr[i];
    return kSweepBins - 1 - min(len, kSweepBins - 1);  // longest first
  };
  for (int s0 = s_begin; s0 < s_end; s0 += kWave) {
    const int s = s0 + lane;
    const bool valid = s < s_end;
    const int bin = valid ? bin_of(s) : 0;
    for_each_distinct(bin, valid, [&](int v, uint64_t same) {
      if (lane == 0) hist[v * 4 + wave] += (uint32_t)__popcll(same);
    });
  }
  __syncthreads();
  // exclusive scan over hist in (bin, wavefront) order: 16 consecutive entries per thread, read
  // twice rather than held in registers (the tile loop decides the kernel's register count)
  {
    uint32_t sum = 0;
#pragma unroll 1
    for (int q = 0; q < 16; ++q) sum += hist[tid * 16 + q];
    uint32_t incl = sum;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const uint32_t up = __shfl_up(incl, off, kWave);
      if (lane >= off) incl += up;
    }
    __shared__ uint32_t wave_total[4];
    if (lane == kWave - 1) wave_total[wave] = incl;
    __syncthreads();
    uint32_t base = incl - sum;
    for (int q = 0; q < wave; ++q) base += wave_total[q];
#pragma unroll 1
    for (int q = 0; q < 16; ++q) {
      const uint32_t v = hist[tid * 16 + q];
      hist[tid * 16 + q] = base;
      base += v;
    }
  }
  __syncthreads();
  // placement, in slice order inside every (bin, wavefront) run: stable
  for (int s0 = s_begin; s0 < s_end; s0 += kWave) {
    const int s = s0 + lane;
    const bool valid = s < s_end;
    const int bin = valid ? bin_of(s) : 0;
    for_each_distinct(bin, valid, [&](int v, uint64_t same) {
      const uint32_t first = hist[v * 4 + wave];
      if (valid && bin == v) perm[first + __popcll(same & ((uint64_t(1) << lane) - 1))] = (uint16_t)s;
      __builtin_amdgcn_wave_barrier();
      if (lane == 0) hist[v * 4 + wave] = first + (uint32_t)__popcll(same);
      __builtin_amdgcn_wave_barrier();
    });
  }
  __syncthreads();
  int count = 0;
  for (int r = 0;; ++r) {
    const int64_t rank = ((int64_t)r * G + w) * parts + part;
    if (rank >= slices || r >= kSweepMaxItems) break;
    if (tid == 0) items[r] = perm[rank];
    ++count;
  }
  __syncthreads();
  return count;
}

template <bool BF16, int OUT, int NT, int RS>
__global__ __launch_bounds__(256) void bsr_spmm_sweep_kernel(int blk, int feat, int slices, int f_tiles, int parts,
                                                             const uint16_t* __restrict__ A,
                                                             const uint16_t* __restrict__ X, void* __restrict__ Y,
                                                             const int32_t* __restrict__ indptr,
                                                             const int32_t* __restrict__ indices,
                                                             const int32_t* __restrict__ row_ids) {
  constexpr int TF = kTileF * NT;
  constexpr int kXsWords = 2 * (kTileK * TF * 2 + 2048 * RS) / 4;
  constexpr int kSortWords = 4 * kSweepBins + kSweepMaxSlices / 2;
  __shared__ __attribute__((aligned(16))) uint32_t lds[kXsWords > kSortWords ? kXsWords : kSortWords];
  __shared__ uint16_t items[kSweepMaxItems];
  const int xcd = blockIdx.x & 7, w = blockIdx.x >> 3, G = gridDim.x >> 3;
  const int sub = blk / (32 * RS);
  // unit u = f_tile + f_tiles * part (part: every parts-th slice by rank); XCD x takes units x, x + 8, ...
  const int units = f_tiles * parts;
  int part_of_items = -1, count = 0;
#pragma unroll 1
  for (int u = xcd; u < units; u += 8) {
    const int f_tile = u % f_tiles, part = u / f_tiles;
    if (part != part_of_items) {
      __syncthreads();  // the last tile's LDS reads are over
      count = sweep_my_slices(lds, items, indptr, slices, sub, G, w, parts, part);
      part_of_items = part;
    }
#pragma unroll 1
    for (int r = 0; r < count; ++r) {
      const int slice = items[r];
      const int i = slice / sub, bi0 = (slice % sub) * (32 * RS);
      const int i_out = row_ids ? row_ids[i] : i;
      __syncthreads();  // the previous tile's readers are done with both LDS buffers
      bsr_tile<BF16, OUT, NT, RS>(reinterpret_cast<char*>(lds), blk, feat, i, i_out, bi0, f_tile * TF, A, X, Y,
                                  indptr, indices);
    }
  }
}

// Small launches (at most a couple of workgroups per CU): a workgroup's run time is the serial
// chain of its block row's steps, each a memory round trip, and nothing else is resident to hide
// it.  Here the four wavefronts of a workgroup split the steps of the block row instead of the
// feature axis: wavefront w takes steps w, w + 4, ... for all 128 features (four accumulators),
// stages its own X tile in its own piece of LDS (no workgroup barrier in the loop: the LDS
// operations of one wavefront execute in order) and the four partial results are added through
// LDS at the end.  Same tile and the same global traffic as bsr_spmm_kernel, a chain four times
// shorter.
constexpr int kSplitLdsWords = 4 * 4 * 16 * 64;  // reduction: [wavefront][feature tile][register][lane]

template <bool BF16, int OUT>
__global__ __launch_bounds__(256) void bsr_spmm_ksplit_kernel(int blk, int feat, int64_t slices, int f_tiles,
                                                              const uint16_t* __restrict__ A,
                                                              const uint16_t* __restrict__ X, void* __restrict__ Y,
                                                              const int32_t* __restrict__ indptr,
                                                              const int32_t* __restrict__ indices,
                                                              const int32_t* __restrict__ row_ids) {
  __shared__ __attribute__((aligned(16))) uint32_t lds[kSplitLdsWords];  // 64 KB
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int f_tile = (int)(blockIdx.x % f_tiles);
  const int64_t slice = blockIdx.x / f_tiles;
  const int sub = blk / 32;
  const int i = (int)(slice / sub), bi0 = (int)(slice % sub) * 32;
  const int f0 = f_tile * kTileF;
  // staging role of a lane: k pairs kp, kp + 4, kp + 8, kp + 12; 8-feature chunk fc
  const int kp = lane >> 4, fc = lane & 15;
  const bool stage_live = f0 + fc * 8 < feat;
  uint32_t(*xs)[kTileF] = reinterpret_cast<uint32_t(*)[kTileF]>(lds + wave * (16 * kTileF));  // [k pair][feature]

  f32x16 acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

  const int i_out = row_ids ? row_ids[i] : i;
  const int p_begin = indptr[i];
  const int ksteps = blk / kTileK;
  const int steps = (indptr[i + 1] - p_begin) * ksteps;

  // The block columns of the row's first 64 blocks are fetched once, one per lane: looking them up
  // step by step would put a second memory round trip in front of every step's loads of X.
  const int nblk = indptr[i + 1] - p_begin;
  const int j_lane = lane < nblk ? indices[p_begin + lane] : 0;
  u32x4 r0[4], r1[4], areg[2];
  auto fetch = [&](int it) {
    const int b = it / ksteps, k0 = (it % ksteps) * kTileK;
    const int p = p_begin + b;
    const int64_t j = b < kWave ? __shfl(j_lane, b, kWave) : indices[p];
    const uint16_t* ablk = A + (int64_t)p * blk * blk + (int64_t)(bi0 + n) * blk + k0;
    areg[0] = *reinterpret_cast<const u32x4*>(ablk + 8 * h);
    areg[1] = *reinterpret_cast<const u32x4*>(ablk + 16 + 8 * h);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      r0[q] = r1[q] = u32x4{0, 0, 0, 0};
      if (stage_live) {
        const uint16_t* xp = X + ((int64_t)j * blk + k0 + 2 * (kp + 4 * q)) * feat + f0 + fc * 8;
        r0[q] = *reinterpret_cast<const u32x4*>(xp);
        r1[q] = *reinterpret_cast<const u32x4*>(xp + feat);
      }
    }
  };

  if (wave < steps) fetch(wave);
  for (int it = wave; it < steps; it += 4) {
    const u32x4 a0 = areg[0], a1 = areg[1];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      u32x4 lo, hi;
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        lo[2 * d] = __builtin_amdgcn_perm(r1[q][d], r0[q][d], 0x05040100);
        lo[2 * d + 1] = __builtin_amdgcn_perm(r1[q][d], r0[q][d], 0x07060302);
        hi[2 * d] = __builtin_amdgcn_perm(r1[q][d + 2], r0[q][d + 2], 0x05040100);
        hi[2 * d + 1] = __builtin_amdgcn_perm(r1[q][d + 2], r0[q][d + 2], 0x07060302);
      }
      *reinterpret_cast<u32x4*>(&xs[kp + 4 * q][fc * 8]) = lo;
      *reinterpret_cast<u32x4*>(&xs[kp + 4 * q][fc * 8 + 4]) = hi;
    }
    if (it + 4 < steps) fetch(it + 4);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int col = t * 32 + n;
      u32x4 b0, b1;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        b0[d] = xs[4 * h + d][col];
        b1[d] = xs[8 + 4 * h + d][col];
      }
      acc[t] = mfma32<BF16>(a0, b0, acc[t]);
      acc[t] = mfma32<BF16>(a1, b1, acc[t]);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();  // the next step's stores come after these reads
  }

  // ---- add the four partial results: wavefront w ends up with feature tile w
  __syncthreads();  // every wavefront is done with its staging piece
  float* red = reinterpret_cast<float*>(lds);
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) red[((wave * 4 + t) * 16 + v) * 64 + lane] = acc[t][v];
  __syncthreads();
  const int fcol = f0 + wave * 32;
  if (fcol >= feat) return;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) sum += red[((w * 4 + wave) * 16 + v) * 64 + lane];
    const int row = (v & 3) + 4 * h + 8 * (v >> 2);
    const int64_t off = ((int64_t)i_out * blk + bi0 + row) * feat + fcol + n;
    if constexpr (OUT == 1)
      static_cast<float*>(Y)[off] = sum;
    else
      static_cast<uint16_t*>(Y)[off] = to16<BF16>(sum);
  }
}

// ------------------------------------------------------------------ blocks of 16 k+16 rows
// Block sides that are a multiple of 16 but not of 32 (the reference's schedule splits both block
// axes by 16, examples/blocksparse/bsr_spmm.py:379-380): 16-row slices on v_mfma_f32_16x16x32,
// whose k extent of 32 is two 16-column chunks of the block row's blocks in storage order.  A
// workgroup of four wavefronts owns (block row, 16-row slice, 128 features), a wavefront 16 rows
// x 32 features (two accumulators of four registers).  The A operand -- 8 consecutive k of one row
// per lane -- is one 16-byte load from the block; the 32 rows of X of a step go through LDS as
// (k, k+1) pairs, double-buffered, the next step's loads in flight during the multiply.  Rows of
// the staged image are rotated by 16 (k pair / 4) words so that the four k groups a multiply
// reads lie on different banks.
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <bool BF16>
__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
  if constexpr (BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
}

template <bool BF16, int OUT>
__global__ __launch_bounds__(256) void bsr16_spmm_kernel(int blk, int feat, int64_t slices, int f_tiles,
                                                         const uint16_t* __restrict__ A,
                                                         const uint16_t* __restrict__ X, void* __restrict__ Y,
                                                         const int32_t* __restrict__ indptr,
                                                         const int32_t* __restrict__ indices,
                                                         const int32_t* __restrict__ row_ids) {
  __shared__ __attribute__((aligned(16))) uint32_t xs[2][16 * kTileF];  // [buffer][k pair][feature]
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int f_tile = (int)(blockIdx.x % f_tiles);
  const int64_t slice = blockIdx.x / f_tiles;
  if (slice >= slices) return;
  const int sub = blk / 16;  // 16-row slices per block row = 16-column chunks per block
  const int i = (int)(slice / sub), s = (int)(slice % sub);
  const int i_out = row_ids ? row_ids[i] : i;
  const int f0 = f_tile * kTileF;
  // staging role: k pair kp (rows 2kp, 2kp+1 of the step's 32), 8-feature chunk fc
  const int kp = tid >> 4, fc = tid & 15;
  const bool stage_live = f0 + fc * 8 < feat;
  const int stage_at = kp * kTileF + ((fc * 8 + 16 * (kp >> 2)) & (kTileF - 1));
  // operand role: row ii of the slice, k group q (8 of the step's 32 k)
  const int ii = lane & 15, q = lane >> 4;

  const int p_begin = indptr[i];
  const int chunks = (indptr[i + 1] - p_begin) * sub;
  const int steps = (chunks + 1) / 2;

  f32x4 acc[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // the block column of a step's chunk is requested one step before its rows of X
  int j_stage = 0;
  auto fetch_ids = [&](int it) {
    const int c = 2 * it + (kp >> 3);
    j_stage = c < chunks ? indices[p_begin + c / sub] : 0;
  };
  u32x4 r0, r1, a_next;
  auto fetch = [&](int it) {
    a_next = r0 = r1 = u32x4{0, 0, 0, 0};
    const int ca = 2 * it + (q >> 1);
    if (ca < chunks)
      a_next = *reinterpret_cast<const u32x4*>(A + ((int64_t)(p_begin + ca / sub) * blk + s * 16 + ii) * blk +
                                               (ca % sub) * 16 + 8 * (q & 1));
    const int c = 2 * it + (kp >> 3);
    if (stage_live && c < chunks) {
      const uint16_t* xp = X + ((int64_t)j_stage * blk + (c % sub) * 16 + 2 * (kp & 7)) * feat + f0 + fc * 8;
      r0 = *reinterpret_cast<const u32x4*>(xp);
      r1 = *reinterpret_cast<const u32x4*>(xp + feat);
    }
    if (it + 1 < steps) fetch_ids(it + 1);
  };

  if (steps > 0) {
    fetch_ids(0);
    fetch(0);
  }
  for (int it = 0; it < steps; ++it) {
    const int buf = it & 1;
    const u32x4 a_now = a_next;
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
    if (it + 1 < steps) fetch(it + 1);
    __syncthreads();
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int c = ((wave * 32 + 16 * nt + 16 * q) & (kTileF - 1)) + ii;
      u32x4 b;
#pragma unroll
      for (int d = 0; d < 4; ++d) b[d] = xs[buf][(4 * q + d) * kTileF + c];  // rows 8q .. 8q+7 of the step
      acc[nt] = mfma16<BF16>(a_now, b, acc[nt]);
    }
  }
  const int fcol = f0 + wave * 32;
  if (fcol >= feat) return;
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int64_t off = ((int64_t)i_out * blk + s * 16 + 4 * q + v) * feat + fcol + 16 * nt + ii;
      if constexpr (OUT == 1)
        static_cast<float*>(Y)[off] = acc[nt][v];
      else
        static_cast<uint16_t*>(Y)[off] = to16<BF16>(acc[nt][v]);
    }
}

}  // namespace

static int bsr_launch(int32_t dtype, int32_t out_dtype, int32_t mb, int32_t nb, int32_t blk, int32_t feat,
                      int64_t nnzb, const void* d_A, const void* d_X, void* d_Y, const int32_t* d_indptr,
                      const int32_t* d_indices, const int32_t* d_row_ids, void* stream) {
  STIR_REQUIRE(dtype == STIR_F16 || dtype == STIR_BF16, "bsr_spmm: dtype must be STIR_F16 or STIR_BF16");
  STIR_REQUIRE(out_dtype == dtype || out_dtype == STIR_F32, "bsr_spmm: out_dtype must equal dtype or be STIR_F32");
  STIR_REQUIRE(mb >= 0 && nb >= 0 && nnzb >= 0, "bsr_spmm: bad sizes mb=%d nb=%d", mb, nb);
  STIR_REQUIRE(blk > 0 && blk % 16 == 0, "bsr_spmm: blk=%d must be a multiple of 16", blk);
  STIR_REQUIRE(feat > 0 && feat % 32 == 0, "bsr_spmm: feat=%d must be a multiple of 32", feat);
  if (mb == 0) return 0;
  STIR_REQUIRE(d_X && d_Y && d_indptr && (nnzb == 0 || (d_A && d_indices)), "bsr_spmm: null pointer argument");
  hipStream_t st16 = static_cast<hipStream_t>(stream);
  if (blk % 32 != 0) {
    const int f_tiles16 = (int)stir::ceil_div(feat, kTileF);
    const int64_t slices16 = (int64_t)mb * (blk / 16);
    STIR_REQUIRE(slices16 * f_tiles16 < (int64_t(1) << 31), "bsr_spmm: too many tiles for one launch");
    dim3 grid16((unsigned)(slices16 * f_tiles16)), block16(256);
#define STIR_BSR_16(BF, OUT)                                                                                    \
  hipLaunchKernelGGL((bsr16_spmm_kernel<BF, OUT>), grid16, block16, 0, st16, blk, feat, slices16, f_tiles16,     \
                     static_cast<const uint16_t*>(d_A), static_cast<const uint16_t*>(d_X), d_Y, d_indptr, d_indices, \
                     d_row_ids)
    if (dtype == STIR_BF16) {
      if (out_dtype == STIR_F32) STIR_BSR_16(true, 1); else STIR_BSR_16(true, 0);
    } else {
      if (out_dtype == STIR_F32) STIR_BSR_16(false, 1); else STIR_BSR_16(false, 0);
    }
#undef STIR_BSR_16
    STIR_LAUNCH_CHECK();
    return 0;
  }
  // two 32-row slices per workgroup when the block height allows it
  const int rs = (blk % 64 == 0) ? 2 : 1;
  const int64_t slices = (int64_t)mb * (blk / (32 * rs));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint16_t* A = static_cast<const uint16_t*>(d_A);
  const uint16_t* X = static_cast<const uint16_t*>(d_X);
  // A launch of at most two workgroups per CU is bound by the chain of steps of its longest block
  // row: the four wavefronts of a workgroup then split the steps instead of the features.
  {
    const int f_tiles_s = (int)stir::ceil_div(feat, kTileF);
    const int64_t blocks_s = (int64_t)mb * (blk / 32) * f_tiles_s;
    if (blocks_s <= 2 * (int64_t)stir::compute_units()) {
      const int64_t slices_s = (int64_t)mb * (blk / 32);
      dim3 grid_s((unsigned)blocks_s), block_s(256);
#define STIR_BSR_S(BF, OUT)                                                                                  \
  hipLaunchKernelGGL((bsr_spmm_ksplit_kernel<BF, OUT>), grid_s, block_s, 0, st, blk, feat, slices_s, f_tiles_s, \
                     A, X, d_Y, d_indptr, d_indices, d_row_ids)
      if (dtype == STIR_BF16) {
        if (out_dtype == STIR_F32) STIR_BSR_S(true, 1); else STIR_BSR_S(true, 0);
      } else {
        if (out_dtype == STIR_F32) STIR_BSR_S(false, 1); else STIR_BSR_S(false, 0);
      }
#undef STIR_BSR_S
      STIR_LAUNCH_CHECK();
      return 0;
    }
  }
  // Two 32-wide accumulators per wavefront once the feature axis is wide enough to still yield
  // several workgroups per CU.  One prefetched step is enough: measured on MI355X, deeper
  // register rings (2-6 steps) change nothing, the kernel is not bound by latency.
  const int nt = (feat >= 1024) ? 2 : 1;
  const int f_tiles = (int)stir::ceil_div(feat, kTileF * nt);
  dim3 block(256);
  // Launches whose X rows per feature tile do not fit a per-XCD L2 and that give every resident
  // workgroup several tiles are swept in step (bsr_spmm_sweep_kernel).
  const int cus = stir::compute_units();
  const int64_t x_tile_bytes = (int64_t)nb * blk * kTileF * nt * 2;
  const int parts = 8 / std::gcd(f_tiles, 8);
#define STIR_BSR_SWEEP(BF, OUT, NTV, RSV)                                                                     \
  {                                                                                                           \
    static int occupancy = 0; /* workgroups of this kernel per CU; the same on every gfx950 device */        \
    if (occupancy == 0) {                                                                                     \
      int o = 0;                                                                                              \
      STIR_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&o, bsr_spmm_sweep_kernel<BF, OUT, NTV, RSV>, 256, 0)); \
      occupancy = o > 0 ? o : 1;                                                                              \
    }                                                                                                         \
    const int G = occupancy * (cus / 8);                                                                      \
    const int64_t rounds = stir::ceil_div(stir::ceil_div(slices, parts), G);                                  \
    if (rounds <= kSweepMaxItems && slices * f_tiles >= 4 * 8 * (int64_t)G) {                                 \
      hipLaunchKernelGGL((bsr_spmm_sweep_kernel<BF, OUT, NTV, RSV>), dim3(8 * G), block, 0, st, blk, feat,    \
                         (int)slices, f_tiles, parts, A, X, d_Y, d_indptr, d_indices, d_row_ids);             \
      STIR_LAUNCH_CHECK();                                                                                    \
      return 0;                                                                                               \
    }                                                                                                         \
  }
  // (measured: 16384^2, 32x32 blocks, 10 %, 4096 features 650 -> 590 us, L2 hit rate 46 -> 57 %;
  // with fewer than 8 feature tiles or two slices per workgroup the plain order is faster)
  const bool sweep = cus >= 8 && cus % 8 == 0 && rs == 1 && f_tiles >= 8 && x_tile_bytes > (3 << 20) &&
                     slices <= kSweepMaxSlices;
  // Blocks of 128 rows and more: block rows dealt to XCDs (decode_tile_by_rows).  Measured at
  // 16384^2, 10 %, 4096 features: 128 x 128 blocks 387 -> 365 us; 64 x 64 blocks (one slice per
  // block row, so only A is shared) 443 -> 514 us and 32 x 32 blocks 600 -> 950 us: there the
  // feature tile per XCD, which keeps an XCD on one slice of X, is worth more.
  const int sub_rows = blk / (32 * rs);
  const int by_rows = (rs == 2 && sub_rows >= 2 && f_tiles >= 2) ? 1 : 0;
  const int64_t blocks = by_rows ? 8 * stir::ceil_div((int64_t)mb, 8) * sub_rows * f_tiles
                         : f_tiles >= 8 ? 8 * stir::ceil_div(f_tiles, 8) * slices : (int64_t)f_tiles * slices;
  STIR_REQUIRE(blocks < (int64_t(1) << 31), "bsr_spmm: too many tiles for one launch");
  dim3 grid((unsigned)blocks);
#define STIR_BSR_L(BF, OUT, NTV, RSV)                                                                      \
  {                                                                                                        \
    if (sweep && !by_rows) STIR_BSR_SWEEP(BF, OUT, NTV, RSV);                                                        \
    hipLaunchKernelGGL((bsr_spmm_kernel<BF, OUT, NTV, RSV>), grid, block, 0, st, blk, feat, slices, f_tiles, \
                       by_rows, A, X, d_Y, d_indptr, d_indices, d_row_ids);                                \
  }
#define STIR_BSR(BF, OUT)                                                          \
  do {                                                                             \
    if (nt == 2) {                                                                 \
      if (rs == 2) STIR_BSR_L(BF, OUT, 2, 2) else STIR_BSR_L(BF, OUT, 2, 1)        \
    } else {                                                                       \
      if (rs == 2) STIR_BSR_L(BF, OUT, 1, 2) else STIR_BSR_L(BF, OUT, 1, 1)        \
    }                                                                              \
  } while (0)
  if (dtype == STIR_BF16) {
    if (out_dtype == STIR_F32) STIR_BSR(true, 1); else STIR_BSR(true, 0);
  } else {
    if (out_dtype == STIR_F32) STIR_BSR(false, 1); else STIR_BSR(false, 0);
  }
#undef STIR_BSR
#undef STIR_BSR_L
#undef STIR_BSR_SWEEP
  STIR_LAUNCH_CHECK();
  return 0;
}

extern "C" {

int stir_bsr_spmm(int32_t dtype, int32_t out_dtype, int32_t mb, int32_t nb, int32_t blk, int32_t feat,
                  int64_t nnzb, const void* d_A, const void* d_X, void* d_Y, const int32_t* d_indptr,
                  const int32_t* d_indices, void* stream) {
  return bsr_launch(dtype, out_dtype, mb, nb, blk, feat, nnzb, d_A, d_X, d_Y, d_indptr, d_indices, nullptr,
                    stream);
}

int stir_dbsr_spmm(int32_t dtype, int32_t out_dtype, int32_t nnz_rows, int32_t nb, int32_t blk,
                   int32_t feat, int64_t nnzb, const void* d_A, const void* d_X, void* d_Y,
                   const int32_t* d_row_ids, const int32_t* d_indptr, const int32_t* d_indices,
                   void* stream) {
  STIR_REQUIRE(nnz_rows == 0 || d_row_ids, "dbsr_spmm: row ids are null");
  return bsr_launch(dtype, out_dtype, nnz_rows, nb, blk, feat, nnzb, d_A, d_X, d_Y, d_indptr, d_indices,
                    d_row_ids, stream);
}

}  // extern "C"
