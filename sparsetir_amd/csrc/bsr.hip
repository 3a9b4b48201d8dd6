// BSR SpMM on the gfx950 matrix cores: Y[i-th block row] = sum over stored blocks p of
// A_p (blk x blk) * X[indices[p]-th block of rows], 16-bit inputs, fp32 accumulation.
//
// A workgroup of four wavefronts owns one 32-row slice of a block row and a 128*NT-wide slice
// of the feature axis; a wavefront owns NT 32-feature tiles, each a 32x32 fp32 accumulator fed
// by v_mfma_f32_32x32x16_{f16,bf16}.  The A operand wants 8 consecutive k per lane, which is
// exactly how a row of a stored block lies in memory, so it is loaded straight from global
// memory (16 bytes per lane).  The X operand wants 8 consecutive k for one feature column, but
// X is feature-contiguous, so the 32 x TF tile of X goes through LDS: every thread loads two
// adjacent k rows (16 bytes each), interleaves them into (k, k+1) pairs and stores 32 bytes; a
// lane's MFMA operand is then four 4-byte LDS reads.  Tiles are double-buffered in LDS and the
// next step's global loads are in flight while the current one is multiplied.
#include <hip/hip_fp16.h>

#include "common.h"
#include "../../include/sparsetir_amd.h"

namespace {

using stir::kWave;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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

// 1-D grid (see decode_tile); block: 256 threads = 4 wavefronts; wavefront w owns features
// [32*NT*w, 32*NT*(w+1)) of the TF = 128*NT wide tile and RS*NT 32x32 accumulators.  The X tile of
// step it+1 is fetched into registers while step it is multiplied out of LDS (two LDS buffers,
// one barrier per step).  RS = 2 (blocks of 64 rows and more): a workgroup takes two adjacent
// 32-row slices of a block row, so every X fragment read from LDS feeds two MFMAs and the X tile
// is fetched once for 64 rows.
template <bool BF16, int OUT, int NT, int S, int RS>  // OUT: 0 = same 16-bit type as the inputs, 1 = fp32
__global__ __launch_bounds__(256) void bsr_spmm_kernel(int blk, int feat, int64_t slices, int f_tiles,
                                                       const uint16_t* __restrict__ A,
                                                       const uint16_t* __restrict__ X, void* __restrict__ Y,
                                                       const int32_t* __restrict__ indptr,
                                                       const int32_t* __restrict__ indices,
                                                       const int32_t* __restrict__ row_ids) {
  constexpr int TF = kTileF * NT;
  constexpr int FC = TF / 8;      // 8-feature chunks per tile row
  constexpr int KPT = 256 / FC;   // k pairs covered by one pass of the 256 threads
  __shared__ uint32_t xs[2][kTileK / 2][TF];  // [buffer][k pair][feature] -> (X[2kp][f], X[2kp+1][f])
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, h = lane >> 5;
  int64_t slice;
  int f_tile;
  if (!decode_tile(blockIdx.x, slices, f_tiles, slice, f_tile)) return;
  const int sub = blk / (32 * RS);  // slices of 32*RS rows per block row
  const int i = (int)(slice / sub), bi0 = (int)(slice % sub) * (32 * RS);
  const int f0 = f_tile * TF;
  const int kp0 = tid / FC, fc = tid % FC;
  const bool stage_live = f0 + fc * 8 < feat;  // feat is a multiple of 32, so chunks are whole

  f32x16 acc[RS][NT];
#pragma unroll
  for (int rs = 0; rs < RS; ++rs)
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[rs][t][v] = 0.f;

  // doubly-compressed form: stored block row i is block row row_ids[i] of the output
  const int i_out = row_ids ? row_ids[i] : i;
  const int p_begin = indptr[i];
  const int ksteps = blk / kTileK;
  const int steps = (indptr[i + 1] - p_begin) * ksteps;

  // Register ring of S prefetched steps: loads for step it+S are issued as soon as step it has
  // been copied to LDS, so S tiles per wavefront are in flight while the matrix cores work.
  u32x4 r0[S][NT], r1[S][NT], areg[S][RS][2];
  auto fetch = [&](int it, int s) {
    const int p = p_begin + it / ksteps, k0 = (it % ksteps) * kTileK;
    const int64_t j = indices[p];
#pragma unroll
    for (int rs = 0; rs < RS; ++rs) {
      const uint16_t* ablk = A + (int64_t)p * blk * blk + (int64_t)(bi0 + 32 * rs + n) * blk + k0;
      areg[s][rs][0] = *reinterpret_cast<const u32x4*>(ablk + 8 * h);       // k = k0 + 8h + (0..7)
      areg[s][rs][1] = *reinterpret_cast<const u32x4*>(ablk + 16 + 8 * h);  // k = k0 + 16 + 8h + (0..7)
    }
#pragma unroll
    for (int q = 0; q < NT; ++q) {
      r0[s][q] = r1[s][q] = u32x4{0, 0, 0, 0};
      if (stage_live) {
        const uint16_t* xp = X + ((int64_t)j * blk + k0 + 2 * (kp0 + KPT * q)) * feat + f0 + fc * 8;
        r0[s][q] = *reinterpret_cast<const u32x4*>(xp);
        r1[s][q] = *reinterpret_cast<const u32x4*>(xp + feat);
      }
    }
  };

#pragma unroll
  for (int s = 0; s < S; ++s)
    if (s < steps) fetch(s, s);
  for (int it0 = 0; it0 < steps; it0 += S) {
#pragma unroll
    for (int s = 0; s < S; ++s) {
      const int it = it0 + s;
      if (it < steps) {  // uniform over the workgroup
        const int buf = it & 1;
        u32x4 a0[RS], a1[RS];
#pragma unroll
        for (int rs = 0; rs < RS; ++rs) a0[rs] = areg[s][rs][0], a1[rs] = areg[s][rs][1];
#pragma unroll
        for (int q = 0; q < NT; ++q) {
          u32x4 lo, hi;  // (k, k+1) pairs for features fc*8 + 0..3 and 4..7
#pragma unroll
          for (int d = 0; d < 2; ++d) {
            lo[2 * d] = __builtin_amdgcn_perm(r1[s][q][d], r0[s][q][d], 0x05040100);      // low halves
            lo[2 * d + 1] = __builtin_amdgcn_perm(r1[s][q][d], r0[s][q][d], 0x07060302);  // high halves
            hi[2 * d] = __builtin_amdgcn_perm(r1[s][q][d + 2], r0[s][q][d + 2], 0x05040100);
            hi[2 * d + 1] = __builtin_amdgcn_perm(r1[s][q][d + 2], r0[s][q][d + 2], 0x07060302);
          }
          *reinterpret_cast<u32x4*>(&xs[buf][kp0 + KPT * q][fc * 8]) = lo;
          *reinterpret_cast<u32x4*>(&xs[buf][kp0 + KPT * q][fc * 8 + 4]) = hi;
        }
        if (it + S < steps) fetch(it + S, s);
        __syncthreads();  // tile `it` is complete; the other buffer's readers passed the previous barrier
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const int col = (wave * NT + t) * 32 + n;
          u32x4 b0, b1;
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            b0[d] = xs[buf][4 * h + d][col];
            b1[d] = xs[buf][8 + 4 * h + d][col];
          }
#pragma unroll
          for (int rs = 0; rs < RS; ++rs) {
            acc[rs][t] = mfma32<BF16>(a0[rs], b0, acc[rs][t]);
            acc[rs][t] = mfma32<BF16>(a1[rs], b1, acc[rs][t]);
          }
        }
      }
    }
  }
  // acc[rs][t][v] is row 32 rs + (v%4) + 4h + 8(v/4), column n of the t-th 32x32 tile
#pragma unroll
  for (int rs = 0; rs < RS; ++rs) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int fcol = f0 + (wave * NT + t) * 32;
      if (fcol >= feat) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = 32 * rs + (v & 3) + 4 * h + 8 * (v >> 2);
        const int64_t off = ((int64_t)i_out * blk + bi0 + row) * feat + fcol + n;
        if constexpr (OUT == 1)
          static_cast<float*>(Y)[off] = acc[rs][t][v];
        else
          static_cast<uint16_t*>(Y)[off] = to16<BF16>(acc[rs][t][v]);
      }
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

}  // namespace

static int bsr_launch(int32_t dtype, int32_t out_dtype, int32_t mb, int32_t nb, int32_t blk, int32_t feat,
                      int64_t nnzb, const void* d_A, const void* d_X, void* d_Y, const int32_t* d_indptr,
                      const int32_t* d_indices, const int32_t* d_row_ids, void* stream) {
  STIR_REQUIRE(dtype == STIR_F16 || dtype == STIR_BF16, "bsr_spmm: dtype must be STIR_F16 or STIR_BF16");
  STIR_REQUIRE(out_dtype == dtype || out_dtype == STIR_F32, "bsr_spmm: out_dtype must equal dtype or be STIR_F32");
  STIR_REQUIRE(mb >= 0 && nb >= 0 && nnzb >= 0, "bsr_spmm: bad sizes mb=%d nb=%d", mb, nb);
  STIR_REQUIRE(blk > 0 && blk % 32 == 0, "bsr_spmm: blk=%d must be a multiple of 32", blk);
  STIR_REQUIRE(feat > 0 && feat % 32 == 0, "bsr_spmm: feat=%d must be a multiple of 32", feat);
  if (mb == 0) return 0;
  STIR_REQUIRE(d_X && d_Y && d_indptr && (nnzb == 0 || (d_A && d_indices)), "bsr_spmm: null pointer argument");
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
  // register rings (2-6 steps) change nothing, the kernel is bound by the traffic that misses
  // the per-XCD L2, not by latency.
  const int nt = (feat >= 1024) ? 2 : 1;
  const int f_tiles = (int)stir::ceil_div(feat, kTileF * nt);
  const int64_t blocks = f_tiles >= 8 ? 8 * stir::ceil_div(f_tiles, 8) * slices : (int64_t)f_tiles * slices;
  STIR_REQUIRE(blocks < (int64_t(1) << 31), "bsr_spmm: too many tiles for one launch");
  dim3 grid((unsigned)blocks), block(256);
#define STIR_BSR_L(BF, OUT, NTV, RSV)                                                                      \
  hipLaunchKernelGGL((bsr_spmm_kernel<BF, OUT, NTV, 1, RSV>), grid, block, 0, st, blk, feat, slices, f_tiles, \
                     A, X, d_Y, d_indptr, d_indices, d_row_ids)
#define STIR_BSR(BF, OUT)                                                          \
  do {                                                                             \
    if (nt == 2) {                                                                 \
      if (rs == 2) STIR_BSR_L(BF, OUT, 2, 2); else STIR_BSR_L(BF, OUT, 2, 1);      \
    } else {                                                                       \
      if (rs == 2) STIR_BSR_L(BF, OUT, 1, 2); else STIR_BSR_L(BF, OUT, 1, 1);      \
    }                                                                              \
  } while (0)
  if (dtype == STIR_BF16) {
    if (out_dtype == STIR_F32) STIR_BSR(true, 1); else STIR_BSR(true, 0);
  } else {
    if (out_dtype == STIR_F32) STIR_BSR(false, 1); else STIR_BSR(false, 0);
  }
#undef STIR_BSR
#undef STIR_BSR_L
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
