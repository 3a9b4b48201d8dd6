// BSR SpMM on the gfx950 matrix cores: Y[i-th block row] = sum over stored blocks p of
// A_p (blk x blk) * X[indices[p]-th block of rows], 16-bit inputs, fp32 accumulation.
//
// A workgroup of four wavefronts owns one 32-row slice of a block row and a 128-wide slice
// of the feature axis; wavefront w owns features [32w, 32w+32) and accumulates a 32x32 fp32
// tile with v_mfma_f32_32x32x16_{f16,bf16}.  The A operand wants 8 consecutive k per lane,
// which is exactly how a row of a stored block lies in memory, so it is loaded straight from
// global memory (16 bytes per lane).  The X operand wants 8 consecutive k for one feature
// column, but X is feature-contiguous, so the 32 x 128 tile of X goes through LDS: every
// thread loads two adjacent k rows (16 bytes each), interleaves them into (k, k+1) pairs
// and stores 32 bytes; a lane's MFMA operand is then four 4-byte LDS reads.
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

// grid: (mb * (blk/32), ceil(feat/128)); block: 256 threads.
template <bool BF16, int OUT>  // OUT: 0 = same 16-bit type as the inputs, 1 = fp32
__global__ __launch_bounds__(256) void bsr_spmm_kernel(int blk, int feat, const uint16_t* __restrict__ A,
                                                       const uint16_t* __restrict__ X, void* __restrict__ Y,
                                                       const int32_t* __restrict__ indptr,
                                                       const int32_t* __restrict__ indices) {
  __shared__ uint32_t xs[kTileK / 2][kTileF];  // [k pair][feature] -> (X[2kp][f], X[2kp+1][f])
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, h = lane >> 5;
  const int sub = blk / 32;  // 32-row slices per block row
  const int i = blockIdx.x / sub, bi0 = (blockIdx.x % sub) * 32;
  const int f0 = blockIdx.y * kTileF;
  // staging role: k pair kp, feature chunk fc (8 features)
  const int kp = tid >> 4, fc = tid & 15;
  const bool stage_live = f0 + fc * 8 < feat;  // feat is a multiple of 32, so chunks are whole
  const bool wave_live = f0 + wave * 32 < feat;

  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;

  const int p_begin = indptr[i], p_end = indptr[i + 1];
  for (int p = p_begin; p < p_end; ++p) {
    const int64_t j = indices[p];
    const uint16_t* ablk = A + (int64_t)p * blk * blk + (int64_t)(bi0 + n) * blk;
    for (int k0 = 0; k0 < blk; k0 += kTileK) {
      // ---- stage X[j*blk + k0 .. +32][f0 .. +128] as k pairs
      u32x4 r0 = {0, 0, 0, 0}, r1 = {0, 0, 0, 0};
      if (stage_live) {
        const uint16_t* xp = X + ((int64_t)j * blk + k0 + 2 * kp) * feat + f0 + fc * 8;
        r0 = *reinterpret_cast<const u32x4*>(xp);
        r1 = *reinterpret_cast<const u32x4*>(xp + feat);
      }
      // ---- A operand straight from global: rows bi0+n, k = k0 + 16*kk + 8h + (0..7)
      u32x4 a0 = *reinterpret_cast<const u32x4*>(ablk + k0 + 8 * h);
      u32x4 a1 = *reinterpret_cast<const u32x4*>(ablk + k0 + 16 + 8 * h);
      u32x4 lo, hi;  // (k, k+1) pairs for features fc*8 + 0..3 and 4..7
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        lo[2 * q] = __builtin_amdgcn_perm(r1[q], r0[q], 0x05040100);      // low halves
        lo[2 * q + 1] = __builtin_amdgcn_perm(r1[q], r0[q], 0x07060302);  // high halves
        hi[2 * q] = __builtin_amdgcn_perm(r1[q + 2], r0[q + 2], 0x05040100);
        hi[2 * q + 1] = __builtin_amdgcn_perm(r1[q + 2], r0[q + 2], 0x07060302);
      }
      __syncthreads();  // previous step's readers are done
      *reinterpret_cast<u32x4*>(&xs[kp][fc * 8]) = lo;
      *reinterpret_cast<u32x4*>(&xs[kp][fc * 8 + 4]) = hi;
      __syncthreads();
      if (wave_live) {
        u32x4 b0, b1;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          b0[d] = xs[4 * h + d][wave * 32 + n];
          b1[d] = xs[8 + 4 * h + d][wave * 32 + n];
        }
        acc = mfma32<BF16>(a0, b0, acc);
        acc = mfma32<BF16>(a1, b1, acc);
      }
    }
  }
  if (!wave_live) return;
  // acc[v] is row (v%4) + 4h + 8(v/4), column n of the 32x32 tile
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int row = (v & 3) + 4 * h + 8 * (v >> 2);
    const int64_t off = ((int64_t)i * blk + bi0 + row) * feat + f0 + wave * 32 + n;
    if constexpr (OUT == 1)
      static_cast<float*>(Y)[off] = acc[v];
    else
      static_cast<uint16_t*>(Y)[off] = to16<BF16>(acc[v]);
  }
}

}  // namespace

extern "C" int stir_bsr_spmm(int32_t dtype, int32_t out_dtype, int32_t mb, int32_t nb, int32_t blk,
                             int32_t feat, int64_t nnzb, const void* d_A, const void* d_X, void* d_Y,
                             const int32_t* d_indptr, const int32_t* d_indices, void* stream) {
  STIR_REQUIRE(dtype == STIR_F16 || dtype == STIR_BF16, "bsr_spmm: dtype must be STIR_F16 or STIR_BF16");
  STIR_REQUIRE(out_dtype == dtype || out_dtype == STIR_F32, "bsr_spmm: out_dtype must equal dtype or be STIR_F32");
  STIR_REQUIRE(mb >= 0 && nb >= 0 && nnzb >= 0, "bsr_spmm: bad sizes mb=%d nb=%d", mb, nb);
  STIR_REQUIRE(blk > 0 && blk % 32 == 0, "bsr_spmm: blk=%d must be a multiple of 32", blk);
  STIR_REQUIRE(feat > 0 && feat % 32 == 0, "bsr_spmm: feat=%d must be a multiple of 32", feat);
  if (mb == 0) return 0;
  STIR_REQUIRE(d_X && d_Y && d_indptr && (nnzb == 0 || (d_A && d_indices)), "bsr_spmm: null pointer argument");
  const int64_t gx = (int64_t)mb * (blk / 32);
  STIR_REQUIRE(gx < (int64_t(1) << 31), "bsr_spmm: too many block rows for one launch");
  dim3 grid((unsigned)gx, (unsigned)stir::ceil_div(feat, kTileF)), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint16_t* A = static_cast<const uint16_t*>(d_A);
  const uint16_t* X = static_cast<const uint16_t*>(d_X);
#define STIR_BSR(BF, OUT) \
  hipLaunchKernelGGL((bsr_spmm_kernel<BF, OUT>), grid, block, 0, st, blk, feat, A, X, d_Y, d_indptr, d_indices)
  if (dtype == STIR_BF16) {
    if (out_dtype == STIR_F32) STIR_BSR(true, 1); else STIR_BSR(true, 0);
  } else {
    if (out_dtype == STIR_F32) STIR_BSR(false, 1); else STIR_BSR(false, 0);
  }
#undef STIR_BSR
  STIR_LAUNCH_CHECK();
  return 0;
}
