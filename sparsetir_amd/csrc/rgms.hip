// RGMS (relational gather-matmul-scatter) on the gfx950 matrix cores, fp16 in, fp32 out:
//   Y[row, :] += sum over ELL slots s of the row  A[s] * (X[col[s], :] @ W[rel])
// on the bucketed ELL3D layout (group -> rb ELL rows -> cb slots; one relation per group).
//
// A wavefront owns one group and walks it 32 slots at a time.  The 32 gathered X rows are the
// MFMA A operand: lane (m, h) needs 8 consecutive input features of slot m, which is one
// 16-byte load from the gathered row -- no staging.  W[rel] is the B operand; its fragments
// are loaded once per group and stay in registers.  The 32x32 fp32 result tile is scaled by
// the slot weights, summed over the slots of each ELL row inside the wavefront (register adds
// plus one cross-half exchange) and added to Y with one fp32 atomic per (ELL row, feature).
#include "common.h"
#include "../../include/sparsetir_amd.h"

namespace {

using stir::kWave;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct alignas(16) RgmsBucket {
  const uint16_t* A;    // fp16 slot weights, groups*rb*cb
  const int32_t* rows;  // groups*rb
  const int32_t* cols;  // groups*rb*cb
  const int32_t* mids;  // groups
  int64_t groups;
  int64_t group_begin;  // first group of this bucket in the fused launch
  int32_t rb, cb;
  int32_t log2cb;  // log2(cb) when cb is a power of two <= 32, else -1
  int32_t pad;
};

constexpr int kMaxKK = 8;  // feat_in <= 128 keeps the X operand in registers

__device__ __forceinline__ float half_bits_to_float(uint16_t b) {
  return (float)__builtin_bit_cast(_Float16, b);
}

__device__ __forceinline__ void atomic_addf(float* p, float v) {
  __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// KK = feat_in / 16.  grid: one wavefront per group (4 per workgroup); feat_out tiles of 32
// are walked inside.
template <int KK>
__global__ __launch_bounds__(256) void rgms_kernel(const RgmsBucket* __restrict__ table, int nb,
                                                   int64_t total_groups, int feat_out,
                                                   const uint16_t* __restrict__ W,
                                                   const uint16_t* __restrict__ X, float* __restrict__ Y) {
  constexpr int FIN = KK * 16;
  const int lane = threadIdx.x & 63;
  const int n = lane & 31, h = lane >> 5;
  const int64_t gid = (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (gid >= total_groups) return;
  int lo = 0, hi = nb - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[mid].group_begin <= gid) lo = mid; else hi = mid - 1;
  }
  const RgmsBucket bk = table[lo];
  const int64_t g = gid - bk.group_begin;
  const int rel = bk.mids[g];
  const int gsize = bk.rb * bk.cb;
  const uint16_t* Ag = bk.A + g * gsize;
  const int32_t* colg = bk.cols + g * gsize;
  const int32_t* rowg = bk.rows + g * bk.rb;
  const uint16_t* Wr = W + (int64_t)rel * FIN * feat_out;

  for (int nt = 0; nt < feat_out; nt += 32) {
    // B operand: W[rel][16kk + 8h + e][nt + n], e = 0..7
    u32x4 wf[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const uint16_t* wp = Wr + (int64_t)(16 * kk + 8 * h + 2 * d) * feat_out + nt + n;
        wf[kk][d] = (uint32_t)wp[0] | ((uint32_t)wp[feat_out] << 16);
      }
    }
    for (int s0 = 0; s0 < gsize; s0 += 32) {
      const int slot = s0 + n;  // this lane's slot as the A-operand row
      const bool live = slot < gsize;
      const int col = live ? colg[slot] : 0;
      f32x16 acc;
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[v] = 0.f;
      const uint16_t* xp = X + (int64_t)col * FIN + 8 * h;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        const u32x4 xa = *reinterpret_cast<const u32x4*>(xp + 16 * kk);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, xa),
                                                    __builtin_bit_cast(f16x8, wf[kk]), acc, 0, 0, 0);
      }
      // acc[v]: slot s0 + (v%4) + 4h + 8(v/4), output feature nt + n.  Scale by slot weight.
      float wgt[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int sl = s0 + (v & 3) + 4 * h + 8 * (v >> 2);
        wgt[v] = sl < gsize ? half_bits_to_float(Ag[sl]) : 0.f;
        acc[v] *= wgt[v];
      }
      float* yb = Y + nt + n;
      if (bk.log2cb < 0 || bk.log2cb == 0) {
        // one atomic per slot (zero-weight slots contribute nothing and are skipped)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int sl = s0 + (v & 3) + 4 * h + 8 * (v >> 2);
          if (wgt[v] != 0.f) atomic_addf(yb + (int64_t)rowg[sl / bk.cb] * feat_out, acc[v]);
        }
      } else if (bk.log2cb == 1) {
#pragma unroll
        for (int v = 0; v < 16; v += 2) {
          const int sl = s0 + (v & 3) + 4 * h + 8 * (v >> 2);
          if (sl < gsize) atomic_addf(yb + (int64_t)rowg[sl >> 1] * feat_out, acc[v] + acc[v + 1]);
        }
      } else {
        // cb >= 4: the four registers of a quad belong to one ELL row
        float q[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) q[t] = (acc[4 * t] + acc[4 * t + 1]) + (acc[4 * t + 2] + acc[4 * t + 3]);
        if (bk.log2cb == 2) {
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int sl = s0 + 4 * h + 8 * t;
            if (sl < gsize) atomic_addf(yb + (int64_t)rowg[sl >> 2] * feat_out, q[t]);
          }
        } else {
          // cb >= 8: add the other half-wave's quad (slots 8t+4..8t+7 vs 8t..8t+3)
#pragma unroll
          for (int t = 0; t < 4; ++t) q[t] += __shfl_xor(q[t], 32, kWave);
          if (bk.log2cb == 3) {
            // four ELL rows per tile; half h writes rows 2h, 2h+1
#pragma unroll
            for (int t = 0; t < 2; ++t) {
              const int tt = 2 * h + t;
              const int sl = s0 + 8 * tt;
              const float val = tt == 0 ? q[0] : tt == 1 ? q[1] : tt == 2 ? q[2] : q[3];
              if (sl < gsize) atomic_addf(yb + (int64_t)rowg[sl >> 3] * feat_out, val);
            }
          } else if (bk.log2cb == 4) {
            const float val = h == 0 ? q[0] + q[1] : q[2] + q[3];
            const int sl = s0 + 16 * h;
            if (sl < gsize) atomic_addf(yb + (int64_t)rowg[sl >> 4] * feat_out, val);
          } else {  // cb == 32: the whole tile is one ELL row
            const float val = (q[0] + q[1]) + (q[2] + q[3]);
            if (h == 0) atomic_addf(yb + (int64_t)rowg[s0 >> 5] * feat_out, val);
          }
        }
      }
    }
  }
}

}  // namespace

struct stir_rgms_plan {
  int nk;
  RgmsBucket* d_table;
  int64_t total_groups;
};

extern "C" {

int stir_rgms_plan_create(stir_rgms_plan** plan, int32_t num_buckets, const int32_t* rows_bkt,
                          const int32_t* cols_bkt, const int64_t* groups, const void* const* d_A,
                          const int32_t* const* d_rows, const int32_t* const* d_cols,
                          const int32_t* const* d_mids) {
  STIR_REQUIRE(plan && num_buckets > 0, "rgms_plan_create: bad arguments");
  RgmsBucket* host = new RgmsBucket[num_buckets];
  int nk = 0;
  int64_t total = 0;
  for (int b = 0; b < num_buckets; ++b) {
    if (rows_bkt[b] <= 0 || cols_bkt[b] <= 0 || groups[b] < 0) {
      delete[] host;
      return stir::fail("rgms_plan_create: bucket %d has non-positive sizes", b);
    }
    if (groups[b] == 0) continue;
    if (!d_A[b] || !d_rows[b] || !d_cols[b] || !d_mids[b]) {
      delete[] host;
      return stir::fail("rgms_plan_create: bucket %d has groups but a null array", b);
    }
    RgmsBucket e;
    e.A = static_cast<const uint16_t*>(d_A[b]);
    e.rows = d_rows[b];
    e.cols = d_cols[b];
    e.mids = d_mids[b];
    e.groups = groups[b];
    e.group_begin = total;
    e.rb = rows_bkt[b];
    e.cb = cols_bkt[b];
    e.log2cb = -1;
    // the in-wavefront row reduction needs ELL rows aligned to the 32-slot tiles
    if (stir::is_pow2(cols_bkt[b]) && cols_bkt[b] <= 32) {
      int l = 0;
      while ((1 << l) < cols_bkt[b]) ++l;
      e.log2cb = l;
    }
    e.pad = 0;
    host[nk++] = e;
    total += groups[b];
  }
  stir_rgms_plan* p = new stir_rgms_plan();
  p->nk = nk;
  p->total_groups = total;
  p->d_table = nullptr;
  hipError_t err = hipSuccess;
  if (nk > 0) {
    err = hipMalloc(reinterpret_cast<void**>(&p->d_table), sizeof(RgmsBucket) * nk);
    if (err == hipSuccess) err = hipMemcpy(p->d_table, host, sizeof(RgmsBucket) * nk, hipMemcpyHostToDevice);
  }
  delete[] host;
  if (err != hipSuccess) {
    if (p->d_table) (void)hipFree(p->d_table);
    delete p;
    return stir::fail("rgms_plan_create: %s", hipGetErrorString(err));
  }
  *plan = p;
  return 0;
}

int stir_rgms_f16(const stir_rgms_plan* plan, int32_t m, int32_t n, int32_t num_rels,
                  int32_t feat_in, int32_t feat_out, const void* d_W, const void* d_X, float* d_Y,
                  void* stream) {
  STIR_REQUIRE(plan, "rgms: plan is null");
  STIR_REQUIRE(m >= 0 && n >= 0 && num_rels >= 0, "rgms: bad sizes");
  STIR_REQUIRE(feat_in > 0 && feat_in % 16 == 0 && feat_in <= 16 * kMaxKK,
               "rgms: feat_in=%d must be a multiple of 16 and at most %d", feat_in, 16 * kMaxKK);
  STIR_REQUIRE(feat_out > 0 && feat_out % 32 == 0, "rgms: feat_out=%d must be a multiple of 32", feat_out);
  if (plan->nk == 0) return 0;
  STIR_REQUIRE(d_W && d_X && d_Y, "rgms: null pointer argument");
  const int64_t blocks = stir::ceil_div(plan->total_groups, 4);
  STIR_REQUIRE(blocks < (int64_t(1) << 31), "rgms: too many groups for one launch");
  dim3 grid((unsigned)blocks), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint16_t* W = static_cast<const uint16_t*>(d_W);
  const uint16_t* X = static_cast<const uint16_t*>(d_X);
#define STIR_RGMS(KK)                                                                              \
  case KK:                                                                                         \
    hipLaunchKernelGGL((rgms_kernel<KK>), grid, block, 0, st, plan->d_table, plan->nk,             \
                       plan->total_groups, feat_out, W, X, d_Y);                                   \
    break
  switch (feat_in / 16) {
    STIR_RGMS(1);
    STIR_RGMS(2);
    STIR_RGMS(3);
    STIR_RGMS(4);
    STIR_RGMS(5);
    STIR_RGMS(6);
    STIR_RGMS(7);
    STIR_RGMS(8);
  }
#undef STIR_RGMS
  STIR_LAUNCH_CHECK();
  return 0;
}

int stir_rgms_plan_destroy(stir_rgms_plan* plan) {
  if (!plan) return 0;
  if (plan->d_table) (void)hipFree(plan->d_table);
  delete plan;
  return 0;
}

}  // extern "C"
