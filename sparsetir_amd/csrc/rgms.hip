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
// This kernel serves small inputs; from kTileMinSlots slots on, the destination-tiled kernel of
// rgms_tiles.hip (no atomics) takes over.
#include <vector>

#include "common.h"
#include "rgms_out.h"
#include "rgms_tiles.h"
#include "../../include/sparsetir_amd.h"

namespace {

using stir::kWave;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct alignas(16) RgmsBucket {
  const uint16_t* A;    // fp16 slot weights, groups*rb*cb
  const int32_t* rows;  // groups*rb
  const int32_t* cols;  // groups*rb*cb
  const int32_t* mids;  // groups
  int64_t groups;
  int64_t unit_begin;  // first work unit (one wavefront each) of this bucket in the fused launch
  int32_t rb, cb;
  int32_t log2cb;  // log2(cb) when cb is a power of two <= 32, else -1
  int32_t chunks;  // work units per group: ceil(rb*cb / kChunkSlots)
};

// A wavefront processes this many consecutive slots of one group.
constexpr int kChunkSlots = 128;

constexpr int kMaxKK = 8;  // feat_in <= 128 keeps the X operand in registers

// 16-bit storage type of W, X and the slot weights: fp16, or bf16 with BF16
template <bool BF16>
__device__ __forceinline__ float bits_to_float(uint16_t b) {
  if constexpr (BF16)
    return __uint_as_float((uint32_t)b << 16);
  else
    return (float)__builtin_bit_cast(_Float16, b);
}

template <bool BF16>
__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
}

// One group (one relation), one wavefront.  KK = feat_in / 16; LCB = log2(cb) for power-of-two
// cb <= 32, else -1.  The group is processed in chunks of TI tiles (32 slots each): the chunk's
// column ids, slot weights and row ids are fetched with a few coalesced loads (lane l holds slots
// l, l+64, ...), then the X rows of all TI tiles are requested at once, so a chunk costs two
// memory latencies instead of several per tile.
template <int KK, int LCB, bool BF16, typename YT>
__device__ __forceinline__ void rgms_group(const RgmsBucket& bk, int64_t g, int chunk, int feat_out,
                                           const uint16_t* __restrict__ W, const uint16_t* __restrict__ X,
                                           YT* __restrict__ Y, int lane) {
  constexpr int FIN = KK * 16;
  constexpr int TI = KK <= 2 ? 4 : 2;  // tiles in flight
  constexpr int MJ = TI / 2;           // 64-slot metadata registers per lane
  const int n = lane & 31, h = lane >> 5;
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
    YT* yb = Y + nt + n;
    // result of an ELL row with output row `row`, added where `on` holds (the same for every n)
    auto emit = [&](bool on, int row, float v) { stir::y_atomic_add(yb + (int64_t)row * feat_out, v, on, lane); };
    const int s_end = min(gsize, (chunk + 1) * kChunkSlots);
#pragma unroll 1
    for (int s_base = chunk * kChunkSlots; s_base < s_end; s_base += 32 * TI) {
      // ---- chunk metadata: slot s_base + 64j + lane lives in register j of this lane
      int mcol[MJ], mrow[MJ];
      float mw[MJ];
#pragma unroll
      for (int j = 0; j < MJ; ++j) {
        const int sl = s_base + 64 * j + lane;
        const bool live = sl < gsize;
        mcol[j] = live ? colg[sl] : 0;
        mw[j] = live ? bits_to_float<BF16>(Ag[sl]) : 0.f;
        // ELL rows of the chunk (power-of-two cb): row (s_base >> LCB) + 64j + lane
        mrow[j] = 0;
        if constexpr (LCB >= 0) {
          const int r = (s_base >> LCB) + 64 * j + lane;
          if (r < bk.rb) mrow[j] = rowg[r];
        }
      }
      // ---- request the X rows of every tile of the chunk (tiles past the group read row 0)
      u32x4 xa[TI][KK];
#pragma unroll
      for (int t = 0; t < TI; ++t) {
        const int col = __shfl(mcol[t >> 1], 32 * (t & 1) + n, kWave);
        const uint16_t* xp = X + (int64_t)col * FIN + 8 * h;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) xa[t][kk] = *reinterpret_cast<const u32x4*>(xp + 16 * kk);
      }
#pragma unroll
      for (int t = 0; t < TI; ++t) {
        const bool tile_live = s_base + 32 * t < gsize;  // uniform
        // keep the tiles' instruction streams apart: interleaving them would hold every tile's
        // accumulators, weights and row ids live at once
        __builtin_amdgcn_sched_barrier(0);
        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
          acc = mfma32<BF16>(xa[t][kk], wf[kk], acc);
        // acc[v]: slot 32t + (v%4) + 4h + 8(v/4) of the chunk, output feature nt + n.
        // Scale by the slot weight (zero beyond the group).
        float wgt[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          wgt[v] = __shfl(mw[t >> 1], 32 * (t & 1) + (v & 3) + 4 * h + 8 * (v >> 2), kWave);
          acc[v] *= wgt[v];
        }
        // row id of ELL row q of the chunk; its register index j is a compile-time constant
        auto row_of = [&](int q, int j) { return __shfl(mrow[j < MJ ? j : 0], q & 63, kWave); };
        if constexpr (LCB < 0) {
          // cb is not a power of two: one atomic per slot, row ids read directly
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int sl = s_base + 32 * t + (v & 3) + 4 * h + 8 * (v >> 2);
            emit(wgt[v] != 0.f, wgt[v] != 0.f ? rowg[sl / bk.cb] : 0, acc[v]);
          }
        } else if constexpr (LCB == 0) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int sl = 32 * t + (v & 3) + 4 * h + 8 * (v >> 2);
            const int row = row_of(sl, t >> 1);
            emit(wgt[v] != 0.f, row, acc[v]);
          }
        } else if constexpr (LCB == 1) {
#pragma unroll
          for (int v = 0; v < 16; v += 2) {
            const int sl = 32 * t + (v & 3) + 4 * h + 8 * (v >> 2);
            const int row = row_of(sl >> 1, t >> 2);
            emit(s_base + sl < gsize, row, acc[v] + acc[v + 1]);
          }
        } else {
          // cb >= 4: the four registers of a quad belong to one ELL row
          float q4[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) q4[u] = (acc[4 * u] + acc[4 * u + 1]) + (acc[4 * u + 2] + acc[4 * u + 3]);
          if constexpr (LCB == 2) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const int sl = 32 * t + 4 * h + 8 * u;
              const int row = row_of(sl >> 2, 0);
              emit(s_base + sl < gsize, row, q4[u]);
            }
          } else {
            // cb >= 8: add the other half-wave's quad (slots 8u+4..8u+7 vs 8u..8u+3)
#pragma unroll
            for (int u = 0; u < 4; ++u) q4[u] += __shfl_xor(q4[u], 32, kWave);
            if constexpr (LCB == 3) {
              // four ELL rows per tile; half h writes rows 2h, 2h+1
#pragma unroll
              for (int u = 0; u < 2; ++u) {
                const int tt = 2 * h + u;
                const int sl = 32 * t + 8 * tt;
                const float val = tt == 0 ? q4[0] : tt == 1 ? q4[1] : tt == 2 ? q4[2] : q4[3];
                const int row = row_of(sl >> 3, 0);
                emit(s_base + sl < gsize, row, val);
              }
            } else if constexpr (LCB == 4) {
              const float val = h == 0 ? q4[0] + q4[1] : q4[2] + q4[3];
              const int sl = 32 * t + 16 * h;
              const int row = row_of(sl >> 4, 0);
              emit(s_base + sl < gsize, row, val);
            } else {  // cb == 32: the whole tile is one ELL row
              const float val = (q4[0] + q4[1]) + (q4[2] + q4[3]);
              const int row = row_of(t, 0);
              emit(h == 0 && tile_live, row, val);
            }
          }
        }
        (void)tile_live;
      }
    }
  }
}

// grid: one wavefront per work unit (kChunkSlots slots of one group), 4 per workgroup; feat_out
// tiles of 32 are walked inside.
template <int KK, bool BF16, typename YT>
__global__ __launch_bounds__(256) void rgms_kernel(const RgmsBucket* __restrict__ table, int nb,
                                                   int64_t total_units, int feat_out,
                                                   const uint16_t* __restrict__ W,
                                                   const uint16_t* __restrict__ X, YT* __restrict__ Y) {
  const int lane = threadIdx.x & 63;
  const int64_t gid = (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (gid >= total_units) return;
  int lo = 0, hi = nb - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[mid].unit_begin <= gid) lo = mid; else hi = mid - 1;
  }
  const RgmsBucket bk = table[lo];
  const int64_t unit = gid - bk.unit_begin;
  const int64_t g = unit / bk.chunks;
  const int chunk = (int)(unit % bk.chunks);
  switch (bk.log2cb) {
    case 0: rgms_group<KK, 0, BF16, YT>(bk, g, chunk, feat_out, W, X, Y, lane); break;
    case 1: rgms_group<KK, 1, BF16, YT>(bk, g, chunk, feat_out, W, X, Y, lane); break;
    case 2: rgms_group<KK, 2, BF16, YT>(bk, g, chunk, feat_out, W, X, Y, lane); break;
    case 3: rgms_group<KK, 3, BF16, YT>(bk, g, chunk, feat_out, W, X, Y, lane); break;
    case 4: rgms_group<KK, 4, BF16, YT>(bk, g, chunk, feat_out, W, X, Y, lane); break;
    case 5: rgms_group<KK, 5, BF16, YT>(bk, g, chunk, feat_out, W, X, Y, lane); break;
    default: rgms_group<KK, -1, BF16, YT>(bk, g, chunk, feat_out, W, X, Y, lane); break;
  }
}

}  // namespace

// From this many slots on the destination-tiled kernel is used (its index is built by the first
// launch); below, one launch of the atomic kernel costs less.
constexpr int64_t kTileMinSlots = 8192;

struct stir_rgms_plan {
  int nk;
  RgmsBucket* d_table;
  int64_t total_units;
  // destination-tiled path: the edge index is made by the first launch (it needs m, n and
  // num_rels) and kept
  std::vector<stir::TileBucket> tile_buckets;
  int64_t slots;
  bool static_weights;  // promise of the caller, see stir_rgms_plan_set_static_weights
  bool addresses_only;  // see stir_rgms_plan_set_addresses_only: no edge index, every launch reads the arrays
  stir::TileIndexSet tiles;
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
  std::vector<stir::TileBucket> tile_buckets;
  int64_t slots = 0;
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
    e.unit_begin = total;
    e.rb = rows_bkt[b];
    e.cb = cols_bkt[b];
    e.log2cb = -1;
    // the in-wavefront row reduction needs ELL rows aligned to the 32-slot tiles
    if (stir::is_pow2(cols_bkt[b]) && cols_bkt[b] <= 32) {
      int l = 0;
      while ((1 << l) < cols_bkt[b]) ++l;
      e.log2cb = l;
    }
    e.chunks = (int32_t)stir::ceil_div((int64_t)rows_bkt[b] * cols_bkt[b], kChunkSlots);
    host[nk++] = e;
    total += groups[b] * e.chunks;
    tile_buckets.push_back(stir::TileBucket{e.A, e.rows, e.cols, e.mids, e.groups, e.rb, e.cb});
    slots += e.groups * e.rb * e.cb;
  }
  stir_rgms_plan* p = new stir_rgms_plan();
  p->nk = nk;
  p->total_units = total;
  p->d_table = nullptr;
  p->tile_buckets = tile_buckets;
  p->slots = slots;
  p->static_weights = false;
  p->addresses_only = false;
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

// out16: Y holds fp16 values (fp16 inputs only); otherwise fp32.
static int rgms_launch(bool bf16, bool out16, const stir_rgms_plan* plan, int32_t m, int32_t n, int32_t num_rels,
                       int32_t feat_in, int32_t feat_out, const void* d_W, const void* d_X, void* d_Y,
                       void* stream) {
  STIR_REQUIRE(plan, "rgms: plan is null");
  STIR_REQUIRE(m >= 0 && n >= 0 && num_rels >= 0, "rgms: bad sizes");
  STIR_REQUIRE(feat_in > 0 && feat_in % 16 == 0 && feat_in <= 16 * kMaxKK,
               "rgms: feat_in=%d must be a multiple of 16 and at most %d", feat_in, 16 * kMaxKK);
  STIR_REQUIRE(feat_out > 0 && feat_out % 32 == 0, "rgms: feat_out=%d must be a multiple of 32", feat_out);
  if (plan->nk == 0) return 0;
  STIR_REQUIRE(d_W && d_X && d_Y, "rgms: null pointer argument");
  STIR_REQUIRE(!out16 || reinterpret_cast<uintptr_t>(d_Y) % 4 == 0, "rgms: an fp16 Y must be 4-byte aligned");
  const int64_t blocks = stir::ceil_div(plan->total_units, 4);
  STIR_REQUIRE(blocks < (int64_t(1) << 31), "rgms: too many groups for one launch");
  dim3 grid((unsigned)blocks), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint16_t* W = static_cast<const uint16_t*>(d_W);
  const uint16_t* X = static_cast<const uint16_t*>(d_X);
  if (!plan->addresses_only && plan->slots >= kTileMinSlots && plan->slots < (int64_t(1) << 31)) {
    // the plan's edge index and packed copy of W are filled in by the launches: a plan serves
    // one call at a time
    stir_rgms_plan* mp = const_cast<stir_rgms_plan*>(plan);
    if (stir::tile_set_prepare(mp->tiles, mp->tile_buckets, m, n, num_rels, feat_in, feat_out, mp->static_weights, st))
      return -1;
    return stir::tile_set_launch(bf16, out16, mp->tiles, feat_in, feat_out, d_W, d_X, d_Y, st);
  }
#define STIR_RGMS_GO(KK, BF, YT)                                                               \
  hipLaunchKernelGGL((rgms_kernel<KK, BF, YT>), grid, block, 0, st, plan->d_table, plan->nk,   \
                     plan->total_units, feat_out, W, X, static_cast<YT*>(d_Y))
#define STIR_RGMS(KK)                                     \
  case KK:                                                \
    if (out16)                                            \
      STIR_RGMS_GO(KK, false, _Float16);                  \
    else if (bf16)                                        \
      STIR_RGMS_GO(KK, true, float);                      \
    else                                                  \
      STIR_RGMS_GO(KK, false, float);                     \
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
#undef STIR_RGMS_GO
  STIR_LAUNCH_CHECK();
  return 0;
}

int stir_rgms_f16(const stir_rgms_plan* plan, int32_t m, int32_t n, int32_t num_rels, int32_t feat_in,
                  int32_t feat_out, const void* d_W, const void* d_X, float* d_Y, void* stream) {
  return rgms_launch(false, false, plan, m, n, num_rels, feat_in, feat_out, d_W, d_X, d_Y, stream);
}

int stir_rgms_f16_out_f16(const stir_rgms_plan* plan, int32_t m, int32_t n, int32_t num_rels, int32_t feat_in,
                          int32_t feat_out, const void* d_W, const void* d_X, void* d_Y, void* stream) {
  return rgms_launch(false, true, plan, m, n, num_rels, feat_in, feat_out, d_W, d_X, d_Y, stream);
}

int stir_rgms_bf16(const stir_rgms_plan* plan, int32_t m, int32_t n, int32_t num_rels, int32_t feat_in,
                   int32_t feat_out, const void* d_W, const void* d_X, float* d_Y, void* stream) {
  return rgms_launch(true, false, plan, m, n, num_rels, feat_in, feat_out, d_W, d_X, d_Y, stream);
}

int stir_rgms_plan_set_static_weights(stir_rgms_plan* plan, int32_t on) {
  STIR_REQUIRE(plan, "rgms_plan_set_static_weights: plan is null");
  STIR_REQUIRE(plan->tiles.m < 0 || plan->static_weights == (on != 0),
               "rgms_plan_set_static_weights: the plan has been launched already");
  plan->static_weights = on != 0;
  return 0;
}

int stir_rgms_plan_set_addresses_only(stir_rgms_plan* plan, int32_t on) {
  STIR_REQUIRE(plan, "rgms_plan_set_addresses_only: plan is null");
  STIR_REQUIRE(plan->tiles.m < 0 || plan->addresses_only == (on != 0),
               "rgms_plan_set_addresses_only: the plan has built its edge index already");
  plan->addresses_only = on != 0;
  return 0;
}

int stir_rgms_plan_destroy(stir_rgms_plan* plan) {
  if (!plan) return 0;
  if (plan->d_table) (void)hipFree(plan->d_table);
  stir::tile_set_free(plan->tiles);
  delete plan;
  return 0;
}

}  // extern "C"
