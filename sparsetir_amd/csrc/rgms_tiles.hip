// Destination-tiled RGMS declared in rgms_tiles.h: index construction and the MFMA kernel.
//
// Per step a wavefront takes the next 32 edges of its tile (sorted by relation, then row):
//   stage 1  T[e, :] = X[src_e, :] @ W[rel_e]      one MFMA chain per distinct relation of the
//                                                  step; the rows of other relations enter as zeros
//   stage 2  Ytile  += S @ T                       S[i, e] = weight_e if edge e ends in row i
// The gathered X rows are the stage-1 A operand straight from global memory (lane (e, h) loads 8
// consecutive input features of its edge).  T leaves stage 1 in accumulator layout, which is the
// B-operand layout of stage 2 up to a fixed permutation of the edge index; S is laid out with the
// same permutation.  T is split into two (fp16) or three (bf16) 16-bit terms so that stage 2
// keeps fp32 accuracy.  S is assembled in a per-wavefront LDS tile: the lane of edge e stores
// weight_e at (row_e, e), every lane reads its operand row, then the entry is cleared again.
#include "rgms_tiles.h"
#include "rgms_out.h"

#include <hipcub/hipcub.hpp>
#include <type_traits>


namespace stir {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) uint16_t GlobalU16;  // a global-memory load, not a flat one

struct alignas(16) DevBucket {
  const uint16_t* A;
  const int32_t* rows;
  const int32_t* cols;
  const int32_t* mids;
  int64_t slot_begin;  // first slot of the bucket in the numbering over all buckets
  int32_t rb, cb;
};

struct alignas(16) Edge {
  int32_t src;         // row of X
  uint32_t w_lo, w_hi;  // device address of the 16-bit slot weight
  uint32_t rel_dl;     // relation << 5 | destination row inside its tile
};

// Record of an index built for weights that do not change: no address, the weight itself.
struct alignas(8) PackedEdge {
  int32_t src;
  uint32_t w_rel_dl;  // 16-bit weight << 16 | relation << 5 | destination row inside its tile
};
constexpr int kPackedMaxRels = 1 << 11;

struct alignas(16) Unit {
  int64_t edge_begin;
  int32_t edge_count;
  int32_t tile_flag;  // tile << 1 | 1 when the tile has several units (atomic write-back)
};

constexpr int kTileRows = 32;
constexpr int kStepEdges = 32;
constexpr int kMaxKK = 8;
#ifndef STIR_UNIT_WAVES
#define STIR_UNIT_WAVES 4
#endif
constexpr int kUnitWaves = STIR_UNIT_WAVES;  // wavefronts that share a unit

__device__ __forceinline__ int bucket_of(const DevBucket* __restrict__ tab, int nb, int64_t q) {
  int lo = 0, hi = nb - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (tab[mid].slot_begin <= q) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// key = (destination tile, relation - rel_lo, row inside the tile), value = slot
// Slots of a relation outside [rel_lo, rel_lo + rel_count) and, with drop_zero, slots of weight
// zero get the key one past the last tile, so they sort behind every tile and no unit covers them.
__global__ __launch_bounds__(256) void edge_keys_kernel(const DevBucket* __restrict__ tab, int nb, int64_t slots, int m,
                                                        int num_rels, int rel_lo, int rel_count, int drop_zero,
                                                        uint64_t* __restrict__ keys, int32_t* __restrict__ vals,
                                                        int32_t* __restrict__ bad) {
  const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (q >= slots) return;
  const DevBucket bk = tab[bucket_of(tab, nb, q)];
  const int64_t local = q - bk.slot_begin;
  const int64_t gs = (int64_t)bk.rb * bk.cb;
  const int64_t g = local / gs;
  const int r = (int)((local - g * gs) / bk.cb);
  int dest = bk.rows[g * bk.rb + r];
  int rel = bk.mids[g];
  if ((unsigned)dest >= (unsigned)m || (unsigned)rel >= (unsigned)num_rels) {
    *bad = 1;
    dest = rel = 0;
  }
  rel -= rel_lo;
  uint64_t key = ((((uint64_t)(dest >> 5)) * rel_count + rel) << 5) | (uint64_t)(dest & 31);
  if ((unsigned)rel >= (unsigned)rel_count || (drop_zero && (bk.A[local] & 0x7fff) == 0))
    key = ((uint64_t)((m + kTileRows - 1) / kTileRows) * rel_count) << 5;
  keys[q] = key;
  vals[q] = (int32_t)q;
}

template <typename Rec>
__global__ __launch_bounds__(256) void edge_records_kernel(const DevBucket* __restrict__ tab, int nb, int64_t slots,
                                                           int64_t kept, int n, int num_rels,
                                                           const uint64_t* __restrict__ keys,
                                                           const int32_t* __restrict__ vals, Rec* __restrict__ edges,
                                                           int32_t* __restrict__ bad) {
  const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (p >= slots) return;
  const int64_t q = vals[p];
  const DevBucket bk = tab[bucket_of(tab, nb, q)];
  const int64_t local = q - bk.slot_begin;
  int src = bk.cols[local];
  if ((unsigned)src >= (unsigned)n) {
    *bad = 2;
    src = 0;
  }
  const uint64_t key = keys[p];
  const uint32_t rel_dl = (uint32_t)(((key >> 5) % (uint64_t)num_rels) << 5) | (uint32_t)(key & 31);
  Rec e;
  e.src = src;
  if constexpr (sizeof(Rec) == sizeof(PackedEdge)) {
    e.w_rel_dl = ((uint32_t)bk.A[local] << 16) | rel_dl;
  } else {
    const uint64_t addr = reinterpret_cast<uint64_t>(bk.A + local);
    e.w_lo = (uint32_t)addr;
    e.w_hi = (uint32_t)(addr >> 32);
    e.rel_dl = rel_dl;
  }
  if (p < kept) edges[p] = e;  // the slots behind the last tile are checked, not recorded
}

// begin[t] = first sorted edge of tile t (t = tiles gives the edge count)
__global__ __launch_bounds__(256) void tile_bounds_kernel(const uint64_t* __restrict__ keys, int64_t slots,
                                                          int64_t tiles, int num_rels, int64_t* __restrict__ begin) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t > tiles) return;
  const uint64_t target = ((uint64_t)t * num_rels) << 5;
  int64_t lo = 0, hi = slots;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (keys[mid] < target) lo = mid + 1; else hi = mid;
  }
  begin[t] = lo;
}

// A tile of up to 1.5 * cap steps is one unit; longer ones are cut into units of cap steps.
__device__ __forceinline__ int units_of(int64_t edges, int cap) {
  const int64_t steps = (edges + kStepEdges - 1) / kStepEdges;
  if (steps == 0) return 0;
  if (steps <= cap + cap / 2) return 1;
  return (int)((steps + cap - 1) / cap);
}

__global__ __launch_bounds__(256) void unit_count_kernel(const int64_t* __restrict__ begin, int64_t tiles, int cap,
                                                         int32_t* __restrict__ count) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t > tiles) return;
  count[t] = t < tiles ? units_of(begin[t + 1] - begin[t], cap) : 0;
}

__global__ __launch_bounds__(256) void unit_fill_kernel(const int64_t* __restrict__ begin,
                                                        const int32_t* __restrict__ unit_begin, int64_t tiles, int cap,
                                                        Unit* __restrict__ units) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= tiles) return;
  const int64_t e0 = begin[t], e1 = begin[t + 1];
  const int nu = units_of(e1 - e0, cap);
  const int64_t per = nu == 1 ? e1 - e0 : (int64_t)cap * kStepEdges;
  for (int u = 0; u < nu; ++u) {
    Unit un;
    un.edge_begin = e0 + u * per;
    un.edge_count = (int32_t)min(per, e1 - un.edge_begin);
    un.tile_flag = (int32_t)(t << 1) | (nu > 1 ? 1 : 0);
    units[unit_begin[t] + u] = un;
  }
}

__global__ __launch_bounds__(256) void unit_sort_keys_kernel(const Unit* __restrict__ units, int64_t n,
                                                             int32_t* __restrict__ keys, int32_t* __restrict__ vals) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  keys[i] = units[i].edge_count;
  vals[i] = (int32_t)i;
}

__global__ __launch_bounds__(256) void unit_permute_kernel(const Unit* __restrict__ in, const int32_t* __restrict__ order,
                                                           int64_t n, Unit* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = in[order[i]];
}

// W[rel][16kk + 8h + 2d (+1)][32nt + n] -> operand word d of lane (n, h), one wavefront per
// (rel, nt, kk)
__global__ __launch_bounds__(256) void pack_w_kernel(const uint16_t* __restrict__ W, u32x4* __restrict__ Wp,
                                                     int64_t frags, int kk_count, int feat_out) {
  const int lane = threadIdx.x & 63, n = lane & 31, h = lane >> 5;
  const int64_t f = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (f >= frags) return;
  const int ntiles = feat_out / 32;
  const int kk = (int)(f % kk_count);
  const int nt = (int)((f / kk_count) % ntiles);
  const int64_t rel = f / ((int64_t)kk_count * ntiles);
  const uint16_t* w = W + (rel * kk_count * 16 + 16 * kk + 8 * h) * feat_out + 32 * nt + n;
  u32x4 v;
#pragma unroll
  for (int d = 0; d < 4; ++d)
    v[d] = (uint32_t)w[(int64_t)(2 * d) * feat_out] | ((uint32_t)w[(int64_t)(2 * d + 1) * feat_out] << 16);
  Wp[f * 64 + lane] = v;
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

// acc += S-operand @ (8 rows of T held as fp32 in t[0..7]), T split into 16-bit terms whose sum
// carries at least 21 significant bits -- or, with ONE_TERM (an fp16 Y, which keeps 11 bits),
// rounded to fp16 once.
template <bool BF16, bool ONE_TERM>
__device__ __forceinline__ f32x16 stage2(u32x4 sa, const float* t, f32x16 acc) {
  if constexpr (ONE_TERM) {
    static_assert(!BF16, "one term: fp16 only");
    typedef _Float16 r2 __attribute__((ext_vector_type(2)));
    u32x4 b;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const r2 pair = {(_Float16)t[2 * d], (_Float16)t[2 * d + 1]};  // round to nearest
      b[d] = __builtin_bit_cast(uint32_t, pair);
    }
    acc = mfma32<false>(sa, b, acc);
  } else if constexpr (BF16) {
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = t[i];
#pragma unroll
    for (int term = 0; term < 3; ++term) {
      u32x4 b;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const uint32_t lo = __float_as_uint(r[2 * d]), hi = __float_as_uint(r[2 * d + 1]);
        b[d] = __builtin_amdgcn_perm(hi, lo, 0x07060302);  // the two upper halves (truncation)
        r[2 * d] -= __uint_as_float(lo & 0xffff0000u);
        r[2 * d + 1] -= __uint_as_float(hi & 0xffff0000u);
      }
      acc = mfma32<true>(sa, b, acc);
    }
  } else {
    typedef __fp16 h2 __attribute__((ext_vector_type(2)));
    u32x4 bh, bl;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const h2 hi = __builtin_amdgcn_cvt_pkrtz(t[2 * d], t[2 * d + 1]);
      bh[d] = __builtin_bit_cast(uint32_t, hi);
      // residuals t - hi with the fp16 halves read in place (one instruction each instead of a
      // conversion and a subtraction)
      float r0, r1;
      asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel_hi:[1,0,0]" : "=v"(r0) : "v"(bh[d]), "v"(t[2 * d]));
      asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r1) : "v"(bh[d]), "v"(t[2 * d + 1]));
      const h2 lo = __builtin_amdgcn_cvt_pkrtz(r0, r1);
      bl[d] = __builtin_bit_cast(uint32_t, lo);
    }
    acc = mfma32<false>(sa, bh, acc);
    acc = mfma32<false>(sa, bl, acc);
  }
  return acc;
}

constexpr int kSStride = 40;  // 16-bit elements per row of the S tile (32 used; 80-byte rows)

// Stage 2 of a step: acc2 += S @ T, with T = acc1 as it left stage 1 and S[i, e] = weight of edge e
// if it ends in row i of the tile.  The lane of edge e (lanes 0..31) puts its weight at
// (dl, jcol) of the wavefront's all-zero S tile, every lane reads its operand row, and the entry
// is cleared again; LDS operations of one wavefront execute in order, so no barrier is needed.
// Steps of at most 16 edges skip the second half of k.
template <bool BF16, bool ONE_TERM>
__device__ __forceinline__ f32x16 scatter_step(uint16_t* S, int dl, int jcol, int mrow, int h, uint16_t weight,
                                               int left, const f32x16& acc1, f32x16 acc2) {
  if (h == 0) S[dl * kSStride + jcol] = weight;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  const u32x4 sa0 = *reinterpret_cast<const u32x4*>(S + mrow * kSStride + 8 * h);
  u32x4 sa1 = {0u, 0u, 0u, 0u};
  if (left > 16) sa1 = *reinterpret_cast<const u32x4*>(S + mrow * kSStride + 16 + 8 * h);
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  if (h == 0) S[dl * kSStride + jcol] = 0;
  float t[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) t[v] = acc1[v];
  acc2 = stage2<BF16, ONE_TERM>(sa0, t, acc2);
  if (left > 16) acc2 = stage2<BF16, ONE_TERM>(sa1, t + 8, acc2);
  return acc2;
}

// One workgroup per unit.  Its four wavefronts take the unit's steps in turn (wavefront w the
// steps w, w + 4, ...: more wavefronts in flight per tile, since a step costs a full memory
// round trip), each with its own accumulator tile; the four tiles are added through LDS and the
// workgroup writes the 32 rows of Y once.  KK = feat_in / 16.
template <int KK, bool BF16, typename Rec, typename YT>
__global__ __launch_bounds__(64 * kUnitWaves) void rgms_tile_kernel(const Unit* __restrict__ units,
                                                        const Rec* __restrict__ edges, int m, int feat_out,
                                                        const u32x4* __restrict__ Wp, const uint16_t* __restrict__ X,
                                                        YT* __restrict__ Y) {
  constexpr int FIN = KK * 16;
  constexpr bool kPacked = sizeof(Rec) == sizeof(PackedEdge);
  constexpr int PW = KK <= 4 ? 2 : 1;  // relations whose W fragments are requested together
  constexpr int kThreads = 64 * kUnitWaves, kSumIters = kTileRows * 32 / kThreads;
  __shared__ __attribute__((aligned(16))) uint16_t s_all[kUnitWaves][kTileRows * kSStride];
  __shared__ float partial[kUnitWaves][16 * 64];  // [wavefront][accumulator register][lane]
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t uid = blockIdx.x;
  uint16_t* S = s_all[wave];
  {
    uint32_t* s32 = reinterpret_cast<uint32_t*>(S);
#pragma unroll
    for (int k = 0; k < kTileRows * kSStride / 2 / 64; ++k) s32[lane + 64 * k] = 0;
  }
  const Unit u = units[uid];
  const int mrow = lane & 31, h = lane >> 5;
  const int ntiles = feat_out / 32;
  // Step row e sits at column j of the S tile such that lane (i, h) finds the 8 edges of its
  // stage-2 operand word c at columns 16c + 8h .. +8: these are the rows (t%4) + 4h + 8(2c + t/4)
  // that stage 1 leaves in accumulator registers 8c + t of the lanes of half h.
  const int jcol = 16 * (mrow >> 4) + 8 * ((mrow >> 2) & 1) + 4 * ((mrow >> 3) & 1) + (mrow & 3);
  const int64_t e_end = u.edge_begin + u.edge_count;
  const int tile = u.tile_flag >> 1;

  for (int nti = 0; nti < ntiles; ++nti) {
    f32x16 acc2;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc2[v] = 0.f;
    // lanes past the last edge repeat it with weight zero
    constexpr int64_t kStride = kUnitWaves * kStepEdges;  // edges between a wavefront's steps
    Rec next = edges[min(u.edge_begin + wave * kStepEdges + mrow, e_end - 1)];
    Rec after = edges[min(u.edge_begin + wave * kStepEdges + kStride + mrow, e_end - 1)];
#pragma unroll 1
    for (int64_t e0 = u.edge_begin + wave * kStepEdges; e0 < e_end; e0 += kStride) {
      const Rec cur = next;
      next = after;
      const int left = (int)min((int64_t)kStepEdges, e_end - e0);  // uniform
      const bool live = mrow < left;
      int rel, dl;
      if constexpr (kPacked)
        rel = (int)((cur.w_rel_dl >> 5) & (kPackedMaxRels - 1)), dl = (int)(cur.w_rel_dl & 31);
      else
        rel = (int)(cur.rel_dl >> 5), dl = (int)(cur.rel_dl & 31);
      // the first PW runs of equal relation (the step is sorted by relation)
      int r[PW], pos = 0;
#pragma unroll
      for (int q = 0; q < PW; ++q) {
        r[q] = -1;
        if (pos < kStepEdges) {
          r[q] = __builtin_amdgcn_readlane(rel, pos);
          pos += __popcll(__ballot(rel == r[q]) & 0xffffffffull);
        }
      }
      // every load of the step is requested here; the records of the step after the next go
      // last, so that waiting for the operands leaves them in flight (loads retire in order, so
      // they have until the next step's operands are waited for)
      u32x4 xa[KK], wf[PW][KK];
      const uint16_t* xp = X + (int64_t)cur.src * FIN + 8 * h;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) xa[kk] = *reinterpret_cast<const u32x4*>(xp + 16 * kk);
      uint16_t wbits;
      if constexpr (kPacked)
        wbits = (uint16_t)(cur.w_rel_dl >> 16);
      else
        wbits = *reinterpret_cast<const GlobalU16*>(((uint64_t)cur.w_hi << 32) | cur.w_lo);
#pragma unroll
      for (int q = 0; q < PW; ++q) {
        if (r[q] >= 0) {
          const u32x4* w = Wp + (uint32_t)((r[q] * ntiles + nti) * (KK * 64) + lane);
#pragma unroll
          for (int kk = 0; kk < KK; ++kk) wf[q][kk] = w[kk * 64];
        }
      }
      after = edges[min(e0 + 2 * kStride + mrow, e_end - 1)];  // past the end: the last record again

      // ---- stage 1
      f32x16 acc1;
#pragma unroll
      for (int v = 0; v < 16; ++v) acc1[v] = 0.f;  // a constant operand of the first MFMA, not 16 moves
      auto add_run = [&](int rq, const u32x4* w, f32x16 c) {
        const bool sel = rel == rq;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          u32x4 a;
#pragma unroll
          for (int d = 0; d < 4; ++d) a[d] = sel ? xa[kk][d] : 0u;
          c = mfma32<BF16>(a, w[kk], c);
        }
        return c;
      };
      bool single = pos >= kStepEdges;  // the requested runs cover the step ...
      if constexpr (PW > 1) single = single && r[1] < 0;  // ... and the first one does so alone
      if (single) {
        // one relation in the whole step: nothing to mask
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) acc1 = mfma32<BF16>(xa[kk], wf[0][kk], acc1);
      } else {
        acc1 = add_run(r[0], wf[0], acc1);
#pragma unroll
        for (int q = 1; q < PW; ++q)
          if (r[q] >= 0) acc1 = add_run(r[q], wf[q], acc1);
      }
      while (pos < kStepEdges) {  // steps with more than PW relations: one at a time
        const int rq = __builtin_amdgcn_readlane(rel, pos);
        pos += __popcll(__ballot(rel == rq) & 0xffffffffull);
        const u32x4* w = Wp + (uint32_t)((rq * ntiles + nti) * (KK * 64) + lane);
        u32x4 wl[KK];
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) wl[kk] = w[kk * 64];
        acc1 = add_run(rq, wl, acc1);
      }

      // ---- stage 2
      acc2 = scatter_step<BF16, std::is_same<YT, _Float16>::value>(S, dl, jcol, mrow, h, live ? wbits : (uint16_t)0, left, acc1, acc2);
    }

    // ---- add the four tiles and write back.  acc2[v] of lane (n, h) is row (v%4) + 4h + 8(v/4)
    // of the tile, output feature 32 nti + n.
#pragma unroll
    for (int v = 0; v < 16; ++v) partial[wave][v * 64 + lane] = acc2[v];
    const bool atomic = u.tile_flag & 1;
    float yold[kSumIters];  // requested before the barrier
#pragma unroll
    for (int k = 0; k < kSumIters; ++k) {
      const int elem = threadIdx.x + kThreads * k;
      const int64_t yrow = (int64_t)tile * kTileRows + (elem >> 5);
      yold[k] = (!atomic && yrow < m) ? y_load(Y + yrow * feat_out + 32 * nti + (elem & 31)) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kSumIters; ++k) {
      const int elem = threadIdx.x + kThreads * k, row = elem >> 5, col = elem & 31;
      const int at = ((row & 3) + 4 * (row >> 3)) * 64 + col + 32 * ((row >> 2) & 1);
      float sum = partial[0][at];
#pragma unroll
      for (int w = 1; w < kUnitWaves; ++w) sum += partial[w][at];
      const int64_t yrow = (int64_t)tile * kTileRows + row;
      // (a row belongs to 32 consecutive threads: the two lanes of a pair share `yrow`)
      YT* y = Y + yrow * feat_out + 32 * nti + col;
      if (atomic)  // uniform over the workgroup
        y_atomic_add(y, sum, yrow < m, threadIdx.x);
      else if (yrow < m)
        y_store(y, yold[k] + sum);
    }
    if (nti + 1 < ntiles) __syncthreads();  // the partial sums are rewritten by the next pass
  }
}

// ---- the same computation by resident workgroups that keep all of W in LDS
//
// When W (num_rels x feat_in x feat_out 16-bit values) fits beside the S tiles in the 160 KB of LDS
// of a compute unit, one workgroup per compute unit stays for the whole launch: it brings W into
// LDS once, already in MFMA operand order (so no separate packing launch and no W traffic through
// the vector memory path, which otherwise carries twice the bytes of the gathered X rows), and
// its T teams of two wavefronts each work through one share of the launch.  The shares are cut
// from the sorted edges by the host so that every team gets the same amount of work (build_shares).
// The two wavefronts of a team take the steps of a unit in turn, each with a full 32 x 32 tile of
// partial sums; at the end each keeps 16 rows, receives the partner's part of them through LDS and
// writes them back (teams of four spent a quarter of the launch meeting and summing: 41 against
// 36 us; single wavefronts cut nearly every tile in two and pay for it in atomics: 38 us).
// The X rows of a step are requested one step ahead and the records three steps ahead; a team's
// wavefronts synchronise among themselves only, through a counter in LDS.
constexpr int kSBytes = kTileRows * kSStride * 2;  // S tile of one wavefront
constexpr int kLdsMaxKK = 4;
constexpr int kTeamWaves = 2;  // wavefronts that share a unit in the resident kernel

// lane -> 16-byte slot of its operand inside a fragment of W in LDS: consecutive lanes stay on
// distinct banks, and so do the eight writers of one column phase (see the fill loop)
__device__ __forceinline__ int w_slot(int lane) { return lane ^ ((lane >> 3) & 7); }

template <int KK, bool BF16, typename Rec, int T, typename YT>
__global__ __launch_bounds__(64 * kTeamWaves * T) void rgms_tile_lds_kernel(
    const int32_t* __restrict__ share_ptr, const Unit* __restrict__ share_units, const Rec* __restrict__ edges, int m,
    int feat_out, int num_rels, const uint16_t* __restrict__ W, const uint16_t* __restrict__ X,
    YT* __restrict__ Y) {
  constexpr int FIN = KK * 16;
  constexpr bool kPacked = sizeof(Rec) == sizeof(PackedEdge);
  constexpr int UW = kTeamWaves;
  constexpr int kThreads = 64 * UW * T;  // T teams of two wavefronts
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int ntiles = feat_out / 32;
  const int frags = num_rels * ntiles * KK;
  u32x4* Wl = reinterpret_cast<u32x4*>(lds);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int team = wave / UW, tw = wave % UW;
  const int mrow = lane & 31, h = lane >> 5;
  constexpr int kStride = UW * kStepEdges;  // edges between a wavefront's steps

  // lanes past the last edge of a unit repeat it (with weight zero, see `live`)
  // (indexed from the unit's first edge, so that the lane's part of the address is 32 bits wide)
  auto record = [&](const Unit& un, int e) {
    return (edges + un.edge_begin)[min((uint32_t)(e + mrow), (uint32_t)(un.edge_count - 1))];
  };
  auto weight_of = [&](const Rec& rec) -> uint16_t {
    if constexpr (kPacked)
      return (uint16_t)(rec.w_rel_dl >> 16);
    else
      return *reinterpret_cast<const GlobalU16*>(((uint64_t)rec.w_hi << 32) | rec.w_lo);
  };
  auto fetch = [&](const Rec& rec, u32x4 (&x)[KK], uint16_t& wb) {
    // byte offsets into X fit 32 bits (checked by the host)
    const uint32_t at = (uint32_t)rec.src * (FIN * 2) + 16 * h;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
      x[kk] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const unsigned char*>(X) + at + 32 * kk);
    wb = weight_of(rec);
  };
  // What a pass (one unit, one tile of 32 output features) starts from: the records of the
  // wavefront's first three steps and the rows of X of the first.  The records are requested when
  // the pass before begins and the rows when its last step is done, so that a pass does not open
  // with two memory round trips; unit descriptors are read two units ahead for the same reason.
  Rec cur, nx1, nx2;
  u32x4 xa[KK], xb[KK];
  uint16_t wa, wb;
  auto first_records = [&](const Unit& un, Rec& r0, Rec& r1, Rec& r2) {
    const int e = tw * kStepEdges;
    r0 = record(un, e), r1 = record(un, e + kStride), r2 = record(un, e + 2 * kStride);
  };

  // the team's share of the launch: units share_ptr[team] .. share_ptr[team + 1].  Its first
  // descriptors and records are requested before W is brought in, which takes as long.
  const int u_first = share_ptr[blockIdx.x * T + team], u_last = share_ptr[blockIdx.x * T + team + 1];
  Unit u, u1;
  u.edge_begin = 0, u.edge_count = 1, u.tile_flag = 0;
  if (u_first < u_last) u = share_units[u_first];
  u1 = u;
  if (u_first + 1 < u_last) u1 = share_units[u_first + 1];
  first_records(u, cur, nx1, nx2);

  // W[rel][16kk + 8h + i][32nt + 8c + j], i, j < 8, is one thread's block: eight 16-byte loads,
  // transposed in registers into the operands of lanes (8c + j, h).  Eight consecutive threads
  // take the eight (c, h) of a fragment, so their stores of equal j go to distinct banks.  Two
  // blocks per thread are in flight.
  {
    auto block_rows = [&](int blk, u32x4 (&in)[8]) {
      const int g = blk & 7, f = blk >> 3;
      const int kk = f % KK, nt = (f / KK) % ntiles, rel = f / (KK * ntiles);
      const uint16_t* w = W + ((int64_t)rel * FIN + 16 * kk + 8 * (g >> 2)) * feat_out + 32 * nt + 8 * (g & 3);
#pragma unroll
      for (int i = 0; i < 8; ++i) in[i] = *reinterpret_cast<const u32x4*>(w + (int64_t)i * feat_out);
    };
    auto block_store = [&](int blk, const u32x4 (&in)[8]) {
      const int g = blk & 7, f = blk >> 3;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        u32x4 o;
#pragma unroll
        for (int d = 0; d < 4; ++d)
          o[d] = __builtin_amdgcn_perm(in[2 * d + 1][j / 2], in[2 * d][j / 2], (j & 1) ? 0x07060302u : 0x05040100u);
        Wl[f * 64 + w_slot(8 * g + j)] = o;
      }
    };
    const int blocks = frags * 8;
    for (int blk = threadIdx.x; blk < blocks; blk += 2 * kThreads) {
      u32x4 in0[8], in1[8];
      const bool second = blk + kThreads < blocks;
      block_rows(blk, in0);
      if (second) block_rows(blk + kThreads, in1);
      block_store(blk, in0);
      if (second) block_store(blk + kThreads, in1);
    }
  }
  unsigned char* team_lds = lds + (size_t)frags * 1024 + team * (UW * kSBytes);
  uint16_t* S = reinterpret_cast<uint16_t*>(team_lds + tw * kSBytes);
  float* my_partial = reinterpret_cast<float*>(team_lds + tw * kSBytes);  // 8 registers x 64 lanes, over S
  // The team's wavefronts meet at a counter in LDS (a workgroup barrier would tie the teams of the
  // workgroup together; every wavefront of a team runs the same sequence of meetings, so each
  // wait ends).  The counter sits in the unused tail of row 26 of the first S tile, which neither
  // the S accesses nor the partial sums (the first 2 KB of each tile) touch.
  uint32_t* meet = reinterpret_cast<uint32_t*>(team_lds + 26 * kSStride * 2 + 64);
  uint32_t met = 0;
  auto team_arrive = [&]() {
    met += UW;
    if (lane == 0) __hip_atomic_fetch_add(meet, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  auto team_wait = [&]() {
    while (__hip_atomic_load(meet, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < met) __builtin_amdgcn_s_sleep(1);
  };
  auto team_barrier = [&]() {
    team_arrive();
    team_wait();
  };
  {
    uint32_t* s32 = reinterpret_cast<uint32_t*>(S);
#pragma unroll
    for (int k = 0; k < kSBytes / 4 / 64; ++k) s32[lane + 64 * k] = 0;  // the meeting counter too
  }
  __syncthreads();
  if (u_first >= u_last) return;  // no workgroup barrier below this line
  const int slot = w_slot(lane);
  const int jcol = 16 * (mrow >> 4) + 8 * ((mrow >> 2) & 1) + 4 * ((mrow >> 3) & 1) + (mrow & 3);
  fetch(cur, xa, wa);
  for (int ui = u_first;; ++ui) {
    const bool more_units = ui + 1 < u_last;
    Unit u2 = u1;
    if (ui + 2 < u_last) u2 = share_units[ui + 2];
    const int e_end = u.edge_count, e_first = tw * kStepEdges;  // counted from the unit's first edge
    const int tile = u.tile_flag >> 1;
    const bool atomic = u.tile_flag & 1;

    for (int nti = 0; nti < ntiles; ++nti) {
      // The next pass: the same unit at the next feature tile, or the next unit.
      const bool next_pass = nti + 1 < ntiles || more_units;
      Rec p0 = cur, p1 = cur, p2 = cur;
      if (next_pass) first_records(nti + 1 < ntiles ? u : u1, p0, p1, p2);
      // What the wavefront's 16 rows of the tile hold now, in accumulator layout (register v of lane
      // (n, h) is row 16 tw + (v%4) + 4h + 8(v/4), feature n); needed at the end only.
      float yold[8];
#pragma unroll
      for (int v = 0; v < 8; ++v) {
        const int64_t yrow = (int64_t)tile * kTileRows + 16 * tw + (v & 3) + 4 * h + 8 * (v >> 2);
        yold[v] = (!atomic && yrow < m) ? y_load(Y + yrow * feat_out + 32 * nti + mrow) : 0.f;
      }
      f32x16 acc2;
#pragma unroll
      for (int v = 0; v < 16; ++v) acc2[v] = 0.f;
      auto step = [&](const Rec& rec, const u32x4 (&x)[KK], uint16_t wbits, int e0) {
        const int left = min(kStepEdges, e_end - e0);  // uniform
        const bool live = mrow < left;
        int rel, dl;
        if constexpr (kPacked)
          rel = (int)((rec.w_rel_dl >> 5) & (kPackedMaxRels - 1)), dl = (int)(rec.w_rel_dl & 31);
        else
          rel = (int)(rec.rel_dl >> 5), dl = (int)(rec.rel_dl & 31);

        // ---- stage 1: one MFMA chain per run of equal relation (the step is sorted by relation)
        f32x16 acc1;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc1[v] = 0.f;  // a constant operand of the first MFMA, not 16 moves
        int rq = __builtin_amdgcn_readlane(rel, 0);
        int pos_e = __popcll(__ballot(rel == rq) & 0xffffffffull);
        if (pos_e >= kStepEdges) {
          // one relation in the whole step: nothing to mask
          const u32x4* w = Wl + (rq * ntiles + nti) * (KK * 64) + slot;
#pragma unroll
          for (int kk = 0; kk < KK; ++kk) acc1 = mfma32<BF16>(x[kk], w[kk * 64], acc1);
        } else {
          auto add_run = [&](int r_, f32x16 c) {
            const u32x4* w = Wl + (r_ * ntiles + nti) * (KK * 64) + slot;
            const bool sel = rel == r_;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
              u32x4 a_;
#pragma unroll
              for (int d = 0; d < 4; ++d) a_[d] = sel ? x[kk][d] : 0u;
              c = mfma32<BF16>(a_, w[kk * 64], c);
            }
            return c;
          };
          acc1 = add_run(rq, acc1);
          do {
            rq = __builtin_amdgcn_readlane(rel, pos_e);
            pos_e += __popcll(__ballot(rel == rq) & 0xffffffffull);
            acc1 = add_run(rq, acc1);
          } while (pos_e < kStepEdges);
        }

        // ---- stage 2
        if (e0 == e_first) team_wait();  // the sums of the pass before have been read out of the S tiles
        acc2 = scatter_step<BF16, std::is_same<YT, _Float16>::value>(S, dl, jcol, mrow, h, live ? wbits : (uint16_t)0, left, acc1, acc2);
      };
      // Two steps per turn of the loop, so that the two sets of X registers swap roles without
      // copies: while a step is computed, the rows of X of the step after it are on their way,
      // and so are the records three steps ahead.
#pragma unroll 1
      for (int e0 = e_first; e0 < e_end; e0 += 2 * kStride) {
        fetch(nx1, xb, wb);
        const Rec nx3 = record(u, e0 + 3 * kStride);
        step(cur, xa, wa, e0);
        if (e0 + kStride >= e_end) break;
        fetch(nx2, xa, wa);
        const Rec nx4 = record(u, e0 + 4 * kStride);
        step(nx1, xb, wb, e0 + kStride);
        cur = nx2, nx1 = nx3, nx2 = nx4;
      }

      // Everything requested so far has had the whole pass to arrive.  Naming the old values of
      // Y here settles them, so that the stores below do not wait for the loads that follow.
#pragma unroll
      for (int v = 0; v < 8; ++v) asm volatile("" : "+v"(yold[v]));
      if (next_pass) {
        cur = p0, nx1 = p1, nx2 = p2;
        fetch(cur, xa, wa);
      }

      if (e_first >= e_end) team_wait();  // (a wavefront without steps has not met the others yet)
      // ---- teams of two: each wavefront owns 16 rows of the tile (eight accumulator registers),
      // hands the other eight to its partner through LDS and writes its rows back from registers.
      float* theirs = reinterpret_cast<float*>(team_lds + (1 - tw) * kSBytes);
      if (tw == 0) {
#pragma unroll
        for (int v = 0; v < 8; ++v) my_partial[v * 64 + lane] = acc2[8 + v];
      } else {
#pragma unroll
        for (int v = 0; v < 8; ++v) my_partial[v * 64 + lane] = acc2[v];
      }
      team_barrier();
      float own[8];
      if (tw == 0) {
#pragma unroll
        for (int v = 0; v < 8; ++v) own[v] = acc2[v] + theirs[v * 64 + lane];
      } else {
#pragma unroll
        for (int v = 0; v < 8; ++v) own[v] = acc2[8 + v] + theirs[v * 64 + lane];
      }
#pragma unroll
      for (int v = 0; v < 8; ++v) theirs[v * 64 + lane] = 0.f;  // the partner's S tile is all zeros again
#pragma unroll
      for (int v = 0; v < 8; ++v) {
        const int64_t yrow = (int64_t)tile * kTileRows + 16 * tw + (v & 3) + 4 * h + 8 * (v >> 2);
        YT* y = Y + yrow * feat_out + 32 * nti + mrow;  // lanes 2k and 2k + 1: the same row, features 2k, 2k + 1
        if (atomic)  // uniform over the wavefront
          y_atomic_add(y, own[v], yrow < m, lane);
        else if (yrow < m)
          y_store(y, yold[v] + own[v]);
      }
      team_arrive();  // waited for where the next pass first writes to its S tile
    }
    if (!more_units) break;
    u = u1, u1 = u2;
  }
}

struct DevBuf {
  void* p = nullptr;
  ~DevBuf() {
    if (p) (void)hipFree(p);
  }
  hipError_t alloc(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 16); }
  template <typename T>
  T* as() const { return static_cast<T*>(p); }
};

int bit_length(uint64_t x) {
  int b = 0;
  while (x) ++b, x >>= 1;
  return b;
}

// A resident workgroup has 8 or 12 wavefronts ("quads" of four: each wavefront needs an S tile in
// LDS beside W).  16 would leave 128 registers per wavefront, which the kernel only just fits or
// spills, and measured no faster where W left the room (60 relations of 32 x 32).
constexpr int kResidentMaxQuads = 3;
// W beyond the LDS: at most this many ranges of relations, each with a launch of its own; more
// relations than that read W from memory in one launch
constexpr int kMaxRelationParts = 3;

// Launches the resident kernel with `quads` x 4 wavefronts per workgroup.
template <int KK, bool BF16, typename Rec, typename YT>
int launch_resident(int quads, dim3 grid, size_t lds, hipStream_t stream, const int32_t* share_ptr,
                    const Unit* share_units, const Rec* edges, int m, int feat_out, int num_rels, const uint16_t* W,
                    const uint16_t* X, YT* Y) {
  auto go = [&](auto* fn) -> int {
    if (int rc = allow_lds(reinterpret_cast<const void*>(fn))) return rc;
    hipLaunchKernelGGL(fn, grid, dim3(256 * quads), lds, stream, share_ptr, share_units, edges, m, feat_out, num_rels, W,
                       X, Y);
    return 0;
  };
  constexpr int kTeamsPerQuad = 4 / kTeamWaves;
  if (quads == 2) return go(rgms_tile_lds_kernel<KK, BF16, Rec, 2 * kTeamsPerQuad, YT>);
  if (quads == 3) return go(rgms_tile_lds_kernel<KK, BF16, Rec, 3 * kTeamsPerQuad, YT>);
  return fail("rgms: no kernel for %d wavefronts per workgroup", 4 * quads);
}

// What a unit costs a team beyond its steps (exchanging half of the tile with the partner, writing
// Y back, the start of the next pass), in steps of the unit.  Measured optimum, flat between 2 and 6.
constexpr int64_t kUnitOverheadSteps = 3;

// Cuts the sorted edges into `teams` shares of (nearly) equal cost, in tile order; the cost of a
// tile is its steps plus the overhead above.  A tile that lies inside one share is a unit that
// writes its rows of Y alone; the pieces of a tile that is cut by a share boundary all add with
// atomics.  A boundary that falls into the overhead part of a tile moves to the tile's start.
int build_shares(TileIndex& ix, int64_t teams, hipStream_t stream) {
  const int64_t tiles = (int64_t)ix.tile_begin.size() - 1;
  // cost coordinate: tile t occupies [at[t], at[t + 1]), its overhead first, then its steps
  std::vector<int64_t> at(size_t(tiles + 1), 0);
  auto steps_of = [&](int64_t t) { return ceil_div(ix.tile_begin[t + 1] - ix.tile_begin[t], (int64_t)kStepEdges); };
  for (int64_t t = 0; t < tiles; ++t) at[t + 1] = at[t] + (steps_of(t) ? steps_of(t) + kUnitOverheadSteps : 0);
  const int64_t total = at[tiles];
  // boundary g as (tile, step inside the tile)
  auto boundary = [&](int64_t g, int64_t& t) -> int64_t {
    const int64_t c = total * g / teams;
    while (t < tiles && at[t + 1] <= c) ++t;
    if (t >= tiles) return 0;
    return std::max<int64_t>(0, c - at[t] - kUnitOverheadSteps);
  };
  std::vector<int32_t> ptr(size_t(teams + 1), 0);
  std::vector<Unit> units;
  units.reserve(size_t(tiles + 2 * teams));
  int64_t t0 = 0, s0 = boundary(0, t0);
  for (int64_t g = 0; g < teams; ++g) {
    int64_t t1 = t0;
    const int64_t s1 = g + 1 < teams ? boundary(g + 1, t1) : 0;
    if (g + 1 == teams) t1 = tiles;
    ptr[g] = (int32_t)units.size();
    // steps [s0, end) of tile t0, whole tiles between, steps [0, s1) of tile t1
    for (int64_t k = t0; k <= t1 && k < tiles; ++k) {
      const int64_t n = steps_of(k);
      const int64_t a = k == t0 ? s0 : 0, b = k == t1 ? s1 : n;
      if (a >= b) continue;
      Unit un;
      un.edge_begin = ix.tile_begin[k] + a * kStepEdges;
      un.edge_count = (int32_t)(std::min(ix.tile_begin[k + 1], ix.tile_begin[k] + b * kStepEdges) - un.edge_begin);
      un.tile_flag = (int32_t)(k << 1) | ((a == 0 && b == n) ? 0 : 1);
      units.push_back(un);
    }
    t0 = t1, s0 = s1;
  }
  ptr[teams] = (int32_t)units.size();
  STIR_REQUIRE(units.size() < (size_t(1) << 31), "rgms: too many units");
  if (ix.d_share_ptr) STIR_HIP(hipFree(ix.d_share_ptr));
  if (ix.d_share_units) STIR_HIP(hipFree(ix.d_share_units));
  ix.d_share_ptr = ix.d_share_units = nullptr;
  ix.share_teams = 0;
  STIR_HIP(hipMalloc(&ix.d_share_ptr, sizeof(int32_t) * ptr.size()));
  STIR_HIP(hipMalloc(&ix.d_share_units, sizeof(Unit) * std::max<size_t>(units.size(), 1)));
  STIR_HIP(hipMemcpyAsync(ix.d_share_ptr, ptr.data(), sizeof(int32_t) * ptr.size(), hipMemcpyHostToDevice, stream));
  STIR_HIP(hipMemcpyAsync(ix.d_share_units, units.data(), sizeof(Unit) * units.size(), hipMemcpyHostToDevice, stream));
  STIR_HIP(hipStreamSynchronize(stream));  // the host vectors go away
  ix.share_teams = teams;
  return 0;
}

// The index of the relations [rel_lo, rel_lo + rel_count) of all_rels; ix.num_rels becomes rel_count.
int tile_index_build(TileIndex& ix, const std::vector<TileBucket>& buckets, int32_t m, int32_t n, int32_t all_rels,
                     int32_t rel_lo, int32_t rel_count, bool static_weights, hipStream_t stream) {
  const int32_t num_rels = rel_count;
  const bool packed = static_weights && num_rels <= kPackedMaxRels;
  if (ix.d_edges) STIR_HIP(hipFree(ix.d_edges));
  if (ix.d_units) STIR_HIP(hipFree(ix.d_units));
  if (ix.d_share_ptr) STIR_HIP(hipFree(ix.d_share_ptr));
  if (ix.d_share_units) STIR_HIP(hipFree(ix.d_share_units));
  ix.d_edges = ix.d_units = ix.d_share_ptr = ix.d_share_units = nullptr;
  ix.share_teams = 0;
  ix.tile_begin.clear();
  ix.m = -1;
  ix.edges = ix.units = 0;
  std::vector<DevBucket> host;
  int64_t slots = 0;
  for (const TileBucket& b : buckets) {
    if (b.groups == 0) continue;
    host.push_back(DevBucket{b.A, b.rows, b.cols, b.mids, slots, b.rb, b.cb});
    slots += b.groups * b.rb * b.cb;
  }
  STIR_REQUIRE(slots < (int64_t(1) << 31), "rgms: %lld slots exceed the edge index", (long long)slots);
  ix.rel_lo = rel_lo;
  if (slots == 0 || m == 0) {
    ix.m = m, ix.n = n, ix.num_rels = num_rels;
    return 0;
  }
  const int nb = (int)host.size();
  const int64_t tiles = ceil_div(m, kTileRows);
  // keys run up to (tiles * num_rels) << 5 inclusive: that value marks the dropped slots
  const int end_bit = bit_length(((uint64_t)tiles * num_rels) << 5);
  const int cus = std::max(1, compute_units());
  // Units (one workgroup each) of at most `cap` steps.  A tile is cut only when it is long against
  // the others -- more than about three average tiles -- or when the launch would otherwise
  // leave most of the chip idle (few tiles): the longest unit is the critical path of the launch.
  // CSFToELL3D pads every relation's rows by repeating its last row id, so the tiles that hold
  // those rows carry thousands of zero-weight slots and are always cut.
  const int64_t steps_bound = slots / kStepEdges + tiles;
  const int64_t by_chip = kUnitWaves * ceil_div(steps_bound, (int64_t)cus * 8);
  const int64_t by_tile = 2 * ceil_div(steps_bound, tiles);
  const int cap = (int)std::max<int64_t>(16, std::min(by_chip, by_tile));

  size_t sort_bytes = 0, scan_bytes = 0;
  STIR_HIP(hipcub::DeviceRadixSort::SortPairs(nullptr, sort_bytes, (const uint64_t*)nullptr, (uint64_t*)nullptr,
                                              (const int32_t*)nullptr, (int32_t*)nullptr, (int)slots, 0, end_bit,
                                              stream));
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(nullptr, scan_bytes, (const int32_t*)nullptr, (int32_t*)nullptr,
                                            (int)(tiles + 1), stream));
  DevBuf tab, keys_in, keys, vals_in, vals, tmp, bad, begin, count, ubegin;
  STIR_HIP(tab.alloc(sizeof(DevBucket) * host.size()));
  STIR_HIP(keys_in.alloc(sizeof(uint64_t) * size_t(slots)));
  STIR_HIP(keys.alloc(sizeof(uint64_t) * size_t(slots)));
  STIR_HIP(vals_in.alloc(sizeof(int32_t) * size_t(slots)));
  STIR_HIP(vals.alloc(sizeof(int32_t) * size_t(slots)));
  STIR_HIP(tmp.alloc(std::max(sort_bytes, scan_bytes)));
  STIR_HIP(bad.alloc(sizeof(int32_t)));
  STIR_HIP(begin.alloc(sizeof(int64_t) * size_t(tiles + 1)));
  STIR_HIP(count.alloc(sizeof(int32_t) * size_t(tiles + 1)));
  STIR_HIP(ubegin.alloc(sizeof(int32_t) * size_t(tiles + 1)));
  STIR_HIP(hipMemcpyAsync(tab.p, host.data(), sizeof(DevBucket) * host.size(), hipMemcpyHostToDevice, stream));
  STIR_HIP(hipMemsetAsync(bad.p, 0, sizeof(int32_t), stream));
  const dim3 block(256);
  const dim3 slot_grid((unsigned)ceil_div(slots, 256)), tile_grid((unsigned)ceil_div(tiles + 1, 256));
  hipLaunchKernelGGL(edge_keys_kernel, slot_grid, block, 0, stream, tab.as<DevBucket>(), nb, slots, m, all_rels,
                     rel_lo, rel_count, packed ? 1 : 0, keys_in.as<uint64_t>(), vals_in.as<int32_t>(), bad.as<int32_t>());
  STIR_LAUNCH_CHECK();
  STIR_HIP(hipcub::DeviceRadixSort::SortPairs(tmp.p, sort_bytes, keys_in.as<const uint64_t>(), keys.as<uint64_t>(),
                                              vals_in.as<const int32_t>(), vals.as<int32_t>(), (int)slots, 0,
                                              end_bit, stream));
  hipLaunchKernelGGL(tile_bounds_kernel, tile_grid, block, 0, stream, keys.as<const uint64_t>(), slots, tiles,
                     num_rels, begin.as<int64_t>());
  STIR_LAUNCH_CHECK();
  hipLaunchKernelGGL(unit_count_kernel, tile_grid, block, 0, stream, begin.as<const int64_t>(), tiles, cap,
                     count.as<int32_t>());
  STIR_LAUNCH_CHECK();
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(tmp.p, scan_bytes, count.as<const int32_t>(), ubegin.as<int32_t>(),
                                            (int)(tiles + 1), stream));
  int32_t h_bad = 0, h_units = 0;
  ix.tile_begin.resize(size_t(tiles + 1));
  STIR_HIP(hipMemcpyAsync(ix.tile_begin.data(), begin.p, sizeof(int64_t) * size_t(tiles + 1), hipMemcpyDeviceToHost,
                          stream));
  STIR_HIP(hipMemcpyAsync(&h_bad, bad.p, sizeof(int32_t), hipMemcpyDeviceToHost, stream));
  STIR_HIP(hipMemcpyAsync(&h_units, ubegin.as<int32_t>() + tiles, sizeof(int32_t), hipMemcpyDeviceToHost, stream));
  STIR_HIP(hipStreamSynchronize(stream));
  if (h_bad == 1) return fail("rgms: a row id lies outside [0, %d) or a relation id outside [0, %d)", m, all_rels);
  // records of the slots that lie in a tile (the others belong to other relations or are padding)
  const int64_t kept = ix.tile_begin[size_t(tiles)];
  DevBuf edges;
  STIR_HIP(edges.alloc((packed ? sizeof(PackedEdge) : sizeof(Edge)) * size_t(std::max<int64_t>(kept, 1))));
  if (packed)
    hipLaunchKernelGGL(edge_records_kernel<PackedEdge>, slot_grid, block, 0, stream, tab.as<DevBucket>(), nb, slots,
                       kept, n, num_rels, keys.as<const uint64_t>(), vals.as<const int32_t>(), edges.as<PackedEdge>(),
                       bad.as<int32_t>());
  else
    hipLaunchKernelGGL(edge_records_kernel<Edge>, slot_grid, block, 0, stream, tab.as<DevBucket>(), nb, slots, kept, n,
                       num_rels, keys.as<const uint64_t>(), vals.as<const int32_t>(), edges.as<Edge>(),
                       bad.as<int32_t>());
  STIR_LAUNCH_CHECK();
  STIR_HIP(hipMemcpyAsync(&h_bad, bad.p, sizeof(int32_t), hipMemcpyDeviceToHost, stream));
  STIR_HIP(hipStreamSynchronize(stream));
  if (h_bad == 2) return fail("rgms: a column id lies outside [0, %d)", n);
  DevBuf units;
  STIR_HIP(units.alloc(sizeof(Unit) * size_t(h_units)));
  hipLaunchKernelGGL(unit_fill_kernel, tile_grid, block, 0, stream, begin.as<const int64_t>(),
                     ubegin.as<const int32_t>(), tiles, cap, units.as<Unit>());
  STIR_LAUNCH_CHECK();
  // Longest units first: workgroups are dispatched in unit order, and a long unit that starts in the
  // last round of workgroups would be the tail of the launch.
  if (h_units > 1) {
    DevBuf ukeys_in, ukeys, uvals_in, uvals, utmp, sorted;
    size_t usort_bytes = 0;
    STIR_HIP(hipcub::DeviceRadixSort::SortPairsDescending(nullptr, usort_bytes, (const int32_t*)nullptr,
                                                          (int32_t*)nullptr, (const int32_t*)nullptr,
                                                          (int32_t*)nullptr, h_units, 0, 32, stream));
    STIR_HIP(ukeys_in.alloc(sizeof(int32_t) * size_t(h_units)));
    STIR_HIP(ukeys.alloc(sizeof(int32_t) * size_t(h_units)));
    STIR_HIP(uvals_in.alloc(sizeof(int32_t) * size_t(h_units)));
    STIR_HIP(uvals.alloc(sizeof(int32_t) * size_t(h_units)));
    STIR_HIP(utmp.alloc(usort_bytes));
    STIR_HIP(sorted.alloc(sizeof(Unit) * size_t(h_units)));
    const dim3 unit_grid((unsigned)ceil_div(h_units, 256));
    hipLaunchKernelGGL(unit_sort_keys_kernel, unit_grid, block, 0, stream, units.as<const Unit>(), (int64_t)h_units,
                       ukeys_in.as<int32_t>(), uvals_in.as<int32_t>());
    STIR_LAUNCH_CHECK();
    STIR_HIP(hipcub::DeviceRadixSort::SortPairsDescending(utmp.p, usort_bytes, ukeys_in.as<const int32_t>(),
                                                          ukeys.as<int32_t>(), uvals_in.as<const int32_t>(),
                                                          uvals.as<int32_t>(), h_units, 0, 32, stream));
    hipLaunchKernelGGL(unit_permute_kernel, unit_grid, block, 0, stream, units.as<const Unit>(),
                       uvals.as<const int32_t>(), (int64_t)h_units, sorted.as<Unit>());
    STIR_LAUNCH_CHECK();
    STIR_HIP(hipStreamSynchronize(stream));
    std::swap(units.p, sorted.p);
  }
  STIR_HIP(hipStreamSynchronize(stream));
  ix.d_edges = edges.p, edges.p = nullptr;
  ix.d_units = units.p, units.p = nullptr;
  ix.edges = kept;
  ix.units = h_units;
  ix.m = m, ix.n = n, ix.num_rels = num_rels;
  ix.packed_records = packed;
  return 0;
}

// Y += RGMS(W, X) over the edges of one index; W starts at the index's first relation.
// out16: Y is fp16 (fp16 inputs only), else fp32.
int tile_rgms_launch(bool bf16, bool out16, TileIndex& ix, int32_t feat_in, int32_t feat_out, const void* d_W,
                     const void* d_X, void* d_Y, hipStream_t stream) {
  STIR_REQUIRE(ix.m >= 0, "rgms: the edge index has not been built");
  if (ix.units == 0) return 0;
  STIR_REQUIRE(feat_in % 16 == 0 && feat_in / 16 <= kMaxKK && feat_out % 32 == 0, "rgms: unsupported feature sizes");
  const int kk_count = feat_in / 16;
  const int64_t frags = (int64_t)ix.num_rels * (feat_out / 32) * kk_count;
  STIR_REQUIRE(frags < (int64_t(1) << 25), "rgms: W of %lld operand fragments exceeds the 32-bit fragment offsets", (long long)frags);
  const Unit* units = static_cast<const Unit*>(ix.d_units);
  const Edge* edges = static_cast<const Edge*>(ix.d_edges);
  const PackedEdge* pedges = static_cast<const PackedEdge*>(ix.d_edges);
  const uint16_t* X = static_cast<const uint16_t*>(d_X);
  const uint16_t* W = static_cast<const uint16_t*>(d_W);
  float* Y32 = static_cast<float*>(d_Y);
  _Float16* Y16 = static_cast<_Float16*>(d_Y);
  STIR_REQUIRE(!(bf16 && out16), "rgms: fp16 output takes fp16 inputs");

  // W resident in LDS when it fits beside the S tiles of at least two teams
  const size_t w_bytes = size_t(frags) * 64 * sizeof(u32x4);
  int quads = 0;
  if (kk_count <= kLdsMaxKK && reinterpret_cast<uintptr_t>(d_W) % 16 == 0 &&
      (int64_t)ix.n * feat_in * 2 < (int64_t(1) << 32)) {
    const size_t lds_limit = lds_bytes_per_workgroup();
    for (int q = kResidentMaxQuads; q >= 2 && quads == 0; --q)
      if (w_bytes + size_t(q) * 4 * kSBytes <= lds_limit) quads = q;
  }
  if (quads) {
    const int teams = quads * 4 / kTeamWaves;  // per workgroup
    const size_t lds = w_bytes + size_t(quads) * 4 * kSBytes;
    // one workgroup per compute unit, fewer when a team would get less than a handful of steps
    const int64_t steps_bound = ix.edges / kStepEdges + (int64_t)ix.tile_begin.size();
    const int64_t wgs = std::min<int64_t>(std::max(1, compute_units()), ceil_div(steps_bound, (int64_t)teams * 8));
    if (ix.share_teams != wgs * teams)
      if (int rc = build_shares(ix, wgs * teams, stream)) return rc;
    const dim3 grid((unsigned)wgs);
    const int32_t* share_ptr = static_cast<const int32_t*>(ix.d_share_ptr);
    const Unit* share_units = static_cast<const Unit*>(ix.d_share_units);
#define STIR_LDS_R(KKV, BF, REC, PTR, YP)                                                               \
  if (int rc = launch_resident<KKV, BF, REC>(quads, grid, lds, stream, share_ptr, share_units, PTR, ix.m, feat_out, \
                                             ix.num_rels, W, X, YP))                                       \
    return rc
#define STIR_LDS_Y(KKV, REC, PTR)                           \
  if (out16) {                                              \
    STIR_LDS_R(KKV, false, REC, PTR, Y16);                  \
  } else if (bf16) {                                        \
    STIR_LDS_R(KKV, true, REC, PTR, Y32);                   \
  } else {                                                  \
    STIR_LDS_R(KKV, false, REC, PTR, Y32);                  \
  }
#define STIR_LDS(KKV)                        \
  case KKV:                                  \
    if (ix.packed_records) {                 \
      STIR_LDS_Y(KKV, PackedEdge, pedges)    \
    } else {                                 \
      STIR_LDS_Y(KKV, Edge, edges)           \
    }                                        \
    break
    switch (kk_count) {
      STIR_LDS(1);
      STIR_LDS(2);
      STIR_LDS(3);
      STIR_LDS(4);
    }
#undef STIR_LDS
#undef STIR_LDS_Y
#undef STIR_LDS_R
    STIR_LAUNCH_CHECK();
    return 0;
  }

  const size_t need = w_bytes;
  if (need > ix.wpack_bytes) {
    if (ix.d_wpack) STIR_HIP(hipFree(ix.d_wpack));
    ix.d_wpack = nullptr;
    ix.wpack_bytes = 0;
    STIR_HIP(hipMalloc(&ix.d_wpack, need));
    ix.wpack_bytes = need;
  }
  u32x4* Wp = static_cast<u32x4*>(ix.d_wpack);
  hipLaunchKernelGGL(pack_w_kernel, dim3((unsigned)ceil_div(frags, 4)), dim3(256), 0, stream,
                     W, Wp, frags, kk_count, feat_out);
  STIR_LAUNCH_CHECK();
  const dim3 grid((unsigned)ix.units), block(64 * kUnitWaves);
#define STIR_TILES_R(KKV, BF, REC, PTR, YT, YP) \
  hipLaunchKernelGGL((rgms_tile_kernel<KKV, BF, REC, YT>), grid, block, 0, stream, units, PTR, ix.m, feat_out, Wp, X, YP)
#define STIR_TILES_Y(KKV, REC, PTR)                       \
  if (out16)                                              \
    STIR_TILES_R(KKV, false, REC, PTR, _Float16, Y16);    \
  else if (bf16)                                          \
    STIR_TILES_R(KKV, true, REC, PTR, float, Y32);        \
  else                                                    \
    STIR_TILES_R(KKV, false, REC, PTR, float, Y32)
#define STIR_TILES(KKV)                       \
  case KKV:                                   \
    if (ix.packed_records) {                  \
      STIR_TILES_Y(KKV, PackedEdge, pedges);  \
    } else {                                  \
      STIR_TILES_Y(KKV, Edge, edges);         \
    }                                         \
    break
  switch (kk_count) {
    STIR_TILES(1);
    STIR_TILES(2);
    STIR_TILES(3);
    STIR_TILES(4);
    STIR_TILES(5);
    STIR_TILES(6);
    STIR_TILES(7);
    STIR_TILES(8);
  }
#undef STIR_TILES
#undef STIR_TILES_Y
#undef STIR_TILES_R
  STIR_LAUNCH_CHECK();
  return 0;
}

}  // namespace

void tile_index_free(TileIndex& ix) {
  if (ix.d_edges) (void)hipFree(ix.d_edges);
  if (ix.d_units) (void)hipFree(ix.d_units);
  if (ix.d_wpack) (void)hipFree(ix.d_wpack);
  if (ix.d_share_ptr) (void)hipFree(ix.d_share_ptr);
  if (ix.d_share_units) (void)hipFree(ix.d_share_units);
  ix = TileIndex();
}

void tile_set_free(TileIndexSet& set) {
  for (TileIndex& ix : set.parts) tile_index_free(ix);
  set = TileIndexSet();
}

int tile_set_prepare(TileIndexSet& set, const std::vector<TileBucket>& buckets, int32_t m, int32_t n,
                     int32_t num_rels, int32_t feat_in, int32_t feat_out, bool static_weights, hipStream_t stream) {
  STIR_REQUIRE(num_rels > 0 && num_rels < (1 << 26), "rgms: num_rels=%d out of range", num_rels);
  // Relations per part: all of them, unless W is too large for the LDS of a compute unit and a few
  // ranges of relations are not -- then every range gets an index and a launch of its own.
  int32_t per_part = num_rels;
  if (feat_in % 16 == 0 && feat_in / 16 <= kLdsMaxKK && feat_out % 32 == 0 &&
      (int64_t)n * feat_in * 2 < (int64_t(1) << 32)) {
    const size_t rel_bytes = size_t(feat_out / 32) * (feat_in / 16) * 64 * sizeof(u32x4);
    const size_t lds_limit = lds_bytes_per_workgroup();
    auto fit = [&](int quads) { return (int64_t)((lds_limit - size_t(quads) * 4 * kSBytes) / rel_bytes); };
    if (num_rels > fit(2) && fit(kResidentMaxQuads) > 0) {
      const int64_t parts = ceil_div((int64_t)num_rels, fit(kResidentMaxQuads));
      if (parts <= kMaxRelationParts) per_part = (int32_t)ceil_div((int64_t)num_rels, parts);
    }
  }
  if (set.m == m && set.n == n && set.num_rels == num_rels && set.rels_per_part == per_part) return 0;
  tile_set_free(set);
  const int parts = (int)ceil_div(num_rels, per_part);
  set.parts.resize(size_t(parts));
  for (int p = 0; p < parts; ++p) {
    const int32_t lo = p * per_part;
    if (int rc = tile_index_build(set.parts[size_t(p)], buckets, m, n, num_rels, lo, std::min(per_part, num_rels - lo),
                                  static_weights, stream)) {
      tile_set_free(set);
      return rc;
    }
  }
  set.m = m, set.n = n, set.num_rels = num_rels, set.rels_per_part = per_part;
  return 0;
}

int tile_set_launch(bool bf16, bool out16, TileIndexSet& set, int32_t feat_in, int32_t feat_out, const void* d_W,
                    const void* d_X, void* d_Y, hipStream_t stream) {
  STIR_REQUIRE(set.m >= 0, "rgms: the edge index has not been built");
  for (TileIndex& ix : set.parts) {
    const uint16_t* W = static_cast<const uint16_t*>(d_W) + (int64_t)ix.rel_lo * feat_in * feat_out;
    if (int rc = tile_rgms_launch(bf16, out16, ix, feat_in, feat_out, W, d_X, d_Y, stream)) return rc;
  }
  return 0;
}

}  // namespace stir

