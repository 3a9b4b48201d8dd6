// RGMS in fp32 for gfx950, two front ends over one tile routine:
//   * ELL3D buckets (group -> rb ELL rows -> cb slots, one relation per group), the composable
//     form of examples/rgms/rgcn/bench_rgcn_composable.py:186-206;
//   * CSF traversal (relation -> stored row -> column), the form of
//     examples/rgms/rgcn/bench_rgcn_non_composable.py:82-105.
// Both compute  Y[row, fo] += sum_edges A * sum_fi W[rel, fo, fi] * X[col, fi]  into a zeroed Y.
//
// W[rel] is the same for every edge of a (relation, row) pair, so a wavefront first sums the
// weighted X rows of each of up to 32 rows of its tile (rows are spread over lane groups of
// float4 lanes; the per-row sums go to the wavefront's piece of LDS), and only then multiplies
// the 32 x feat_in block of sums by W[rel]^T on the matrix cores (v_mfma_f32_32x32x2_f32).  The
// product leaves with one fp32 atomic per (row, feature); an atomic instruction covers 32
// consecutive floats of two rows.  A tile whose rows belong to several relations repeats the
// product once per relation and writes only that relation's rows.
#include <vector>

#include "common.h"
#include "rgms_f32_tiles.h"
#include "../../include/sparsetir_amd.h"

namespace {

using stir::kWave;

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kTileRows = 32;

__device__ __forceinline__ void atomic_addf(float* p, float v) {
  __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Per-wavefront LDS: the row sums S[32][FP + 1] (the odd stride spreads rows over banks) and,
// for the CSF front end, the tile's 33 edge offsets.
template <int FP>
struct TileLds {
  float S[kTileRows * (FP + 1)];
  int32_t ptr[kTileRows + 1];
};

// Phase 1: S[r, :] = sum over the edges p in [range(r).x, range(r).y) of A[p] * X[cols[p], :] for
// the 32 rows of the tile (zero for r >= nrows).  A row belongs to one lane group (G lanes, one
// float4 each): group g takes rows g, g + NG, ...; the columns and weights of a row arrive a
// chunk of at least 16 edges at a time, fetched by the group's lanes side by side and handed round
// with cross-lane reads, the first chunks of up to eight of its rows requested together before it
// adds anything.  Rows with more than kLongRow edges are left to
// a second pass in which all lane groups share the row's edges and combine their partial sums
// with cross-lane adds.  Nothing here is atomic (LDS float atomics run at a fraction of the rate
// of plain LDS stores on this chip), and every S entry is written exactly once.
constexpr int kLongRow = 32;

template <int FP, class Range>
__device__ __forceinline__ void accumulate_rows(float* S, const float* __restrict__ X, const float* __restrict__ A,
                                                const int32_t* __restrict__ cols, int fin, int lane, int nrows,
                                                Range range) {
  constexpr int G = FP / 4, NG = kWave / G;
  constexpr int RPG = kTileRows / NG;        // rows per lane group
  constexpr int PER = G >= 16 ? 1 : 16 / G;  // edges whose column and weight one lane fetches per chunk
  constexpr int CHUNK = G * PER;             // edges of a row per chunk (at least 16)
  constexpr int CH = G < 4 ? G : 4;          // gathers in flight per lane (8 cost a wavefront of occupancy: 165 against 158 us)
  const int g = lane / G, gl = lane % G;
  // Every gather is unconditional (no register cleared first, no lane branches): an edge of weight
  // zero -- the padding of an ELL row, column 0 -- fetches row 0 of X and adds 0 * X[0, :], as the
  // reference's kernel does; lanes whose features lie beyond feat_in fetch the first features
  // instead and their sums are replaced by zeros before they are stored.
  const bool chunk_live = 4 * gl < fin;
  const float* Xl = X + (chunk_live ? 4 * gl : 0);
  auto ld_x = [&](int c) { return *reinterpret_cast<const float4*>(Xl + (int64_t)c * fin); };
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
  auto fma4 = [](float4& acc, float w, const float4& x) {
    acc.x += w * x.x, acc.y += w * x.y, acc.z += w * x.z, acc.w += w * x.w;
  };
  // The edges of a row are fetched by the row's lane group, one chunk per round trip (lane gl takes
  // edges gl, gl + G, ... of the chunk: coalesced), and handed round inside the group; the first
  // chunk of every row of the group is requested before anything else, so that a tile of rows
  // of up to CHUNK edges costs one round trip for its columns and weights.
  constexpr int RB = RPG < 8 ? RPG : 8;  // rows of a lane group whose first chunks are in flight together
#pragma unroll 1
  for (int k0 = 0; k0 < RPG; k0 += RB) {
    int rb[RB], re[RB];
    int col[RB][PER];
    float w[RB][PER];
    bool keep[RB];
#pragma unroll
    for (int k = 0; k < RB; ++k) {
      const int r = g + NG * (k0 + k);
      int2 be = make_int2(0, 0);
      if (r < nrows) be = range(r);
      keep[k] = be.y - be.x <= kLongRow;
      rb[k] = be.x;
      re[k] = keep[k] ? be.y : be.x;
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int p = rb[k] + i * G + gl;
        col[k][i] = p < re[k] ? cols[p] : 0;
        w[k][i] = p < re[k] ? A[p] : 0.f;
      }
    }
#pragma unroll
    for (int k = 0; k < RB; ++k) {
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
      for (int base = rb[k]; base < re[k]; base += CHUNK) {
        if (base != rb[k]) {  // a row of more than CHUNK edges: its next chunk
#pragma unroll
          for (int i = 0; i < PER; ++i) {
            const int p = base + i * G + gl;
            col[k][i] = p < re[k] ? cols[p] : 0;
            w[k][i] = p < re[k] ? A[p] : 0.f;
          }
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) {
#pragma unroll
          for (int c = 0; c < G; c += CH) {
            if (base + i * G + c >= re[k]) continue;  // the same for every lane of the group
            float4 x[CH];
            float wv[CH];
#pragma unroll
            for (int u = 0; u < CH; ++u) {
              const int src = g * G + c + u;  // a lane of this group
              const int cc = __shfl(col[k][i], src, kWave);
              wv[u] = __shfl(w[k][i], src, kWave);  // zero beyond the row's end and on padding
              x[u] = ld_x(cc);
            }
#pragma unroll
            for (int u = 0; u < CH; ++u) fma4(acc, wv[u], x[u]);
          }
        }
      }
      if (keep[k]) {
        if (!chunk_live) acc = zero4;
        float* s = S + (g + NG * (k0 + k)) * (FP + 1) + 4 * gl;
        s[0] = acc.x, s[1] = acc.y, s[2] = acc.z, s[3] = acc.w;
      }
    }
  }  // batches of rows
  // long rows: lane l < nrows knows whether row l is one
  constexpr int U = 4;  // edges per lane group and step
  int2 mine = make_int2(0, 0);
  if (lane < nrows) mine = range(lane);
  uint64_t todo = __ballot(mine.y - mine.x > kLongRow);
  while (todo) {
    const int r = __ffsll((long long)todo) - 1;
    todo &= todo - 1;
    const int b = __shfl(mine.x, r, kWave), e = __shfl(mine.y, r, kWave);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 1
    for (int p = b + g; p < e; p += NG * U) {
      int c2[U];
      float w2[U];
      float4 x2[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const bool live = p + u * NG < e;
        c2[u] = live ? cols[p + u * NG] : 0;
        w2[u] = live ? A[p + u * NG] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) x2[u] = ld_x(c2[u]);
#pragma unroll
      for (int u = 0; u < U; ++u) fma4(acc, w2[u], x2[u]);
    }
#pragma unroll
    for (int off = G; off < kWave; off <<= 1) {
      acc.x += __shfl_xor(acc.x, off, kWave);
      acc.y += __shfl_xor(acc.y, off, kWave);
      acc.z += __shfl_xor(acc.z, off, kWave);
      acc.w += __shfl_xor(acc.w, off, kWave);
    }
    if (g == 0) {
      if (!chunk_live) acc = zero4;
      float* s = S + r * (FP + 1) + 4 * gl;
      s[0] = acc.x, s[1] = acc.y, s[2] = acc.z, s[3] = acc.w;
    }
  }
}

// B operand of the product for relation `rel`, output features nt..nt+31: lane (n, h) holds
// W[rel][nt + n][h*KH + kk], kk < KH (zero beyond feat_in / feat_out).
template <int FP>
__device__ __forceinline__ void load_w(float (&wv)[FP / 2], const float* __restrict__ W, int rel, int nt, int fin,
                                       int fout, int lane) {
  constexpr int KH = FP / 2;
  const int n = lane & 31, h = lane >> 5;
  const bool col_live = nt + n < fout;
  const float* wp = W + ((int64_t)rel * fout + nt + n) * fin + h * KH;
#pragma unroll
  for (int c = 0; c < KH / 4; ++c) {
    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
    if (col_live && h * KH + 4 * c < fin) t = *reinterpret_cast<const float4*>(wp + 4 * c);
    wv[4 * c] = t.x, wv[4 * c + 1] = t.y, wv[4 * c + 2] = t.z, wv[4 * c + 3] = t.w;
  }
}

// Phase 2: Y[rowid[r], :] += S[r, :] @ W[rel[r]]^T for the tile's rows r < nrows.  Lane l < 32
// holds row l's output row id and relation.  Relations are non-decreasing over the rows.  `wv`
// arrives loaded for (relation of row 0, nt = 0), requested before phase 1 so that its latency
// overlaps the gathers.
template <int FP>
__device__ __forceinline__ void transform_scatter(const float* S, const float* __restrict__ W,
                                                  float* __restrict__ Y, int fin, int fout, int lane,
                                                  int nrows, int my_rowid, int my_rel, float (&wv)[FP / 2]) {
  constexpr int KH = FP / 2;  // MFMA steps; half h of the wavefront covers inputs h*KH .. h*KH+KH-1
  const int n = lane & 31, h = lane >> 5;
  const int first = __shfl(my_rel, 0, kWave);
  int cur = first;
  while (true) {
    for (int nt = 0; nt < fout; nt += 32) {
      if (cur != first || nt != 0) load_w<FP>(wv, W, cur, nt, fin, fout, lane);
      f32x16 acc;
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[v] = 0.f;
      const float* sp = S + n * (FP + 1) + h * KH;
#pragma unroll
      for (int kk = 0; kk < KH; ++kk) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(sp[kk], wv[kk], acc, 0, 0, 0);
      // acc[v]: tile row (v%4) + 4h + 8(v/4), output feature nt + n
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = (v & 3) + 4 * h + 8 * (v >> 2);
        const int rowid = __shfl(my_rowid, r, kWave);
        const int rel = __shfl(my_rel, r, kWave);
        if (nt + n < fout && r < nrows && rel == cur) atomic_addf(Y + (int64_t)rowid * fout + nt + n, acc[v]);
      }
    }
    // next relation present in the tile
    const uint64_t later = __ballot(lane < nrows && my_rel > cur);
    if (later == 0) break;
    cur = __shfl(my_rel, __ffsll((long long)later) - 1, kWave);
  }
}

// Wavefronts per SIMD the compiler is to fit: with 32 input features it ends at 97 registers
// plus 16 accumulator registers (four wavefronts) by itself and fits five without a spill when
// asked (156 against 158 us on a 1.3 M-row RGCN input; six need spills: 180 us).
template <int FP>
constexpr int kMinWaves = FP == 32 ? 5 : 1;

// ----------------------------------------------------------------------------- ELL3D front end
struct alignas(16) RgmsF32Bucket {
  const float* A;       // slot weights, groups*rb*cb
  const int32_t* rows;  // groups*rb
  const int32_t* cols;  // groups*rb*cb
  const int32_t* mids;  // groups
  int64_t ell_rows;     // groups*rb
  int64_t unit_begin;   // first tile of this bucket in the fused launch
  int32_t rb, cb;
  int32_t tile_rows;        // ELL rows per tile: a whole number of groups when rb < 32, else 32
  int32_t chunks_per_group; // tiles per group when rb >= 32, else 0
};

template <int FP, int WAVES>
__global__ __launch_bounds__(WAVES * 64, kMinWaves<FP>) void rgms_ell3d_f32_kernel(const RgmsF32Bucket* __restrict__ table,
                                                                    int nb, int64_t total_units, int fin, int fout,
                                                                    const float* __restrict__ W,
                                                                    const float* __restrict__ X,
                                                                    float* __restrict__ Y) {
  __shared__ TileLds<FP> lds[WAVES];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t gid = (int64_t)blockIdx.x * WAVES + wave;
  if (gid >= total_units) return;
  int lo = 0, hi = nb - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[mid].unit_begin <= gid) lo = mid; else hi = mid - 1;
  }
  const RgmsF32Bucket bk = table[lo];
  const int64_t unit = gid - bk.unit_begin;
  // ELL rows [r0, r0 + nrows) of the bucket
  int64_t r0;
  int nrows;
  if (bk.chunks_per_group > 0) {
    const int64_t g = unit / bk.chunks_per_group;
    const int chunk = (int)(unit % bk.chunks_per_group);
    r0 = g * bk.rb + (int64_t)chunk * kTileRows;
    nrows = min(kTileRows, bk.rb - chunk * kTileRows);
  } else {
    r0 = unit * bk.tile_rows;
    nrows = (int)min((int64_t)bk.tile_rows, bk.ell_rows - r0);
  }
  float* S = lds[wave].S;
  int my_rowid = 0, my_rel = 0;
  if (lane < nrows) {
    my_rowid = bk.rows[r0 + lane];
    my_rel = bk.mids[(r0 + lane) / bk.rb];
  }
  float wv[FP / 2];
  load_w<FP>(wv, W, __shfl(my_rel, 0, kWave), 0, fin, fout, lane);
  const int64_t s0 = r0 * bk.cb;
  const int cb = bk.cb;
  accumulate_rows<FP>(S, X, bk.A + s0, bk.cols + s0, fin, lane, nrows,
                      [cb](int r) { return make_int2(r * cb, (r + 1) * cb); });
  __builtin_amdgcn_wave_barrier();
  transform_scatter<FP>(S, W, Y, fin, fout, lane, nrows, my_rowid, my_rel, wv);
}

// ----------------------------------------------------------------------------- CSF front end
template <int FP, int WAVES>
__global__ __launch_bounds__(WAVES * 64, kMinWaves<FP>) void rgms_csf_f32_kernel(int num_rels, int64_t nnz_i, int fin, int fout,
                                                                  const float* __restrict__ A,
                                                                  const float* __restrict__ W,
                                                                  const float* __restrict__ X, float* __restrict__ Y,
                                                                  const int32_t* __restrict__ indptr_i,
                                                                  const int32_t* __restrict__ indices_i,
                                                                  const int32_t* __restrict__ indptr_j,
                                                                  const int32_t* __restrict__ indices_j) {
  __shared__ TileLds<FP> lds[WAVES];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t p0 = ((int64_t)blockIdx.x * WAVES + wave) * kTileRows;
  if (p0 >= nnz_i) return;
  const int nrows = (int)min((int64_t)kTileRows, nnz_i - p0);
  float* S = lds[wave].S;
  int32_t* ptr = lds[wave].ptr;
  const int my_ptr = lane <= nrows ? indptr_j[p0 + lane] : 0;
  int my_rowid = 0, my_rel = 0;
  if (lane < nrows) {
    my_rowid = indices_i[p0 + lane];
    // relation of stored row p: upper_bound(indptr_i, p) - 1
    int a = 0, b = num_rels + 1;
    while (a < b) {
      const int c = a + ((b - a) >> 1);
      if ((int64_t)indptr_i[c] > p0 + lane) b = c; else a = c + 1;
    }
    my_rel = min(max(a - 1, 0), num_rels - 1);  // stays inside W even if nnz_i disagrees with indptr_i
  }
  float wv[FP / 2];
  load_w<FP>(wv, W, __shfl(my_rel, 0, kWave), 0, fin, fout, lane);
  if (lane <= nrows) ptr[lane] = my_ptr;
  __builtin_amdgcn_wave_barrier();
  accumulate_rows<FP>(S, X, A, indices_j, fin, lane, nrows, [ptr](int r) { return make_int2(ptr[r], ptr[r + 1]); });
  __builtin_amdgcn_wave_barrier();
  transform_scatter<FP>(S, W, Y, fin, fout, lane, nrows, my_rowid, my_rel, wv);
}

constexpr int kMaxFin = 128;

int padded_fin(int fin) {
  int fp = 8;
  while (fp < fin) fp *= 2;
  return fp;
}

int check_feats(const char* who, int fin, int fout) {
  STIR_REQUIRE(fin > 0 && fin % 4 == 0 && fin <= kMaxFin, "%s: feat_in=%d must be a multiple of 4 and at most %d",
               who, fin, kMaxFin);
  STIR_REQUIRE(fout > 0, "%s: feat_out=%d must be positive", who, fout);
  return 0;
}

}  // namespace

// The destination-tiled kernel (rgms_f32_tiles.hip: no atomics, every tile of Y written once, the
// same bits from run to run) is chosen by the caller, from this many slots on; measured on the
// RGCN layer of 100k nodes, 65 relations and 2M edges it takes 122 us from the CSF arrays and
// 134 us from ELL3D buckets (whose padding slots are edges like any other), against 159 us for
// the kernels with atomics.
constexpr int64_t kF32TileMinSlots = 8192;

struct stir_rgms_f32_plan {
  int nk;
  RgmsF32Bucket* d_table;
  int64_t total_units;
  // destination-tiled path: the index is made by the first launch (it needs m, n and num_rels)
  stir::F32Source source;
  int64_t slots;
  bool deterministic;  // see stir_rgms_f32_plan_set_deterministic
  stir::F32TileIndex tiles;
};

struct stir_rgms_csf_f32_plan {
  stir::F32Source source;
  stir::F32TileIndex tiles;
};

extern "C" {

int stir_rgms_f32_plan_create(stir_rgms_f32_plan** plan, int32_t num_buckets, const int32_t* rows_bkt,
                              const int32_t* cols_bkt, const int64_t* groups, const float* const* d_A,
                              const int32_t* const* d_rows, const int32_t* const* d_cols,
                              const int32_t* const* d_mids) {
  STIR_REQUIRE(plan && num_buckets > 0, "rgms_f32_plan_create: bad arguments");
  RgmsF32Bucket* host = new RgmsF32Bucket[num_buckets];
  int nk = 0;
  int64_t total = 0, slots = 0;
  stir::F32Source source;
  for (int b = 0; b < num_buckets; ++b) {
    if (rows_bkt[b] <= 0 || cols_bkt[b] <= 0 || groups[b] < 0) {
      delete[] host;
      return stir::fail("rgms_f32_plan_create: bucket %d has non-positive sizes", b);
    }
    if (groups[b] == 0) continue;
    if (!d_A[b] || !d_rows[b] || !d_cols[b] || !d_mids[b]) {
      delete[] host;
      return stir::fail("rgms_f32_plan_create: bucket %d has groups but a null array", b);
    }
    if ((int64_t)kTileRows * cols_bkt[b] > (int64_t(1) << 30)) {
      delete[] host;
      return stir::fail("rgms_f32_plan_create: bucket %d is too wide", b);
    }
    RgmsF32Bucket e;
    e.A = d_A[b];
    e.rows = d_rows[b];
    e.cols = d_cols[b];
    e.mids = d_mids[b];
    e.ell_rows = groups[b] * rows_bkt[b];
    e.unit_begin = total;
    e.rb = rows_bkt[b];
    e.cb = cols_bkt[b];
    if (rows_bkt[b] >= kTileRows) {
      e.tile_rows = kTileRows;
      e.chunks_per_group = (int32_t)stir::ceil_div(rows_bkt[b], kTileRows);
      total += groups[b] * e.chunks_per_group;
    } else {
      e.tile_rows = (kTileRows / rows_bkt[b]) * rows_bkt[b];
      e.chunks_per_group = 0;
      total += stir::ceil_div(e.ell_rows, e.tile_rows);
    }
    host[nk++] = e;
    source.buckets.push_back(stir::F32Bucket{e.A, e.rows, e.cols, e.mids, groups[b], e.rb, e.cb});
    slots += e.ell_rows * e.cb;
  }
  stir_rgms_f32_plan* p = new stir_rgms_f32_plan();
  p->nk = nk;
  p->total_units = total;
  p->d_table = nullptr;
  p->source = source;
  p->slots = slots;
  p->deterministic = false;
  hipError_t err = hipSuccess;
  if (nk > 0) {
    err = hipMalloc(reinterpret_cast<void**>(&p->d_table), sizeof(RgmsF32Bucket) * nk);
    if (err == hipSuccess) err = hipMemcpy(p->d_table, host, sizeof(RgmsF32Bucket) * nk, hipMemcpyHostToDevice);
  }
  delete[] host;
  if (err != hipSuccess) {
    if (p->d_table) (void)hipFree(p->d_table);
    delete p;
    return stir::fail("rgms_f32_plan_create: %s", hipGetErrorString(err));
  }
  *plan = p;
  return 0;
}

int stir_rgms_f32_plan_destroy(stir_rgms_f32_plan* plan) {
  if (!plan) return 0;
  if (plan->d_table) (void)hipFree(plan->d_table);
  stir::f32_tiles_free(plan->tiles);
  delete plan;
  return 0;
}

int stir_rgms_f32_plan_set_deterministic(stir_rgms_f32_plan* plan, int32_t on) {
  STIR_REQUIRE(plan, "rgms_f32_plan_set_deterministic: plan is null");
  if (!on) stir::f32_tiles_free(plan->tiles);
  plan->deterministic = on != 0;
  return 0;
}

#define STIR_RGMS_F32_DISPATCH(LAUNCH)  \
  switch (padded_fin(feat_in)) {        \
    case 8: LAUNCH(8, 4); break;        \
    case 16: LAUNCH(16, 4); break;      \
    case 32: LAUNCH(32, 4); break;      \
    case 64: LAUNCH(64, 4); break;      \
    default: LAUNCH(128, 2); break;     \
  }

int stir_rgms_f32(const stir_rgms_f32_plan* plan, int32_t m, int32_t n, int32_t num_rels, int32_t feat_in,
                  int32_t feat_out, const float* d_W, const float* d_X, float* d_Y, void* stream) {
  STIR_REQUIRE(plan, "rgms_f32: plan is null");
  STIR_REQUIRE(m >= 0 && n >= 0 && num_rels >= 0, "rgms_f32: bad sizes");
  if (check_feats("rgms_f32", feat_in, feat_out)) return -1;
  if (plan->nk == 0) return 0;
  STIR_REQUIRE(d_W && d_X && d_Y, "rgms_f32: null pointer argument");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (plan->deterministic && plan->slots >= kF32TileMinSlots && plan->slots < (int64_t(1) << 31) &&
      stir::f32_tiles_serves(feat_in, feat_out) && stir::f32_tiles_fits(n, feat_in, plan->slots) && m > 0 && n > 0 &&
      num_rels > 0) {
    // the plan's edge index is made by the first launch: a plan serves one call at a time
    stir_rgms_f32_plan* mp = const_cast<stir_rgms_f32_plan*>(plan);
    if (stir::f32_tiles_prepare(mp->tiles, mp->source, m, n, num_rels, feat_in, st)) return -1;
    return stir::f32_tiles_launch(mp->tiles, feat_in, feat_out, d_W, d_X, d_Y, st);
  }
#define STIR_LAUNCH(FP, WAVES)                                                                            \
  {                                                                                                       \
    const int64_t blocks = stir::ceil_div(plan->total_units, WAVES);                                      \
    STIR_REQUIRE(blocks < (int64_t(1) << 31), "rgms_f32: too many tiles for one launch");                 \
    hipLaunchKernelGGL((rgms_ell3d_f32_kernel<FP, WAVES>), dim3((unsigned)blocks), dim3(WAVES * 64), 0, st, \
                       plan->d_table, plan->nk, plan->total_units, feat_in, feat_out, d_W, d_X, d_Y);     \
  }
  STIR_RGMS_F32_DISPATCH(STIR_LAUNCH)
#undef STIR_LAUNCH
  STIR_LAUNCH_CHECK();
  return 0;
}

int stir_rgms_csf_f32(int32_t m, int32_t n, int32_t num_rels, int32_t feat_in, int32_t feat_out, int64_t nnz_i,
                      int64_t nnz_j, const float* d_A, const float* d_W, const float* d_X, float* d_Y,
                      const int32_t* d_indptr_i, const int32_t* d_indices_i, const int32_t* d_indptr_j,
                      const int32_t* d_indices_j, void* stream) {
  STIR_REQUIRE(m >= 0 && n >= 0 && num_rels >= 0 && nnz_i >= 0 && nnz_j >= 0, "rgms_csf_f32: bad sizes");
  STIR_REQUIRE(nnz_j < (int64_t(1) << 31), "rgms_csf_f32: nnz_j=%lld exceeds int32 offsets", (long long)nnz_j);
  if (check_feats("rgms_csf_f32", feat_in, feat_out)) return -1;
  if (nnz_i == 0) return 0;
  STIR_REQUIRE(d_A || nnz_j == 0, "rgms_csf_f32: edge values are null");
  STIR_REQUIRE(d_W && d_X && d_Y && d_indptr_i && d_indices_i && d_indptr_j && (d_indices_j || nnz_j == 0),
               "rgms_csf_f32: null pointer argument");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t tiles = stir::ceil_div(nnz_i, kTileRows);
#define STIR_LAUNCH(FP, WAVES)                                                                          \
  {                                                                                                     \
    const int64_t blocks = stir::ceil_div(tiles, WAVES);                                                \
    STIR_REQUIRE(blocks < (int64_t(1) << 31), "rgms_csf_f32: too many tiles for one launch");           \
    hipLaunchKernelGGL((rgms_csf_f32_kernel<FP, WAVES>), dim3((unsigned)blocks), dim3(WAVES * 64), 0, st, \
                       num_rels, nnz_i, feat_in, feat_out, d_A, d_W, d_X, d_Y, d_indptr_i, d_indices_i,  \
                       d_indptr_j, d_indices_j);                                                        \
  }
  STIR_RGMS_F32_DISPATCH(STIR_LAUNCH)
#undef STIR_LAUNCH
  STIR_LAUNCH_CHECK();
  return 0;
}

int stir_rgms_csf_f32_plan_create(stir_rgms_csf_f32_plan** plan, int64_t nnz_i, int64_t nnz_j, const float* d_A,
                                  const int32_t* d_indptr_i, const int32_t* d_indices_i, const int32_t* d_indptr_j,
                                  const int32_t* d_indices_j) {
  STIR_REQUIRE(plan, "rgms_csf_f32_plan_create: plan is null");
  STIR_REQUIRE(nnz_i >= 0 && nnz_j >= 0 && nnz_j < (int64_t(1) << 31), "rgms_csf_f32_plan_create: bad sizes");
  STIR_REQUIRE(nnz_j == 0 || (d_A && d_indptr_i && d_indices_i && d_indptr_j && d_indices_j && nnz_i > 0),
               "rgms_csf_f32_plan_create: null pointer argument");
  stir_rgms_csf_f32_plan* p = new stir_rgms_csf_f32_plan();
  p->source.csf = true;
  p->source.A = d_A;
  p->source.indptr_i = d_indptr_i;
  p->source.indices_i = d_indices_i;
  p->source.indptr_j = d_indptr_j;
  p->source.indices_j = d_indices_j;
  p->source.nnz_i = nnz_i;
  p->source.nnz_j = nnz_j;
  *plan = p;
  return 0;
}

int stir_rgms_csf_f32_planned(stir_rgms_csf_f32_plan* plan, int32_t m, int32_t n, int32_t num_rels, int32_t feat_in,
                              int32_t feat_out, const float* d_W, const float* d_X, float* d_Y, void* stream) {
  STIR_REQUIRE(plan, "rgms_csf_f32_planned: plan is null");
  STIR_REQUIRE(m >= 0 && n >= 0 && num_rels >= 0, "rgms_csf_f32: bad sizes");
  if (check_feats("rgms_csf_f32", feat_in, feat_out)) return -1;
  const stir::F32Source& s = plan->source;
  if (s.nnz_j == 0) return 0;
  STIR_REQUIRE(d_W && d_X && d_Y, "rgms_csf_f32: null pointer argument");
  if (!stir::f32_tiles_serves(feat_in, feat_out) || !stir::f32_tiles_fits(n, feat_in, s.nnz_j) ||
      s.nnz_j < kF32TileMinSlots || m <= 0 || n <= 0 || num_rels <= 0)
    return stir_rgms_csf_f32(m, n, num_rels, feat_in, feat_out, s.nnz_i, s.nnz_j, s.A, d_W, d_X, d_Y, s.indptr_i,
                             s.indices_i, s.indptr_j, s.indices_j, stream);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (stir::f32_tiles_prepare(plan->tiles, s, m, n, num_rels, feat_in, st)) return -1;
  return stir::f32_tiles_launch(plan->tiles, feat_in, feat_out, d_W, d_X, d_Y, st);
}

int stir_rgms_csf_f32_plan_destroy(stir_rgms_csf_f32_plan* plan) {
  if (!plan) return 0;
  stir::f32_tiles_free(plan->tiles);
  delete plan;
  return 0;
}

}  // extern "C"
