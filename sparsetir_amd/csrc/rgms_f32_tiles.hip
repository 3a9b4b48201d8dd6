// Destination-tiled fp32 RGMS declared in rgms_f32_tiles.h: index construction and the kernel.
//
// Index (once per plan): every slot of the ELL3D buckets -- or every stored column of the CSF
// arrays -- is an edge with the key (destination row / 64, relation, destination row % 64).  One
// stable radix sort orders the edges by key; runs of equal key are the (relation, row) pairs
// (run-length encoding of the sorted keys), and a binary search per tile finds where its pairs
// begin.  An edge record holds the source row and the address of the edge's weight (weights are
// read at every launch); a pair record its relation, its row inside the tile and its run of edges.
//
// The pairs of one (tile, relation) run are cut into batches of at most 16, listed per tile.
//
// Kernel: one workgroup of four wavefronts per 64-row tile of Y; wavefront w takes the tile's
// batches w, w + 4, ... and sums into a partial tile of its own in LDS.  Per batch (up to 16 pairs
// of one relation):
//   1. S[i, :] = sum over the edges e of pair i of weight_e * X[src_e, :], in registers: lane
//      (i = l % 16, q = l / 16) holds inputs 8q .. 8q+7 (+32 per further 32 inputs) of pair i and
//      walks the pair's edges;
//   2. P = S @ W[rel]^T on v_mfma_f32_16x16x4_f32.  The instruction's k index is lane / 16; the
//      t-th instruction takes input 8q + t from lane (., q) in both operands, so S needs no
//      rearrangement and a lane's W operands are 32 contiguous bytes of a row of W[rel];
//   3. row i of P is added to row (destination row % 64) of the wavefront's partial tile with a
//      plain LDS read-modify-write: the pairs of one relation end in different rows, and no other
//      wavefront touches this partial tile (LDS float atomics run at a third of a lane per clock
//      and compute unit on this chip, slower than atomics in memory).
// A batch is a chain of dependent loads (batch record -> pair records -> edge records -> rows of
// X), so the records run ahead of the arithmetic: batch records three batches ahead, pair records
// two, the first two edge records of every pair one; only the rows of X are waited for.
// At the end the four partial tiles are added to the tile's rows of Y, each element once.
#include "rgms_f32_tiles.h"

#include <hipcub/hipcub.hpp>

namespace stir {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 64;
constexpr int kTileShift = 6;
constexpr int kBatch = 16;  // pairs per matrix-core product

struct alignas(16) BatchF32 {
  int64_t pair_begin;
  int32_t npairs;  // at most kBatch
  int32_t rel;
};

struct alignas(16) DevBucketF32 {
  const float* A;
  const int32_t* rows;
  const int32_t* cols;
  const int32_t* mids;
  int64_t slot_begin;  // first slot of the bucket in the numbering over all buckets
  int32_t rb, cb;
};

struct CsfArrays {
  const float* A;
  const int32_t* indptr_i;
  const int32_t* indices_i;
  const int32_t* indptr_j;
  const int32_t* indices_j;
  int64_t nnz_i;
};

struct alignas(16) EdgeF32 {
  int32_t src;  // row of X
  int32_t pad;
  const float* w;  // the edge's weight
};

struct alignas(16) PairF32 {
  uint32_t rel_dl;  // relation << 6 | destination row inside its tile
  int32_t count;    // edges of the pair
  int64_t first;    // its first sorted edge
};

__device__ __forceinline__ int bucket_of(const DevBucketF32* __restrict__ tab, int nb, int64_t q) {
  int lo = 0, hi = nb - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (tab[mid].slot_begin <= q) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// last index i in [0, count] with ptr[i] <= q, minus nothing: the row of position q when ptr is a
// row-pointer array of count rows (count + 1 entries)
__device__ __forceinline__ int64_t row_of(const int32_t* __restrict__ ptr, int64_t count, int64_t q) {
  int64_t lo = 0, hi = count;  // answer in [0, count - 1] for well-formed input
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if ((int64_t)ptr[mid] <= q) lo = mid; else hi = mid - 1;
  }
  return min(lo, count - 1);
}

// destination row, relation, source row and weight address of edge q
template <bool CSF>
__device__ __forceinline__ void edge_of(const DevBucketF32* __restrict__ tab, int nb, const CsfArrays& csf,
                                        int num_rels, int64_t q, int& dest, int& rel, int& src, const float*& w) {
  if constexpr (CSF) {
    const int64_t p = row_of(csf.indptr_j, csf.nnz_i, q);
    dest = csf.indices_i[p];
    rel = (int)row_of(csf.indptr_i, num_rels, p);
    src = csf.indices_j[q];
    w = csf.A + q;
  } else {
    const DevBucketF32 bk = tab[bucket_of(tab, nb, q)];
    const int64_t local = q - bk.slot_begin;
    const int64_t gs = (int64_t)bk.rb * bk.cb;
    const int64_t g = local / gs;
    const int r = (int)((local - g * gs) / bk.cb);
    dest = bk.rows[g * bk.rb + r];
    rel = bk.mids[g];
    src = bk.cols[local];
    w = bk.A + local;
  }
}

template <bool CSF>
__global__ __launch_bounds__(256) void f32_edge_keys_kernel(const DevBucketF32* __restrict__ tab, int nb, CsfArrays csf,
                                                            int64_t slots, int m, int n, int num_rels,
                                                            uint64_t* __restrict__ keys, int32_t* __restrict__ vals,
                                                            int32_t* __restrict__ bad) {
  const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (q >= slots) return;
  int dest, rel, src;
  const float* w;
  edge_of<CSF>(tab, nb, csf, num_rels, q, dest, rel, src, w);
  if ((unsigned)dest >= (unsigned)m || (unsigned)rel >= (unsigned)num_rels) {
    *bad = 1;
    dest = rel = 0;
  }
  if ((unsigned)src >= (unsigned)n) *bad = 2;
  keys[q] = ((((uint64_t)(dest >> kTileShift)) * num_rels + rel) << kTileShift) | (uint64_t)(dest & (kTileRows - 1));
  vals[q] = (int32_t)q;
}

template <bool CSF>
__global__ __launch_bounds__(256) void f32_edge_records_kernel(const DevBucketF32* __restrict__ tab, int nb,
                                                               CsfArrays csf, int64_t slots, int num_rels,
                                                               const int32_t* __restrict__ vals,
                                                               EdgeF32* __restrict__ edges) {
  const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (p >= slots) return;
  int dest, rel, src;
  const float* w;
  edge_of<CSF>(tab, nb, csf, num_rels, vals[p], dest, rel, src, w);
  EdgeF32 e;
  e.src = src;
  e.pad = 0;
  e.w = w;
  edges[p] = e;
}

__global__ __launch_bounds__(256) void f32_pairs_kernel(const uint64_t* __restrict__ unique, const int32_t* __restrict__ counts,
                                                        const int32_t* __restrict__ first, int64_t pairs, int num_rels,
                                                        PairF32* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= pairs) return;
  const uint64_t key = unique[i];
  PairF32 p;
  p.rel_dl = (uint32_t)(((key >> kTileShift) % (uint64_t)num_rels) << kTileShift) | (uint32_t)(key & (kTileRows - 1));
  p.count = counts[i];
  p.first = first[i];
  out[i] = p;
}

// batches of run i (a (tile, relation) run of `count` pairs starting at pair `first`)
__global__ __launch_bounds__(256) void f32_batch_count_kernel(const int32_t* __restrict__ run_pairs, int64_t runs,
                                                              int32_t* __restrict__ run_batches) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < runs) run_batches[i] = (run_pairs[i] + kBatch - 1) / kBatch;
}

__global__ __launch_bounds__(256) void f32_batch_fill_kernel(const uint64_t* __restrict__ run_keys,
                                                             const int32_t* __restrict__ run_pairs,
                                                             const int32_t* __restrict__ run_first_pair,
                                                             const int32_t* __restrict__ run_first_batch, int64_t runs,
                                                             int num_rels, BatchF32* __restrict__ batches) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= runs) return;
  const int count = run_pairs[i];
  const int rel = (int)(run_keys[i] % (uint64_t)num_rels);
  for (int k = 0; k * kBatch < count; ++k) {
    BatchF32 b;
    b.pair_begin = (int64_t)run_first_pair[i] + k * kBatch;
    b.npairs = min(kBatch, count - k * kBatch);
    b.rel = rel;
    batches[run_first_batch[i] + k] = b;
  }
}

// begin[t] = first batch of tile t (t = tiles gives the batch count): the first run whose key
// (tile * num_rels + relation) is not below t * num_rels
__global__ __launch_bounds__(256) void f32_tile_batches_kernel(const uint64_t* __restrict__ run_keys,
                                                               const int32_t* __restrict__ run_first_batch, int64_t runs,
                                                               int64_t total_batches, int64_t tiles, int num_rels,
                                                               int64_t* __restrict__ begin) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t > tiles) return;
  const uint64_t target = (uint64_t)t * num_rels;
  int64_t lo = 0, hi = runs;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (run_keys[mid] < target) lo = mid + 1; else hi = mid;
  }
  begin[t] = lo < runs ? run_first_batch[lo] : total_batches;
}

__global__ __launch_bounds__(256) void f32_shift_keys_kernel(const uint64_t* __restrict__ in, int64_t count,
                                                             uint64_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < count) out[i] = in[i] >> kTileShift;
}

typedef __attribute__((address_space(1))) const float GlobalF32;  // a global-memory load, not a flat one

// W[rel][16 nt + i][32 s + 8 q + 4 c .. + 3] -> Wp[((rel * NT + nt) * KS + s) * 2 + c][lane (i, q)]: the
// B operands of a batch as four-float words in lane order, so that the kernel's loads of W are
// contiguous (a lane of the multiply owns one row of W per output tile: read in place, the 64
// lanes of a load would touch 16 different lines four times over).  Zero beyond feat_in and
// feat_out.  One thread per word.
__global__ __launch_bounds__(256) void f32_pack_w_kernel(const float* __restrict__ W, float4* __restrict__ Wp,
                                                         int64_t words, int nt_count, int ks_count, int fin, int fout) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= words) return;
  const int lane = (int)(t & 63), i = lane & 15, q = lane >> 4;
  int64_t f = t >> 6;
  const int c = (int)(f & 1);
  f >>= 1;
  const int s = (int)(f % ks_count);
  f /= ks_count;
  const int nt = (int)(f % nt_count);
  const int64_t rel = f / nt_count;
  const int out = 16 * nt + i, k = 32 * s + 8 * q + 4 * c;
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (out < fout && k < fin) v = *reinterpret_cast<const float4*>(W + (rel * fout + out) * fin + k);
  Wp[t] = v;
}

// KS: feat_in <= 32 * KS; NT: feat_out <= 16 * NT.
//
// Two lane layouts.  Gathering: a row of X (or its first 32 KS floats) is spread over CPR = 8 KS
// neighbouring lanes, four floats each, so that a load instruction reads 64 / CPR whole rows and
// the texture addresser sees whole lines per quad of lanes; a lane serves the same (pair, chunk)
// for every edge of the pair and sums in registers.  Multiplying: lane (i = l % 16, q = l / 16)
// holds inputs 8q .. 8q+7 of pair i.  The sums change layout through a 16 x 32 KS tile of LDS per
// wavefront, one write and one read per batch; the pairs' rows inside the tile of Y travel the
// same way.
//
// The loads of the batch loop are unconditional -- indices are clamped to records that exist and
// what must not count is multiplied by zero afterwards -- so that the loop body is one basic
// block: the rows of X of the current batch are requested first and waited for alone, while the
// records of the next batches, requested behind them, stay in flight during the arithmetic.
// Offsets into X, the pair records and the edge records are 32-bit byte offsets from scalar bases
// (the launch checks that they fit).
template <int KS, int NT>
__global__ __launch_bounds__(256) void rgms_f32_tile_kernel(int m, int fin, int fout, int64_t total_batches,
                                                               const int64_t* __restrict__ tile_batches,
                                                               const BatchF32* __restrict__ batches,
                                                               const PairF32* __restrict__ pairs,
                                                               const EdgeF32* __restrict__ edges,
                                                               const float4* __restrict__ Wp,
                                                               const float* __restrict__ X, float* __restrict__ Y) {
  constexpr int FO = 16 * NT;      // floats per row of a partial tile
  constexpr int CPR = 8 * KS;      // lanes (16-byte chunks) per gathered row
  constexpr int RPI = 64 / CPR;    // rows per load instruction
  constexpr int PASSES = kBatch / RPI;
  constexpr int SS = 32 * KS + 4;  // floats per row of the S tile: 16 lanes reading 32 bytes each hit 64 banks
  constexpr int U = 2;             // edges of a pair whose records are fetched a batch ahead
  __shared__ __attribute__((aligned(16))) float ytile[4][kTileRows * FO];
  __shared__ __attribute__((aligned(16))) float stile[4][kBatch * SS];
  __shared__ __attribute__((aligned(16))) int32_t dtile[4][kBatch];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i = lane & 15, q = lane >> 4;  // multiplying
  const int gr = lane / CPR, gc = lane % CPR;  // gathering
  const int64_t tile = blockIdx.x;
  float* yt = ytile[wave];
  float* st = stile[wave];
  int32_t* dt = dtile[wave];
  for (int e = lane; e < kTileRows * FO; e += 64) yt[e] = 0.f;

  const int64_t b_end = tile_batches[tile + 1];
  int64_t b = tile_batches[tile] + wave;
  const bool chunk_live = 4 * gc < fin;  // fin is a multiple of 4: chunks are whole
  const uint32_t x_off = chunk_live ? 16u * gc : 0u;
  const float x_keep = chunk_live ? 1.f : 0.f;
  const uint32_t row_bytes = 4u * (uint32_t)fin;
  const char* Xb = reinterpret_cast<const char*>(X);
  const char* Pb = reinterpret_cast<const char*>(pairs);
  const char* Eb = reinterpret_cast<const char*>(edges);

  struct Batch {
    uint32_t pair_off;  // bytes
    int npairs, rel;
  };
  auto load_batch = [&](int64_t bi) {  // the same for every lane: one address per wavefront
    const BatchF32 t = batches[min(bi, total_batches - 1)];
    Batch r;
    r.pair_off = __builtin_amdgcn_readfirstlane((uint32_t)t.pair_begin * 16u);
    r.npairs = bi < b_end ? __builtin_amdgcn_readfirstlane(t.npairs) : 0;
    r.rel = __builtin_amdgcn_readfirstlane(t.rel);
    return r;
  };
  // gathering layout: in pass p the lane serves pair p * RPI + gr of the batch
  struct PairsG {
    uint32_t first[PASSES];  // bytes into the edge records
    int count[PASSES];
    int dl[PASSES];
  };
  auto load_pairs = [&](const Batch& bt) {  // a lane without a pair repeats the batch's first one with no edges
    PairsG r;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int slot = p * RPI + gr;
      const PairF32 pr = *reinterpret_cast<const PairF32*>(Pb + (bt.pair_off + (slot < bt.npairs ? 16u * slot : 0u)));
      r.first[p] = (uint32_t)pr.first * 16u;
      r.count[p] = slot < bt.npairs ? pr.count : 0;
      r.dl[p] = (int)(pr.rel_dl & (kTileRows - 1));
    }
    return r;
  };
  struct EdgesG {
    EdgeF32 e[PASSES][U];
  };
  auto load_edges = [&](const PairsG& pg) {  // beyond the pair's last edge: its first one again
    EdgesG r;
#pragma unroll
    for (int p = 0; p < PASSES; ++p)
#pragma unroll
      for (int u = 0; u < U; ++u)
        r.e[p][u] = *reinterpret_cast<const EdgeF32*>(Eb + (pg.first[p] + (u < pg.count[p] ? 16u * u : 0u)));
    return r;
  };
  auto weight_of = [](const EdgeF32& e) { return *reinterpret_cast<GlobalF32*>(reinterpret_cast<uintptr_t>(e.w)); };
  auto fma4 = [](float4& acc, float w, const float4& x) {
    acc.x += w * x.x, acc.y += w * x.y, acc.z += w * x.z, acc.w += w * x.w;
  };

  // the pipeline: batch records three ahead, pair records two, first edge records one
  Batch bt0 = load_batch(b), bt1 = load_batch(b + 4), bt2 = load_batch(b + 8);
  PairsG pg0 = load_pairs(bt0), pg1 = load_pairs(bt1);
  EdgesG eg0 = load_edges(pg0);

  while (bt0.npairs > 0) {  // the same for every lane
    const int rel0 = bt0.rel, npairs = bt0.npairs;
    // the rows of X and the weights of the pairs' first U edges
    float wv[PASSES][U];
    float4 xv[PASSES][U];
#pragma unroll
    for (int p = 0; p < PASSES; ++p)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        wv[p][u] = weight_of(eg0.e[p][u]);
        xv[p][u] = *reinterpret_cast<const float4*>(Xb + ((uint32_t)eg0.e[p][u].src * row_bytes + x_off));
      }
    // B operands of rel0, in lane order
    float4 wq[NT][KS][2];
    const float4* wrel = Wp + (int64_t)rel0 * (NT * KS * 2 * 64) + lane;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int c = 0; c < 2; ++c) wq[nt][s][c] = wrel[((nt * KS + s) * 2 + c) * 64];
    // the records of the batches to come
    const Batch bt3 = load_batch(b + 12);
    const PairsG pg2 = load_pairs(bt2);
    const EdgesG eg1 = load_edges(pg1);

    // the weighted sums of the pairs' rows of X, gathering layout
    float4 sum[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      sum[p] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int u = 0; u < U; ++u) fma4(sum[p], u < pg0.count[p] ? wv[p][u] : 0.f, xv[p][u]);
    }
    int most = 0;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) most = max(most, pg0.count[p]);
    for (int t0 = U; __ballot(t0 < most) != 0; t0 += U) {  // pairs of more than U edges: two round trips per pass
      EdgeF32 er[PASSES][U];
#pragma unroll
      for (int p = 0; p < PASSES; ++p)
#pragma unroll
        for (int u = 0; u < U; ++u)
          er[p][u] = *reinterpret_cast<const EdgeF32*>(Eb + (pg0.first[p] + (t0 + u < pg0.count[p] ? 16u * (t0 + u) : 0u)));
      float w2[PASSES][U];
      float4 x2[PASSES][U];
#pragma unroll
      for (int p = 0; p < PASSES; ++p)
#pragma unroll
        for (int u = 0; u < U; ++u) {
          w2[p][u] = weight_of(er[p][u]);
          x2[p][u] = *reinterpret_cast<const float4*>(Xb + ((uint32_t)er[p][u].src * row_bytes + x_off));
        }
#pragma unroll
      for (int p = 0; p < PASSES; ++p)
#pragma unroll
        for (int u = 0; u < U; ++u) fma4(sum[p], t0 + u < pg0.count[p] ? w2[p][u] : 0.f, x2[p][u]);
    }
    // through LDS into the multiplying layout (chunks beyond feat_in were read from the row's start: zero)
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int slot = p * RPI + gr;
      float4 v = sum[p];
      v.x *= x_keep, v.y *= x_keep, v.z *= x_keep, v.w *= x_keep;
      *reinterpret_cast<float4*>(st + slot * SS + 4 * gc) = v;
      if (gc == 0) dt[slot] = pg0.dl[p];
    }
    float4 sq[KS][2];
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int c = 0; c < 2; ++c) sq[s][c] = *reinterpret_cast<const float4*>(st + i * SS + 32 * s + 8 * q + 4 * c);
    const int4 dl4 = *reinterpret_cast<const int4*>(dt + 4 * q);

    f32x4 acc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const float4 wk = wq[nt][s][c], sk = sq[s][c];
          acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(sk.x, wk.x, acc[nt], 0, 0, 0);
          acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(sk.y, wk.y, acc[nt], 0, 0, 0);
          acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(sk.z, wk.z, acc[nt], 0, 0, 0);
          acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(sk.w, wk.w, acc[nt], 0, 0, 0);
        }

    // acc[nt][v]: pair 4 q + v of the batch, output 16 nt + i.  Rows of the partial tile are 16 NT
    // floats; the column is rotated by 16 for every second pair of rows, which keeps most of the
    // four rows an instruction touches on different banks.
    const int dls[4] = {dl4.x, dl4.y, dl4.z, dl4.w};
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      if (4 * q + v < npairs) {
        const int dl = dls[v];
        float* row = yt + dl * FO;
        const int rot = 16 * ((dl >> 1) & 1);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) row[((16 * nt + rot) & (FO - 1)) + i] += acc[nt][v];
      }
    }
    b += 4;
    bt0 = bt1, bt1 = bt2, bt2 = bt3;
    pg0 = pg1, pg1 = pg2;
    eg0 = eg1;
  }

  __syncthreads();
  const int64_t row0 = tile * kTileRows;
  for (int e = tid; e < kTileRows * fout; e += 256) {
    const int r = e / fout, c = e - r * fout;
    if (row0 + r >= m) break;
    const int at = r * FO + ((((c >> 4) * 16 + 16 * ((r >> 1) & 1)) & (FO - 1)) + (c & 15));
    const float sum = (ytile[0][at] + ytile[1][at]) + (ytile[2][at] + ytile[3][at]);
    float* y = Y + (row0 + r) * fout + c;
    *y += sum;
  }
}

struct Scratch {
  std::vector<void*> ptrs;
  ~Scratch() {
    for (void* p : ptrs) (void)hipFree(p);
  }
  template <typename T>
  int get(T** out, size_t count) {
    void* p = nullptr;
    STIR_HIP(hipMalloc(&p, std::max<size_t>(count * sizeof(T), 256)));
    ptrs.push_back(p);
    *out = static_cast<T*>(p);
    return 0;
  }
};

}  // namespace

namespace {
int build_index(F32TileIndex& idx, const F32Source& src, int32_t m, int32_t n, int32_t num_rels, hipStream_t stream);
}

bool f32_tiles_serves(int32_t feat_in, int32_t feat_out) {
  return feat_in > 0 && feat_in % 4 == 0 && feat_in <= 64 && feat_out > 0 && feat_out <= 64;
}

void f32_tiles_free(F32TileIndex& idx) {
  if (idx.d_edges) (void)hipFree(idx.d_edges);
  if (idx.d_pairs) (void)hipFree(idx.d_pairs);
  if (idx.d_batches) (void)hipFree(idx.d_batches);
  if (idx.d_wpack) (void)hipFree(idx.d_wpack);
  if (idx.d_tile_pairs) (void)hipFree(idx.d_tile_pairs);
  idx = F32TileIndex();
}

int f32_tiles_prepare(F32TileIndex& idx, const F32Source& src, int32_t m, int32_t n, int32_t num_rels,
                      hipStream_t stream) {
  if (idx.m == m && idx.n == n && idx.num_rels == num_rels) return 0;
  f32_tiles_free(idx);
  F32TileIndex built;
  const int rc = build_index(built, src, m, n, num_rels, stream);
  if (rc != 0) {
    f32_tiles_free(built);  // nothing half-made stays behind
    return rc;
  }
  idx = built;
  return 0;
}

namespace {
int build_index(F32TileIndex& idx, const F32Source& src, int32_t m, int32_t n, int32_t num_rels, hipStream_t stream) {
  STIR_REQUIRE(m > 0 && n > 0 && num_rels > 0, "rgms_f32: m, n and num_rels must be positive");
  // edges and their numbering
  std::vector<DevBucketF32> tab;
  int64_t slots = 0;
  if (src.csf) {
    slots = src.nnz_j;
  } else {
    for (const F32Bucket& b : src.buckets) {
      if (b.groups == 0) continue;
      tab.push_back(DevBucketF32{b.A, b.rows, b.cols, b.mids, slots, b.rb, b.cb});
      slots += b.groups * b.rb * b.cb;
    }
  }
  STIR_REQUIRE(slots < (int64_t(1) << 31), "rgms_f32: %lld slots exceed 32-bit edge numbers", (long long)slots);
  const int64_t tiles = ceil_div(m, kTileRows);
  STIR_REQUIRE((double)tiles * num_rels * kTileRows < 9e18, "rgms_f32: sort keys exceed 64 bits");
  idx.m = m, idx.n = n, idx.num_rels = num_rels;
  idx.edges = slots, idx.tiles = tiles;
  STIR_HIP(hipMalloc(&idx.d_tile_pairs, sizeof(int64_t) * (size_t)(tiles + 1)));
  if (slots == 0) {
    idx.pairs = 0;
    STIR_HIP(hipMemsetAsync(idx.d_tile_pairs, 0, sizeof(int64_t) * (size_t)(tiles + 1), stream));
    STIR_HIP(hipStreamSynchronize(stream));
    return 0;
  }
  Scratch tmp;
  DevBucketF32* d_tab = nullptr;
  if (!tab.empty()) {
    if (tmp.get(&d_tab, tab.size())) return -1;
    STIR_HIP(hipMemcpyAsync(d_tab, tab.data(), sizeof(DevBucketF32) * tab.size(), hipMemcpyHostToDevice, stream));
  }
  const CsfArrays csf = {src.A, src.indptr_i, src.indices_i, src.indptr_j, src.indices_j, src.nnz_i};
  uint64_t *keys_in = nullptr, *keys_out = nullptr, *unique = nullptr;
  int32_t *vals_in = nullptr, *vals_out = nullptr, *counts = nullptr, *first = nullptr, *flags = nullptr;
  if (tmp.get(&keys_in, slots) || tmp.get(&keys_out, slots) || tmp.get(&unique, slots) || tmp.get(&vals_in, slots) ||
      tmp.get(&vals_out, slots) || tmp.get(&counts, slots) || tmp.get(&first, slots) || tmp.get(&flags, 2))
    return -1;
  STIR_HIP(hipMemsetAsync(flags, 0, sizeof(int32_t) * 2, stream));
  const dim3 grid((unsigned)ceil_div(slots, 256)), block(256);
  const int nb = (int)tab.size();
  if (src.csf)
    hipLaunchKernelGGL(f32_edge_keys_kernel<true>, grid, block, 0, stream, d_tab, nb, csf, slots, m, n, num_rels, keys_in,
                       vals_in, flags);
  else
    hipLaunchKernelGGL(f32_edge_keys_kernel<false>, grid, block, 0, stream, d_tab, nb, csf, slots, m, n, num_rels,
                       keys_in, vals_in, flags);
  STIR_LAUNCH_CHECK();
  int key_bits = kTileShift;
  while (key_bits < 64 && ((uint64_t)tiles * num_rels) >> (key_bits - kTileShift)) ++key_bits;
  size_t sort_bytes = 0, rle_bytes = 0, scan_bytes = 0;
  STIR_HIP(hipcub::DeviceRadixSort::SortPairs(nullptr, sort_bytes, keys_in, keys_out, vals_in, vals_out, (int)slots, 0,
                                              key_bits, stream));
  STIR_HIP(hipcub::DeviceRunLengthEncode::Encode(nullptr, rle_bytes, keys_out, unique, counts, flags + 1, (int)slots,
                                                 stream));
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(nullptr, scan_bytes, counts, first, (int)slots, stream));
  char* cub_tmp = nullptr;
  if (tmp.get(&cub_tmp, std::max(sort_bytes, std::max(rle_bytes, scan_bytes)))) return -1;
  STIR_HIP(hipcub::DeviceRadixSort::SortPairs(cub_tmp, sort_bytes, keys_in, keys_out, vals_in, vals_out, (int)slots, 0,
                                              key_bits, stream));
  STIR_HIP(hipMalloc(&idx.d_edges, sizeof(EdgeF32) * (size_t)slots));
  if (src.csf)
    hipLaunchKernelGGL(f32_edge_records_kernel<true>, grid, block, 0, stream, d_tab, nb, csf, slots, num_rels, vals_out,
                       static_cast<EdgeF32*>(idx.d_edges));
  else
    hipLaunchKernelGGL(f32_edge_records_kernel<false>, grid, block, 0, stream, d_tab, nb, csf, slots, num_rels,
                       vals_out, static_cast<EdgeF32*>(idx.d_edges));
  STIR_LAUNCH_CHECK();
  STIR_HIP(hipcub::DeviceRunLengthEncode::Encode(cub_tmp, rle_bytes, keys_out, unique, counts, flags + 1, (int)slots,
                                                 stream));
  int32_t host_flags[2] = {0, 0};
  STIR_HIP(hipMemcpyAsync(host_flags, flags, sizeof(host_flags), hipMemcpyDeviceToHost, stream));
  STIR_HIP(hipStreamSynchronize(stream));
  if (host_flags[0] != 0)
    return fail(host_flags[0] == 1 ? "rgms_f32: a row id or relation id lies outside [0, m) / [0, num_rels)"
                                   : "rgms_f32: a column id lies outside [0, n)");
  const int64_t pairs = host_flags[1];
  idx.pairs = pairs;
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(cub_tmp, scan_bytes, counts, first, (int)pairs, stream));
  STIR_HIP(hipMalloc(&idx.d_pairs, sizeof(PairF32) * (size_t)std::max<int64_t>(pairs, 1)));
  hipLaunchKernelGGL(f32_pairs_kernel, dim3((unsigned)ceil_div(pairs, 256)), block, 0, stream, unique, counts, first,
                     pairs, num_rels, static_cast<PairF32*>(idx.d_pairs));
  STIR_LAUNCH_CHECK();
  STIR_LAUNCH_CHECK();
  // the (tile, relation) runs of pairs and their batches.  keys_in / vals_in / keys_out / vals_out are free again
  uint64_t* run_of_pair = keys_in;   // pair key without the row
  uint64_t* run_keys = keys_out;
  int32_t *run_pairs = vals_in, *run_first_pair = vals_out;
  int32_t *run_batches = nullptr, *run_first_batch = nullptr;
  if (tmp.get(&run_batches, pairs + 1) || tmp.get(&run_first_batch, pairs + 1)) return -1;
  hipLaunchKernelGGL(f32_shift_keys_kernel, dim3((unsigned)ceil_div(pairs, 256)), block, 0, stream, unique, pairs,
                     run_of_pair);
  STIR_LAUNCH_CHECK();
  size_t rle2 = 0, scan2 = 0;
  STIR_HIP(hipcub::DeviceRunLengthEncode::Encode(nullptr, rle2, run_of_pair, run_keys, run_pairs, flags + 1, (int)pairs,
                                                 stream));
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(nullptr, scan2, run_pairs, run_first_pair, (int)pairs + 1, stream));
  STIR_REQUIRE(std::max(rle2, scan2) <= std::max(sort_bytes, std::max(rle_bytes, scan_bytes)),
               "rgms_f32: scratch of the index build is too small");
  STIR_HIP(hipcub::DeviceRunLengthEncode::Encode(cub_tmp, rle2, run_of_pair, run_keys, run_pairs, flags + 1, (int)pairs,
                                                 stream));
  STIR_HIP(hipMemcpyAsync(host_flags, flags, sizeof(host_flags), hipMemcpyDeviceToHost, stream));
  STIR_HIP(hipStreamSynchronize(stream));
  const int64_t runs = host_flags[1];
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(cub_tmp, scan2, run_pairs, run_first_pair, (int)runs, stream));
  hipLaunchKernelGGL(f32_batch_count_kernel, dim3((unsigned)ceil_div(runs, 256)), block, 0, stream, run_pairs, runs,
                     run_batches);
  STIR_LAUNCH_CHECK();
  // one entry more than runs: the last one is the batch count (run_batches[runs] is not read as an addend)
  STIR_HIP(hipMemsetAsync(run_batches + runs, 0, sizeof(int32_t), stream));
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(cub_tmp, scan2, run_batches, run_first_batch, (int)runs + 1, stream));
  int32_t total_batches = 0;
  STIR_HIP(hipMemcpyAsync(&total_batches, run_first_batch + runs, sizeof(int32_t), hipMemcpyDeviceToHost, stream));
  STIR_HIP(hipStreamSynchronize(stream));
  idx.batches = total_batches;
  STIR_HIP(hipMalloc(&idx.d_batches, sizeof(BatchF32) * (size_t)std::max<int64_t>(total_batches, 1)));
  hipLaunchKernelGGL(f32_batch_fill_kernel, dim3((unsigned)ceil_div(runs, 256)), block, 0, stream, run_keys, run_pairs,
                     run_first_pair, run_first_batch, runs, num_rels, static_cast<BatchF32*>(idx.d_batches));
  STIR_LAUNCH_CHECK();
  hipLaunchKernelGGL(f32_tile_batches_kernel, dim3((unsigned)ceil_div(tiles + 1, 256)), block, 0, stream, run_keys,
                     run_first_batch, runs, (int64_t)total_batches, tiles, num_rels,
                     static_cast<int64_t*>(idx.d_tile_pairs));
  STIR_LAUNCH_CHECK();
  STIR_HIP(hipStreamSynchronize(stream));  // the scratch arrays go away
  return 0;
}
}  // namespace

int f32_tiles_launch(F32TileIndex& idx, int32_t feat_in, int32_t feat_out, const float* d_W, const float* d_X,
                     float* d_Y, hipStream_t stream) {
  STIR_REQUIRE(f32_tiles_serves(feat_in, feat_out), "rgms_f32: feature sizes %d -> %d are not served by the tiled kernel",
               feat_in, feat_out);
  if (idx.pairs == 0) return 0;
  STIR_REQUIRE(idx.tiles < (int64_t(1) << 31), "rgms_f32: too many tiles for one launch");
  // the kernel's 32-bit byte offsets
  STIR_REQUIRE((int64_t)idx.n * feat_in * 4 < (int64_t(1) << 32) && idx.edges * 16 < (int64_t(1) << 32),
               "rgms_f32: the tiled kernel addresses X and its index with 32-bit offsets");
  const int ks = feat_in <= 32 ? 1 : 2, nt = feat_out <= 32 ? 2 : 4;
  // W in operand order, rewritten by every launch (W may change between launches)
  const int64_t words = (int64_t)idx.num_rels * nt * ks * 2 * 64;
  const size_t need = sizeof(float4) * (size_t)words;
  if (need > idx.wpack_bytes) {
    if (idx.d_wpack) STIR_HIP(hipFree(idx.d_wpack));
    idx.d_wpack = nullptr, idx.wpack_bytes = 0;
    STIR_HIP(hipMalloc(&idx.d_wpack, need));
    idx.wpack_bytes = need;
  }
  float4* wp = static_cast<float4*>(idx.d_wpack);
  hipLaunchKernelGGL(f32_pack_w_kernel, dim3((unsigned)ceil_div(words, 256)), dim3(256), 0, stream, d_W, wp, words, nt, ks,
                     feat_in, feat_out);
  STIR_LAUNCH_CHECK();
  const dim3 grid((unsigned)idx.tiles), block(256);
  const int64_t* tp = static_cast<const int64_t*>(idx.d_tile_pairs);
  const BatchF32* bts = static_cast<const BatchF32*>(idx.d_batches);
  const PairF32* pairs = static_cast<const PairF32*>(idx.d_pairs);
  const EdgeF32* edges = static_cast<const EdgeF32*>(idx.d_edges);
#define STIR_F32_TILE(KS, NT)                                                                                       \
  hipLaunchKernelGGL((rgms_f32_tile_kernel<KS, NT>), grid, block, 0, stream, idx.m, feat_in, feat_out, idx.batches, tp, \
                     bts, pairs, edges, wp, d_X, d_Y)
  if (ks == 1) {
    if (nt == 2) STIR_F32_TILE(1, 2); else STIR_F32_TILE(1, 4);
  } else {
    if (nt == 2) STIR_F32_TILE(2, 2); else STIR_F32_TILE(2, 4);
  }
#undef STIR_F32_TILE
  STIR_LAUNCH_CHECK();
  return 0;
}

}  // namespace stir
