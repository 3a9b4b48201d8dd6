// Destination-tiled fp32 RGMS declared in rgms_f32_tiles.h: index construction and the kernels.
//
// Index (once per plan): every slot of the ELL3D buckets -- or every stored column of the CSF
// arrays -- is an edge with the key (destination row / 64, relation, destination row % 64).  One
// stable radix sort orders the edges by key; runs of equal key are the (relation, row) pairs, cut
// into pieces of at most EMAX = 32 / KS edges (a second key: key << 20 | position in the run /
// EMAX, run-length encoded).  The pairs of one (tile, relation) run are cut into batches of at
// most 16 pairs and at most EMAX edges, listed per tile; a tile with many more batches than the
// average is cut into several units, whose partial tiles go to memory of the plan; the unit of a
// tile that finishes last adds them up, in the order of the units.
// An edge record holds the source row and the address of the edge's weight (weights are read at
// every launch); a pair is one word: row inside the tile, edges, first edge inside its batch.
//
// Kernel: one workgroup of four wavefronts per unit; wavefront w takes the unit's batches w,
// w + 4, ... and sums into a partial tile of its own in LDS.  Per batch:
//   1. the rows of X of the batch's edges, times their weights, go to a tile of LDS, eight rows
//      (128 bytes each) per load instruction: every lane useful whatever the pairs look like;
//   2. lane (i = l % 16, q = l / 16) adds up the rows of pair i from that tile: inputs 8q .. 8q+7
//      (+32 per further 32 inputs) of S[i, :] = sum over the edges e of pair i of w_e X[src_e, :];
//   3. P = S @ W[rel]^T on v_mfma_f32_16x16x4_f32.  The instruction's k index is lane / 16; the
//      t-th instruction takes input 8q + t from lane (., q) in both operands, so S needs no
//      rearrangement and a lane's W operands are 32 contiguous bytes of a row of W[rel];
//   4. row i of P is added to row (destination row % 64) of the wavefront's partial tile with a
//      plain LDS read-modify-write: the pairs of a batch end in different rows or in pieces of
//      one row that this lane order adds one after the other, and no other wavefront touches
//      this partial tile (LDS float atomics run at a third of a lane per clock and compute unit
//      on this chip, slower than atomics in memory).
// A batch is a chain of dependent loads (batch record -> edge records -> rows of X and weights),
// so everything is requested two of the wavefront's batches before the step of the chain that
// needs it, into registers that are never copied while a load is in flight (two sets, a loop
// unrolled by two); the loop body has no branch around a load.
// At the end the four partial tiles are added up: into the tile's rows of Y, each element once,
// or -- for a unit that is a piece of a tile -- into the plan's memory for partial tiles, with
// device-coherent stores.  Such a unit then counts itself in (a counter per cut tile); the one
// that counts last reads the partial tiles of all, coherently, adds them in unit order into Y and
// sets the counter back to zero: no second launch, no fence that writes back or invalidates a
// whole L2, and the same bits whichever unit comes last.
#include "rgms_f32_tiles.h"

#include <algorithm>

#include <hipcub/hipcub.hpp>

namespace stir {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 64;
constexpr int kTileShift = 6;
constexpr int kBatch = 16;    // pairs per matrix-core product
constexpr int kSubBits = 20;  // pieces of one (relation, row) run in the second sort key

struct alignas(16) BatchF32 {
  int32_t pair_begin;  // first pair word
  int32_t edge_begin;  // first sorted edge
  uint32_t counts;     // pairs (at most kBatch) | edges << 8 (at most EMAX) | most edges of a pair << 16
  int32_t rel;
};

struct alignas(16) UnitF32 {
  int32_t tile;
  int32_t batch_begin, batch_end;
  int32_t partial;  // -1: the unit is a whole tile and adds to Y; else its place among the partial tiles
  // of a unit that is a piece of a tile: the first partial tile of the tile, its pieces, and its
  // number among the cut tiles (its counter)
  int32_t first_partial, pieces, cut_tile, pad;
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

// key2[i] = key[i] << kSubBits | (position of sorted edge i in its run of equal key) / emax; `first`
// holds the first sorted edge of every run.  flags[0] = 3 when a run has more pieces than fit.
__global__ __launch_bounds__(256) void f32_subkeys_kernel(const uint64_t* __restrict__ keys,
                                                          const int32_t* __restrict__ first, int64_t runs, int64_t slots,
                                                          int emax, uint64_t* __restrict__ key2, int32_t* __restrict__ flags) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= slots) return;
  int64_t lo = 0, hi = runs - 1;  // last run whose first edge is not behind i
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if ((int64_t)first[mid] <= i) lo = mid; else hi = mid - 1;
  }
  int64_t piece = (i - first[lo]) / emax;
  if (piece >= (int64_t(1) << kSubBits)) {
    flags[0] = 3;
    piece = (int64_t(1) << kSubBits) - 1;
  }
  key2[i] = (keys[i] << kSubBits) | (uint64_t)piece;
}

// the (tile, relation) part of a pair's second key
__global__ __launch_bounds__(256) void f32_shift_keys_kernel(const uint64_t* __restrict__ in, int64_t count,
                                                             uint64_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < count) out[i] = in[i] >> (kSubBits + kTileShift);
}

// Run i is a (tile, relation) run of run_pairs[i] pairs starting at pair run_first_pair[i]: its
// pairs, in order, fill batches of at most kBatch pairs and at most emax edges.  Counts the
// batches (FILL = false) or writes them and the pairs' words (FILL = true).  A pair has at most
// emax edges (f32_subkeys_kernel), so every batch takes at least one.
template <bool FILL>
__global__ __launch_bounds__(256) void f32_batches_kernel(const uint64_t* __restrict__ run_keys,
                                                          const int32_t* __restrict__ run_pairs,
                                                          const int32_t* __restrict__ run_first_pair,
                                                          const int32_t* __restrict__ run_first_batch, int64_t runs,
                                                          int num_rels, int emax, const uint64_t* __restrict__ pair_keys,
                                                          const int32_t* __restrict__ pair_edges,
                                                          const int32_t* __restrict__ pair_first,
                                                          int32_t* __restrict__ run_batches,
                                                          BatchF32* __restrict__ batches, uint32_t* __restrict__ pinfo) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= runs) return;
  const int np = run_pairs[i], fp = run_first_pair[i];
  const int rel = (int)(run_keys[i] % (uint64_t)num_rels);
  int nb = 0;
  for (int j = 0; j < np;) {
    const int pb = j;
    int ne = 0, most = 0;
    do {
      const int c = min(pair_edges[fp + j], emax);
      if (j > pb && (j - pb == kBatch || ne + c > emax)) break;
      if (FILL) {
        const uint32_t dl = (uint32_t)((pair_keys[fp + j] >> kSubBits) & (kTileRows - 1));
        pinfo[fp + j] = dl | ((uint32_t)c << 8) | ((uint32_t)ne << 16);
      }
      ne += c, most = max(most, c), ++j;
    } while (j < np);
    if (FILL) {
      BatchF32 b;
      b.pair_begin = fp + pb;
      b.edge_begin = pair_first[fp + pb];
      b.counts = (uint32_t)(j - pb) | ((uint32_t)ne << 8) | ((uint32_t)most << 16);
      b.rel = rel;
      batches[run_first_batch[i] + nb] = b;
    }
    ++nb;
  }
  if (!FILL) run_batches[i] = nb;
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
// the texture addresser sees whole lines per quad of lanes; the four load instructions of a batch
// cover its EMAX = 32 / KS edges in order.  Multiplying: lane (i = l % 16, q = l / 16) holds
// inputs 8q .. 8q+7 of pair i.  The weighted rows change layout through an EMAX x 32 KS tile of
// LDS per wavefront: written once per edge, read once per edge by the lanes of the edge's pair.
//
// The loads of the batch loop are unconditional -- indices are clamped to records that exist and
// what must not count is multiplied by zero afterwards -- so that the loop body is one basic
// block.  Offsets into X and the edge records are 32-bit byte offsets from scalar bases (the
// launch checks that they fit).
template <int KS, int NT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(KS == 1 && NT == 2 ? 3 : 1, 3)))
void rgms_f32_tile_kernel(int m, int fin, int fout, int total_batches,
                                                            const UnitF32* __restrict__ units,
                                                            const BatchF32* __restrict__ batches,
                                                            const uint32_t* __restrict__ pinfo,
                                                            const EdgeF32* __restrict__ edges,
                                                            const float4* __restrict__ Wp,
                                                            const float* __restrict__ X, float* __restrict__ Y,
                                                            float* partials, uint32_t* arrived) {
  constexpr int FO = 16 * NT;      // floats per row of a partial tile
  constexpr int CPR = 8 * KS;      // lanes (16-byte chunks) per gathered row
  constexpr int RPI = 64 / CPR;    // rows per load instruction
  constexpr int EMAX = 32 / KS;    // edges per batch
  constexpr int NLOAD = EMAX / RPI;
  constexpr int SS = 32 * KS + 4;  // floats per row of the edge tile: 16 lanes reading 32 bytes each hit 64 banks
  static_assert(NLOAD == 4, "four load instructions per batch");
  static_assert(NT == 2 || NT == 4, "a lane's outputs are one 8- or 16-byte word of the partial tile");
  __shared__ __attribute__((aligned(16))) float ytile[4][kTileRows * FO];
  __shared__ __attribute__((aligned(16))) float etile[4][(EMAX + 1) * SS];  // the last row stays zero
  __shared__ int last_of_tile;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i = lane & 15, q = lane >> 4;      // multiplying
  const int gr = lane / CPR, gc = lane % CPR;  // gathering
  const UnitF32 u = units[blockIdx.x];
  float* yt = ytile[wave];
  float* et = etile[wave];
  for (int e = lane; e < kTileRows * FO; e += 64) yt[e] = 0.f;
  for (int e = lane; e < (EMAX + 1) * SS; e += 64) et[e] = 0.f;

  const int b_end = u.batch_end;
  int b = u.batch_begin + wave;
  const bool chunk_live = 4 * gc < fin;  // fin is a multiple of 4: chunks are whole
  const uint32_t x_off = chunk_live ? 16u * gc : 0u;
  const uint32_t row_bytes = 4u * (uint32_t)fin;
  const char* Xb = reinterpret_cast<const char*>(X);
  const char* Eb = reinterpret_cast<const char*>(edges);

  struct Batch {  // the same in every lane
    uint32_t pair_begin, edge_off;  // edge_off in bytes
    int npairs, nedges, most, rel;
  };
  auto raw_batch = [&](int bi) { return batches[min(bi, total_batches - 1)]; };
  auto scalars = [&](const BatchF32& t, int bi) {  // a batch beyond the unit's last one: no pairs, no edges
    Batch r;
    const uint32_t c = bi < b_end ? __builtin_amdgcn_readfirstlane(t.counts) : 0u;
    r.pair_begin = __builtin_amdgcn_readfirstlane((uint32_t)t.pair_begin);
    r.edge_off = __builtin_amdgcn_readfirstlane((uint32_t)t.edge_begin) * 16u;
    r.npairs = (int)(c & 255u), r.nedges = (int)((c >> 8) & 255u), r.most = (int)((c >> 16) & 255u);
    r.rel = __builtin_amdgcn_readfirstlane(t.rel);
    return r;
  };
  struct EdgesG {  // gathering layout: load instruction k serves edge k * RPI + gr of the batch
    int32_t src[NLOAD];
    const float* w[NLOAD];
  };
  auto load_edges = [&](const Batch& bt) {  // beyond the batch's last edge: that one again
    EdgesG r;
#pragma unroll
    for (int k = 0; k < NLOAD; ++k) {
      const int e = k * RPI + gr;
      // (one 16-byte load; taken apart field by field it becomes two)
      const uint4 rec = *reinterpret_cast<const uint4*>(Eb + (bt.edge_off + 16u * (uint32_t)min(e, max(bt.nedges - 1, 0))));
      r.src[k] = (int32_t)rec.x;
      r.w[k] = reinterpret_cast<const float*>((uintptr_t)rec.z | ((uintptr_t)rec.w << 32));
    }
    return r;
  };
  struct RowsG {
    float w[NLOAD];
    float4 x[NLOAD];
  };
  auto load_rows = [&](const EdgesG& eg) {
    RowsG r;
#pragma unroll
    for (int k = 0; k < NLOAD; ++k) {
      r.w[k] = *reinterpret_cast<GlobalF32*>(reinterpret_cast<uintptr_t>(eg.w[k]));
      r.x[k] = *reinterpret_cast<const float4*>(Xb + ((uint32_t)eg.src[k] * row_bytes + x_off));
    }
    return r;
  };
  auto load_pair = [&](const Batch& bt) { return pinfo[bt.pair_begin + (i < bt.npairs ? (uint32_t)i : 0u)]; };

  auto load_w = [&](float4 (&wq)[NT][KS][2], int rel) {  // B operands of `rel`, in lane order
    const float4* wrel = Wp + (int64_t)rel * (NT * KS * 2 * 64) + lane;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int c = 0; c < 2; ++c) wq[nt][s][c] = wrel[((nt * KS + s) * 2 + c) * 64];
  };

  // The pipeline.  Everything a batch needs is requested two of the wavefront's batches ahead of
  // its use -- the record of batch j + 6 (so that its scalars exist at j + 4), the edge records of
  // j + 4 (so that the rows of X of j + 2 can be requested at j), the rows, pair words and W
  // operands of j + 2 -- into two sets of registers, one for the even and one for the odd batches:
  // a set's registers are reloaded right after their last use, nothing in flight is ever copied,
  // and the loop is unrolled by two.
  struct Stage {
    RowsG rw;              // rows of X and weights of batch j
    EdgesG eg;             // edge records of batch j + 2
    BatchF32 raw;          // record of batch j + 4
    uint32_t pw;           // pair word of batch j
    float4 wq[NT][KS][2];  // W operands of batch j
  };
  Batch bt0 = scalars(raw_batch(b), b), bt1 = scalars(raw_batch(b + 4), b + 4);
  Batch bt2 = scalars(raw_batch(b + 8), b + 8), bt3 = scalars(raw_batch(b + 12), b + 12);
  Stage even, odd;
  even.raw = raw_batch(b + 16), odd.raw = raw_batch(b + 20);
  even.eg = load_edges(bt2), odd.eg = load_edges(bt3);
  even.pw = load_pair(bt0), odd.pw = load_pair(bt1);
  load_w(even.wq, bt0.rel);
  load_w(odd.wq, bt1.rel);
  {
    const EdgesG eg0 = load_edges(bt0), eg1 = load_edges(bt1);
    even.rw = load_rows(eg0), odd.rw = load_rows(eg1);
  }

  auto batch = [&](Stage& st) {
    // 1. the weighted rows of this batch, into the edge tile.  Places behind the batch's last edge
    // get whatever was read: no pair reads them.  Chunks beyond feat_in are never written and stay
    // zero.
    if (chunk_live) {
#pragma unroll
      for (int k = 0; k < NLOAD; ++k) {
        const float w = st.rw.w[k];
        float4 v = st.rw.x[k];
        v.x *= w, v.y *= w, v.z *= w, v.w *= w;
        *reinterpret_cast<float4*>(et + (k * RPI + gr) * SS + 4 * gc) = v;
      }
    }
    // requests for the batches to come
    st.rw = load_rows(st.eg);
    const Batch bt4 = scalars(st.raw, b + 16);
    st.eg = load_edges(bt4);
    st.raw = raw_batch(b + 24);
    // 2. the sums of the pairs, multiplying layout: lane (i, q) walks the edges of pair i; a lane
    // whose pair has fewer edges than the batch's longest reads the tile's row of zeros meanwhile
    const uint32_t pw = st.pw;
    const int my_first = (int)((pw >> 16) & 255u), my_count = i < bt0.npairs ? (int)((pw >> 8) & 255u) : 0;
    const int my_dl = (int)(pw & (kTileRows - 1));
    float4 sq[KS][2];
    {  // every pair has a first edge; a lane without a pair takes the row of zeros
      const float* row = et + (my_count > 0 ? my_first : EMAX) * SS + 8 * q;
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int c = 0; c < 2; ++c) sq[s][c] = *reinterpret_cast<const float4*>(row + 32 * s + 4 * c);
    }
    for (int t = 1; t < bt0.most; ++t) {  // the same for every lane
      const float* row = et + (t < my_count ? my_first + t : EMAX) * SS + 8 * q;
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          const float4 v = *reinterpret_cast<const float4*>(row + 32 * s + 4 * c);
          sq[s][c].x += v.x, sq[s][c].y += v.y, sq[s][c].z += v.z, sq[s][c].w += v.w;
        }
    }
    // 3. times W[rel]^T
    f32x4 acc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const float4 wk = st.wq[nt][s][c], sk = sq[s][c];
          acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(sk.x, wk.x, acc[nt], 0, 0, 0);
          acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(sk.y, wk.y, acc[nt], 0, 0, 0);
          acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(sk.z, wk.z, acc[nt], 0, 0, 0);
          acc[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(sk.w, wk.w, acc[nt], 0, 0, 0);
        }
    load_w(st.wq, bt2.rel);
    // 4. acc[nt][v]: pair 4 q + v of the batch, output 16 nt + i, which lives at float NT i + nt of
    // its row of the partial tile: a lane's NT outputs are neighbours, one read and one write.
    // The pairs of a batch end in different rows (a row cut into pieces has at most its last,
    // shorter piece in a batch with other pairs: a full piece fills a batch), so no two lanes
    // update the same float.
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int dl = __shfl(my_dl, 4 * q + v, 64);
      if (4 * q + v < bt0.npairs) {
        float* at = yt + dl * FO + NT * i;
        if constexpr (NT == 2) {
          float2 o = *reinterpret_cast<float2*>(at);
          o.x += acc[0][v], o.y += acc[1][v];
          *reinterpret_cast<float2*>(at) = o;
        } else {
          float4 o = *reinterpret_cast<float4*>(at);
          o.x += acc[0][v], o.y += acc[1][v], o.z += acc[2][v], o.w += acc[3][v];
          *reinterpret_cast<float4*>(at) = o;
        }
      }
    }
    st.pw = load_pair(bt2);  // last: the old word's row number was in use until here
    b += 4;
    bt0 = bt1, bt1 = bt2, bt2 = bt3, bt3 = bt4;  // scalars: copies wait for nothing
  };
  // (With the way out between the two halves, the compiler's wait counts at the top of a round are
  // "everything requested in the round before has arrived".  Without it -- both batches run
  // whether the second exists or not, and the requests of the prologue waited for once before the
  // loop -- the counts leave two batches' worth of loads in flight, and the launch is slower: 139
  // against 130 us on 100k nodes / 65 relations / 2M edges.  The loop is bound by instruction
  // issue, not by the latency of its loads.)
  while (bt0.npairs > 0) {  // the same for every lane
    batch(even);
    if (bt0.npairs == 0) break;
    batch(odd);
  }

  __syncthreads();
  const int64_t row0 = (int64_t)u.tile * kTileRows;
  const int64_t stride = (int64_t)kTileRows * fout;
  for (int e = tid; e < kTileRows * fout; e += 256) {
    const int r = e / fout, c = e - r * fout;
    if (row0 + r >= m) break;
    const int at = r * FO + NT * (c & 15) + (c >> 4);
    const float sum = (ytile[0][at] + ytile[1][at]) + (ytile[2][at] + ytile[3][at]);
    if (u.partial < 0)
      Y[(row0 + r) * fout + c] += sum;
    else
      __hip_atomic_store(partials + u.partial * stride + e, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (u.partial < 0) return;
  // A piece of a tile.  Every wavefront waits until its stores have arrived, then one thread
  // counts the unit in; the unit that counts last finds the partial tiles of all the others in
  // memory (stores and loads of partial tiles pass the L2 of their XCD).
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0) {
    uint32_t* counter = arrived + u.cut_tile;
    const uint32_t before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool last = before + 1 == (uint32_t)u.pieces;
    if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    last_of_tile = last;
  }
  __syncthreads();
  if (!last_of_tile) return;
  for (int e = tid; e < kTileRows * fout; e += 256) {
    if (row0 + e / fout >= m) break;
    float sum = 0.f;
    for (int p = 0; p < u.pieces; ++p)
      sum += __hip_atomic_load(partials + (u.first_partial + p) * stride + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    Y[row0 * fout + e] += sum;
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
int build_index(F32TileIndex& idx, const F32Source& src, int32_t m, int32_t n, int32_t num_rels, int32_t emax,
                hipStream_t stream);
}

bool f32_tiles_serves(int32_t feat_in, int32_t feat_out) {
  return feat_in > 0 && feat_in % 4 == 0 && feat_in <= 64 && feat_out > 0 && feat_out <= 64;
}

bool f32_tiles_fits(int32_t n, int32_t feat_in, int64_t edges) {
  return (int64_t)n * feat_in * 4 < (int64_t(1) << 32) && edges * 16 < (int64_t(1) << 32);
}

void f32_tiles_free(F32TileIndex& idx) {
  if (idx.d_edges) (void)hipFree(idx.d_edges);
  if (idx.d_pairs) (void)hipFree(idx.d_pairs);
  if (idx.d_batches) (void)hipFree(idx.d_batches);
  if (idx.d_units) (void)hipFree(idx.d_units);
  if (idx.d_arrived) (void)hipFree(idx.d_arrived);
  if (idx.d_partials) (void)hipFree(idx.d_partials);
  if (idx.d_wpack) (void)hipFree(idx.d_wpack);
  idx = F32TileIndex();
}

int f32_tiles_prepare(F32TileIndex& idx, const F32Source& src, int32_t m, int32_t n, int32_t num_rels,
                      int32_t feat_in, hipStream_t stream) {
  const int32_t emax = feat_in <= 32 ? 32 : 16;
  if (idx.m == m && idx.n == n && idx.num_rels == num_rels && idx.emax == emax) return 0;
  f32_tiles_free(idx);
  F32TileIndex built;
  const int rc = build_index(built, src, m, n, num_rels, emax, stream);
  if (rc != 0) {
    f32_tiles_free(built);  // nothing half-made stays behind
    return rc;
  }
  idx = built;
  return 0;
}

namespace {
int build_index(F32TileIndex& idx, const F32Source& src, int32_t m, int32_t n, int32_t num_rels, int32_t emax,
                hipStream_t stream) {
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
  STIR_REQUIRE(tiles < (int64_t(1) << 31), "rgms_f32: too many tiles");
  int key_bits = kTileShift;
  while (key_bits < 64 && ((uint64_t)tiles * num_rels) >> (key_bits - kTileShift)) ++key_bits;
  STIR_REQUIRE(key_bits + kSubBits <= 64, "rgms_f32: sort keys exceed 64 bits");
  idx.m = m, idx.n = n, idx.num_rels = num_rels, idx.emax = emax;
  idx.edges = slots, idx.tiles = tiles;
  if (slots == 0) return 0;  // no units: the launch returns at once
  Scratch tmp;
  DevBucketF32* d_tab = nullptr;
  if (!tab.empty()) {
    if (tmp.get(&d_tab, tab.size())) return -1;
    STIR_HIP(hipMemcpyAsync(d_tab, tab.data(), sizeof(DevBucketF32) * tab.size(), hipMemcpyHostToDevice, stream));
  }
  const CsfArrays csf = {src.A, src.indptr_i, src.indices_i, src.indptr_j, src.indices_j, src.nnz_i};
  uint64_t *keys_in = nullptr, *keys_out = nullptr, *unique = nullptr;
  int32_t *vals_in = nullptr, *vals_out = nullptr, *counts = nullptr, *first = nullptr, *flags = nullptr;
  int64_t* tile_begin = nullptr;
  if (tmp.get(&keys_in, slots) || tmp.get(&keys_out, slots) || tmp.get(&unique, slots) || tmp.get(&vals_in, slots) ||
      tmp.get(&vals_out, slots) || tmp.get(&counts, slots) || tmp.get(&first, slots) || tmp.get(&flags, 2) ||
      tmp.get(&tile_begin, tiles + 1))
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
  size_t sort_bytes = 0, rle_bytes = 0, scan_bytes = 0;
  STIR_HIP(hipcub::DeviceRadixSort::SortPairs(nullptr, sort_bytes, keys_in, keys_out, vals_in, vals_out, (int)slots, 0,
                                              key_bits, stream));
  STIR_HIP(hipcub::DeviceRunLengthEncode::Encode(nullptr, rle_bytes, keys_out, unique, counts, flags + 1, (int)slots,
                                                 stream));
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(nullptr, scan_bytes, counts, first, (int)slots + 1, stream));
  char* cub_tmp = nullptr;
  const size_t cub_bytes = std::max(sort_bytes, std::max(rle_bytes, scan_bytes));
  if (tmp.get(&cub_tmp, cub_bytes)) return -1;
  size_t bytes = sort_bytes;
  STIR_HIP(hipcub::DeviceRadixSort::SortPairs(cub_tmp, bytes, keys_in, keys_out, vals_in, vals_out, (int)slots, 0,
                                              key_bits, stream));
  STIR_HIP(hipMalloc(&idx.d_edges, sizeof(EdgeF32) * (size_t)slots));
  if (src.csf)
    hipLaunchKernelGGL(f32_edge_records_kernel<true>, grid, block, 0, stream, d_tab, nb, csf, slots, num_rels, vals_out,
                       static_cast<EdgeF32*>(idx.d_edges));
  else
    hipLaunchKernelGGL(f32_edge_records_kernel<false>, grid, block, 0, stream, d_tab, nb, csf, slots, num_rels,
                       vals_out, static_cast<EdgeF32*>(idx.d_edges));
  STIR_LAUNCH_CHECK();
  // runs of equal key, cut into pieces of at most emax edges by a second key
  bytes = rle_bytes;
  STIR_HIP(hipcub::DeviceRunLengthEncode::Encode(cub_tmp, bytes, keys_out, unique, counts, flags + 1, (int)slots,
                                                 stream));
  int32_t host_flags[2] = {0, 0};
  STIR_HIP(hipMemcpyAsync(host_flags, flags, sizeof(host_flags), hipMemcpyDeviceToHost, stream));
  STIR_HIP(hipStreamSynchronize(stream));
  if (host_flags[0] != 0)
    return fail(host_flags[0] == 1 ? "rgms_f32: a row id or relation id lies outside [0, m) / [0, num_rels)"
                                   : "rgms_f32: a column id lies outside [0, n)");
  const int64_t key_runs = host_flags[1];
  bytes = scan_bytes;
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(cub_tmp, bytes, counts, first, (int)key_runs, stream));
  hipLaunchKernelGGL(f32_subkeys_kernel, grid, block, 0, stream, keys_out, first, key_runs, slots, (int)emax, keys_in,
                     flags);
  STIR_LAUNCH_CHECK();
  bytes = rle_bytes;
  STIR_HIP(hipcub::DeviceRunLengthEncode::Encode(cub_tmp, bytes, keys_in, unique, counts, flags + 1, (int)slots,
                                                 stream));
  STIR_HIP(hipMemcpyAsync(host_flags, flags, sizeof(host_flags), hipMemcpyDeviceToHost, stream));
  STIR_HIP(hipStreamSynchronize(stream));
  STIR_REQUIRE(host_flags[0] == 0, "rgms_f32: a (relation, row) pair has too many edges for the tiled kernel");
  const int64_t pairs = host_flags[1];
  idx.pairs = pairs;
  bytes = scan_bytes;
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(cub_tmp, bytes, counts, first, (int)pairs, stream));
  // the (tile, relation) runs of pairs.  keys_out / vals_in / vals_out are free again; keys_in is
  // once the run-length encoding above has read it (same stream)
  uint64_t* run_of_pair = keys_out;
  uint64_t* run_keys = keys_in;
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
  STIR_REQUIRE(std::max(rle2, scan2) <= cub_bytes, "rgms_f32: scratch of the index build is too small");
  bytes = rle2;
  STIR_HIP(hipcub::DeviceRunLengthEncode::Encode(cub_tmp, bytes, run_of_pair, run_keys, run_pairs, flags + 1, (int)pairs,
                                                 stream));
  STIR_HIP(hipMemcpyAsync(host_flags, flags, sizeof(host_flags), hipMemcpyDeviceToHost, stream));
  STIR_HIP(hipStreamSynchronize(stream));
  const int64_t runs = host_flags[1];
  bytes = scan2;
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(cub_tmp, bytes, run_pairs, run_first_pair, (int)runs, stream));
  const dim3 run_grid((unsigned)ceil_div(runs, 256));
  hipLaunchKernelGGL(f32_batches_kernel<false>, run_grid, block, 0, stream, run_keys, run_pairs, run_first_pair,
                     (const int32_t*)nullptr, runs, num_rels, (int)emax, unique, counts, first, run_batches,
                     (BatchF32*)nullptr, (uint32_t*)nullptr);
  STIR_LAUNCH_CHECK();
  // one entry more than runs: the last one is the batch count (run_batches[runs] is not read as an addend)
  STIR_HIP(hipMemsetAsync(run_batches + runs, 0, sizeof(int32_t), stream));
  bytes = scan2;
  STIR_HIP(hipcub::DeviceScan::ExclusiveSum(cub_tmp, bytes, run_batches, run_first_batch, (int)runs + 1, stream));
  int32_t total_batches = 0;
  STIR_HIP(hipMemcpyAsync(&total_batches, run_first_batch + runs, sizeof(int32_t), hipMemcpyDeviceToHost, stream));
  STIR_HIP(hipStreamSynchronize(stream));
  idx.batches = total_batches;
  STIR_HIP(hipMalloc(&idx.d_batches, sizeof(BatchF32) * (size_t)std::max<int64_t>(total_batches, 1)));
  STIR_HIP(hipMalloc(&idx.d_pairs, sizeof(uint32_t) * (size_t)std::max<int64_t>(pairs, 1)));
  hipLaunchKernelGGL(f32_batches_kernel<true>, run_grid, block, 0, stream, run_keys, run_pairs, run_first_pair,
                     run_first_batch, runs, num_rels, (int)emax, unique, counts, first, (int32_t*)nullptr,
                     static_cast<BatchF32*>(idx.d_batches), static_cast<uint32_t*>(idx.d_pairs));
  STIR_LAUNCH_CHECK();
  hipLaunchKernelGGL(f32_tile_batches_kernel, dim3((unsigned)ceil_div(tiles + 1, 256)), block, 0, stream, run_keys,
                     run_first_batch, runs, (int64_t)total_batches, tiles, num_rels, tile_begin);
  STIR_LAUNCH_CHECK();
  // units: a tile, or -- for a tile with more than 1.5 times `cap` batches -- pieces of at most
  // `cap` batches, cap = twice the average of the tiles that have batches (at least 32)
  std::vector<int64_t> tb((size_t)tiles + 1);
  STIR_HIP(hipMemcpyAsync(tb.data(), tile_begin, sizeof(int64_t) * tb.size(), hipMemcpyDeviceToHost, stream));
  STIR_HIP(hipStreamSynchronize(stream));  // also: the scratch arrays go away
  int64_t busy = 0;
  for (int64_t t = 0; t < tiles; ++t) busy += tb[(size_t)t + 1] > tb[(size_t)t];
  const int64_t cap = std::max<int64_t>(32, busy ? 2 * ceil_div((int64_t)total_batches, busy) : 32);
  std::vector<UnitF32> units;
  int64_t partial_tiles = 0, cut_tiles = 0;
  for (int64_t t = 0; t < tiles; ++t) {
    const int64_t lo = tb[(size_t)t], hi = tb[(size_t)t + 1];
    if (hi <= lo) continue;
    if (2 * (hi - lo) <= 3 * cap) {
      units.push_back(UnitF32{(int32_t)t, (int32_t)lo, (int32_t)hi, -1, 0, 0, 0, 0});
      continue;
    }
    const int64_t pieces = ceil_div(hi - lo, cap), len = ceil_div(hi - lo, pieces);
    STIR_REQUIRE(partial_tiles + pieces < (int64_t(1) << 31), "rgms_f32: too many partial tiles");
    for (int64_t p = 0; p < pieces; ++p)
      units.push_back(UnitF32{(int32_t)t, (int32_t)(lo + p * len), (int32_t)std::min(hi, lo + (p + 1) * len),
                              (int32_t)(partial_tiles + p), (int32_t)partial_tiles, (int32_t)pieces,
                              (int32_t)cut_tiles, 0});
    partial_tiles += pieces, ++cut_tiles;
  }
  // the longest units first
  std::stable_sort(units.begin(), units.end(), [](const UnitF32& a, const UnitF32& b) {
    return a.batch_end - a.batch_begin > b.batch_end - b.batch_begin;
  });
  // A few units beyond whole rounds of resident workgroups (three per CU) would run when the
  // others are done, each as slowly as a unit alone: those are cut into four pieces that run side
  // by side (100k nodes, 65 relations, 2M edges: 1563 units on 768 resident workgroups, 27 beyond
  // two rounds; 133 -> 127 us).  Only when they are few and of ordinary length.
  {
    int dev = 0, cus = 0;
    STIR_HIP(hipGetDevice(&dev));
    STIR_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int64_t resident = 3 * (int64_t)cus, count = (int64_t)units.size();
    const int64_t beyond = resident > 0 ? count % resident : 0;
    constexpr int64_t kPieces = 4;  // 3 to 4 measured best; 6 and 8 give the gain back
    if (count > resident && beyond > 0 && 8 * beyond <= resident) {
      const int64_t ordinary = total_batches / (2 * count);  // half the average length
      std::vector<UnitF32> cut;
      int64_t kept = 0;
      for (int64_t k = count - beyond; k < count; ++k) {
        const UnitF32 whole = units[(size_t)k];
        const int64_t lo = whole.batch_begin, hi = whole.batch_end;
        if (whole.partial >= 0 || hi - lo < std::max<int64_t>(ordinary, 2 * kPieces) ||
            partial_tiles + kPieces >= (int64_t(1) << 31)) {
          units[(size_t)(count - beyond + kept++)] = whole;
          continue;
        }
        const int64_t len = ceil_div(hi - lo, kPieces);
        for (int64_t p = 0; p < kPieces; ++p)
          cut.push_back(UnitF32{whole.tile, (int32_t)(lo + p * len), (int32_t)std::min(hi, lo + (p + 1) * len),
                                (int32_t)(partial_tiles + p), (int32_t)partial_tiles, (int32_t)kPieces,
                                (int32_t)cut_tiles, 0});
        partial_tiles += kPieces, ++cut_tiles;
      }
      units.resize((size_t)(count - beyond + kept));
      units.insert(units.end(), cut.begin(), cut.end());
    }
  }
  idx.units = (int64_t)units.size(), idx.multi = cut_tiles, idx.partial_tiles = partial_tiles;
  STIR_HIP(hipMalloc(&idx.d_units, sizeof(UnitF32) * std::max<size_t>(units.size(), 1)));
  STIR_HIP(hipMemcpy(idx.d_units, units.data(), sizeof(UnitF32) * units.size(), hipMemcpyHostToDevice));
  if (cut_tiles > 0) {  // the counters of the cut tiles: zero between launches
    STIR_HIP(hipMalloc(&idx.d_arrived, sizeof(uint32_t) * (size_t)cut_tiles));
    STIR_HIP(hipMemsetAsync(idx.d_arrived, 0, sizeof(uint32_t) * (size_t)cut_tiles, stream));
    STIR_HIP(hipStreamSynchronize(stream));  // done before a launch on any stream
  }
  return 0;
}
}  // namespace

int f32_tiles_launch(F32TileIndex& idx, int32_t feat_in, int32_t feat_out, const float* d_W, const float* d_X,
                     float* d_Y, hipStream_t stream) {
  STIR_REQUIRE(f32_tiles_serves(feat_in, feat_out), "rgms_f32: feature sizes %d -> %d are not served by the tiled kernel",
               feat_in, feat_out);
  STIR_REQUIRE(idx.emax == (feat_in <= 32 ? 32 : 16), "rgms_f32: the edge index was built for another feat_in");
  if (idx.units == 0) return 0;
  STIR_REQUIRE(idx.units < (int64_t(1) << 31), "rgms_f32: too many units for one launch");
  // the kernel's 32-bit byte offsets
  STIR_REQUIRE(f32_tiles_fits(idx.n, feat_in, idx.edges),
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
  const size_t partial_need = sizeof(float) * (size_t)idx.partial_tiles * kTileRows * (size_t)feat_out;
  if (partial_need > idx.partial_bytes) {
    if (idx.d_partials) STIR_HIP(hipFree(idx.d_partials));
    idx.d_partials = nullptr, idx.partial_bytes = 0;
    STIR_HIP(hipMalloc(&idx.d_partials, partial_need));
    idx.partial_bytes = partial_need;
  }
  float4* wp = static_cast<float4*>(idx.d_wpack);
  hipLaunchKernelGGL(f32_pack_w_kernel, dim3((unsigned)ceil_div(words, 256)), dim3(256), 0, stream, d_W, wp, words, nt, ks,
                     feat_in, feat_out);
  STIR_LAUNCH_CHECK();
  const dim3 grid((unsigned)idx.units), block(256);  // longest units first: they go to whichever slot is free
  const UnitF32* units = static_cast<const UnitF32*>(idx.d_units);
  const BatchF32* bts = static_cast<const BatchF32*>(idx.d_batches);
  const uint32_t* pinfo = static_cast<const uint32_t*>(idx.d_pairs);
  const EdgeF32* edges = static_cast<const EdgeF32*>(idx.d_edges);
  float* partials = static_cast<float*>(idx.d_partials);
#define STIR_F32_TILE(KS, NT)                                                                                   \
  hipLaunchKernelGGL((rgms_f32_tile_kernel<KS, NT>), grid, block, 0, stream, idx.m, feat_in, feat_out,          \
                     (int)idx.batches, units, bts, pinfo, edges, wp, d_X, d_Y, partials,                        \
                     static_cast<uint32_t*>(idx.d_arrived))
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
