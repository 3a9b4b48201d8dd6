// Destination-tiled fp32 RGMS: every 64-row tile of Y is summed on chip and written once, without
// atomics.  Serves both fp32 front ends (ELL3D buckets and the CSF arrays).
//
// The edges (slots) of the operator are re-indexed once per plan, sorted by (destination tile of
// 64 rows, relation, destination row); runs of equal key are the (relation, row) pairs, whose
// weighted sums of X rows meet the relation's W on the matrix cores 16 pairs at a time
// (v_mfma_f32_16x16x4_f32), and the products are added into a partial tile in LDS.  Tiles with
// many more edges than the average are cut into pieces, and so are the few tiles beyond whole
// rounds of resident workgroups; the piece of a tile that finishes last adds the pieces' partial
// tiles in a fixed order: the result does not depend on the order in which wavefronts run.
#pragma once
#include <cstdint>
#include <vector>

#include "common.h"

namespace stir {

struct F32Bucket {
  const float* A;       // device: slot weights, groups*rb*cb
  const int32_t* rows;  // device: groups*rb
  const int32_t* cols;  // device: groups*rb*cb
  const int32_t* mids;  // device: groups
  int64_t groups;
  int32_t rb, cb;
};

// Where the edges come from: ELL3D buckets, or (csf) the four CSF arrays and their edge values.
struct F32Source {
  bool csf = false;
  std::vector<F32Bucket> buckets;
  const float* A = nullptr;
  const int32_t* indptr_i = nullptr;
  const int32_t* indices_i = nullptr;
  const int32_t* indptr_j = nullptr;
  const int32_t* indices_j = nullptr;
  int64_t nnz_i = 0, nnz_j = 0;
};

struct F32TileIndex {
  int32_t m = -1, n = -1, num_rels = -1, emax = 0;  // what the index was built for (emax: edges per batch)
  int64_t edges = 0, pairs = 0, batches = 0, tiles = 0;
  int64_t units = 0, multi = 0, partial_tiles = 0;
  void* d_edges = nullptr;     // edges x 16 bytes, sorted
  void* d_pairs = nullptr;     // pairs x 4 bytes, sorted: row in tile | edges << 8 | first edge in its batch << 16
  void* d_batches = nullptr;   // batches x 16 bytes: up to 16 pairs and emax edges of one (tile, relation) each
  void* d_units = nullptr;     // units x 32 bytes: a tile or a piece of one, as a range of batches; longest first
  void* d_arrived = nullptr;   // a counter per tile cut into several units (`multi` of them), zero between launches
  void* d_partials = nullptr;  // their partial tiles, rewritten by every launch
  size_t partial_bytes = 0;
  void* d_wpack = nullptr;     // W in the multiply's operand order, rewritten by every launch
  size_t wpack_bytes = 0;
};

// True when the kernel serves these feature sizes (else the caller keeps its other kernel).
bool f32_tiles_serves(int32_t feat_in, int32_t feat_out);
// ... and these sizes: the kernel addresses X and its edge records with 32-bit byte offsets.
bool f32_tiles_fits(int32_t n, int32_t feat_in, int64_t edges);
// Builds the index on `stream` (synchronises; allocates).  A no-op when it exists for the same m,
// n, num_rels and batch size (feat_in up to 32, or above).  Fails when a row id, column id or
// relation id is out of range.
int f32_tiles_prepare(F32TileIndex& idx, const F32Source& src, int32_t m, int32_t n, int32_t num_rels,
                      int32_t feat_in, hipStream_t stream);
// Y += RGMS(W, X) over the indexed edges.  W: [R, feat_out, feat_in], X: [n, feat_in], fp32.
int f32_tiles_launch(F32TileIndex& idx, int32_t feat_in, int32_t feat_out, const float* d_W, const float* d_X,
                     float* d_Y, hipStream_t stream);
void f32_tiles_free(F32TileIndex& idx);

}  // namespace stir
