// Destination-tiled RGMS for ELL3D inputs that are not tiny: every 32-row tile of Y is summed in
// registers and written once, without atomics.
//
// The slots of all buckets are re-indexed once per plan as "edges" (source row, relation,
// destination row, address of the slot weight) sorted by (destination tile of 32 rows, relation,
// row inside the tile).  A workgroup owns a tile: its four wavefronts walk the tile's edges 32 at
// a time, each with a 32 x 32 fp32 block of partial sums in MFMA accumulators; the blocks are added
// through LDS and the tile's rows of Y are written once.  Tiles with very many edges are cut into
// several units whose results are added with atomics.
#pragma once
#include <cstdint>
#include <vector>

#include "common.h"

namespace stir {

struct TileBucket {
  const uint16_t* A;    // device: slot weights (16-bit), groups*rb*cb
  const int32_t* rows;  // device: groups*rb
  const int32_t* cols;  // device: groups*rb*cb
  const int32_t* mids;  // device: groups
  int64_t groups;
  int32_t rb, cb;
};

struct TileIndex {
  int32_t m = -1, n = -1, num_rels = -1;  // what the index was built for; num_rels counts from rel_lo
  int32_t rel_lo = 0;                     // first relation of the index
  bool packed_records = false;            // 8-byte records that carry the slot weights (see tile_set_prepare)
  int64_t edges = 0;                      // slots of all buckets
  int64_t units = 0;
  void* d_edges = nullptr;  // edges x 16 (or 8) bytes, sorted
  void* d_units = nullptr;  // units x 16 bytes
  void* d_wpack = nullptr;  // W in MFMA operand order, rewritten by every launch
  size_t wpack_bytes = 0;
  // For the launch whose workgroups stay resident (W in LDS): the sorted edges cut into equal
  // shares of steps, one per team of wavefronts, each share a list of units.  Built at the first
  // such launch and again when the number of teams changes.
  std::vector<int64_t> tile_begin;  // host copy: first sorted edge of every tile, then the edge count
  int64_t share_teams = 0;
  void* d_share_ptr = nullptr;    // share_teams + 1 offsets into d_share_units
  void* d_share_units = nullptr;  // units x 16 bytes, grouped by team
};

// The indices of a plan: one for all relations, or -- when W does not fit the LDS of a compute unit
// and a few ranges of relations do -- one per range, launched one after the other.
struct TileIndexSet {
  int32_t m = -1, n = -1, num_rels = -1, rels_per_part = 0;  // what the set was built for
  std::vector<TileIndex> parts;                               // part p: relations from p * rels_per_part
};

// Builds the indices on `stream` (synchronises; allocates).  A no-op when they already exist for
// the same m, n and num_rels and the feature sizes lead to the same ranges of relations.  Fails
// when a row id, column id or relation id is out of range.
// static_weights: the caller promises that the slot weights keep the values they have now.  Slots
// of weight zero (the padding of ELL3D) are then left out of the index and a record shrinks to
// 8 bytes holding the weight itself (source row; weight << 16 | relation << 5 | row in tile), for
// up to 2048 relations per index; otherwise records hold the weight's address and weights are
// read at every launch.
int tile_set_prepare(TileIndexSet& set, const std::vector<TileBucket>& buckets, int32_t m, int32_t n,
                     int32_t num_rels, int32_t feat_in, int32_t feat_out, bool static_weights, hipStream_t stream);
// Y += RGMS(W, X) over the indexed edges.  W: [R, feat_in, feat_out], X: [n, feat_in], 16-bit.
// Y: [m, feat_out] fp32, or fp16 with out16 (fp16 inputs only; 4-byte aligned).
int tile_set_launch(bool bf16, bool out16, TileIndexSet& set, int32_t feat_in, int32_t feat_out, const void* d_W,
                    const void* d_X, void* d_Y, hipStream_t stream);
void tile_set_free(TileIndexSet& set);

}  // namespace stir
