// Scatter-free accumulation for RGMS: instead of adding every ELL row's result to Y with fp32
// atomics (whose rate is bounded by the L2 atomic units, about one 4-byte operation per channel
// and clock), the kernel writes the results to a staging matrix Z (one row per ELL row, plain
// stores) and a second kernel adds up, for every destination row, the Z rows that belong to it.
// The list of Z rows sorted (stably) by output row depends only on the format's row arrays and is
// made once per plan.
#pragma once
#include <cstdint>
#include <vector>

#include "common.h"

namespace stir {

struct DestBucket {
  const int32_t* rows;  // device: output row of each ELL row of the bucket
  int64_t ell_rows;
  int64_t row_begin;    // first Z row of the bucket
};

struct DestIndex {
  int32_t m = -1;             // number of output rows the index was built for
  int64_t z_rows = 0;         // Z rows (sum of ell_rows)
  int32_t* d_keys = nullptr;  // z_rows: output row of every list entry, ascending
  int32_t* d_list = nullptr;  // z_rows: Z rows (= ELL rows) in the stable order of their output rows
  float* d_Z = nullptr;
  int64_t z_floats = 0;       // allocated size of Z
};

// Builds (or rebuilds, when m changed) the index on `stream` and makes Z at least z_rows * feat_out
// floats.  Allocates; meant for the first call on a plan.
int dest_index_prepare(DestIndex& ix, const std::vector<DestBucket>& buckets, int32_t m, int32_t feat_out,
                       hipStream_t stream);
// Y[i, :] += sum of the Z rows of output row i.
int dest_reduce(const DestIndex& ix, int32_t feat_out, float* d_Y, hipStream_t stream);
void dest_index_free(DestIndex& ix);

}  // namespace stir
