// Host side of the format-decomposition pass: ColumnPartHyb, CSFToELL3D, ConDense.
//
// The reference builds its outputs by appending to growing vectors and counts a row's
// per-partition degree with a multiset lookup per nonzero (src/sparse/format.cc:62-72,91),
// which is quadratic in the degree of a row.  Here each routine runs as a counting pass
// followed by a placement pass into caller-allocated arrays, linear in the number of
// nonzeros, and produces the same arrays bit for bit.
#include <algorithm>
#include <cstring>
#include <vector>

#include "common.h"
#include "../../include/sparsetir_amd.h"

namespace {

// First bucket whose width is >= deg, or the last bucket (format.cc:92-96).
inline int bucket_of(const int32_t* widths, int nb, int deg) {
  int k = int(std::upper_bound(widths, widths + nb, deg - 1) - widths);
  return k == nb ? nb - 1 : k;
}

int check_csr(const char* who, int32_t num_rows, const int32_t* indptr) {
  STIR_REQUIRE(num_rows >= 0, "%s: num_rows=%d", who, num_rows);
  STIR_REQUIRE(indptr != nullptr, "%s: indptr is null", who);
  STIR_REQUIRE(indptr[0] >= 0, "%s: indptr[0]=%d is negative", who, indptr[0]);
  for (int32_t i = 0; i < num_rows; ++i)
    STIR_REQUIRE(indptr[i] <= indptr[i + 1], "%s: indptr decreases at row %d", who, i);
  return 0;
}

int check_buckets(const char* who, const int32_t* widths, int nb) {
  STIR_REQUIRE(nb > 0 && widths != nullptr, "%s: empty bucket list", who);
  for (int b = 0; b < nb; ++b) STIR_REQUIRE(widths[b] > 0, "%s: bucket width %d is not positive", who, widths[b]);
  for (int b = 1; b < nb; ++b)
    STIR_REQUIRE(widths[b - 1] <= widths[b], "%s: bucket widths must ascend", who);
  return 0;
}

template <bool kFill>
int column_part_hyb_pass(int32_t num_rows, int32_t num_cols, const int32_t* indptr,
                         const int32_t* indices, int32_t parts, const int32_t* widths, int32_t nb,
                         int64_t* nrows, int32_t* const* rows_out, int32_t* const* cols_out,
                         int32_t* const* mask_out) {
  const char* who = "ColumnPartHyb";
  if (check_csr(who, num_rows, indptr) || check_buckets(who, widths, nb)) return -1;
  STIR_REQUIRE(num_cols > 0 || indptr[num_rows] == indptr[0], "%s: num_cols=%d", who, num_cols);
  STIR_REQUIRE(parts > 0, "%s: num_col_parts=%d", who, parts);
  const int32_t psize = num_cols > 0 ? (num_cols + parts - 1) / parts : 1;
  std::vector<int64_t> emitted(size_t(parts) * nb, 0);  // ELL rows so far per (part, bucket)
  std::vector<int32_t> deg(parts, 0), seen(parts, 0), which(parts, 0), touched;
  std::vector<int64_t> base(parts, 0);
  touched.reserve(parts);
  for (int32_t i = 0; i < num_rows; ++i) {
    const int32_t lo = indptr[i], hi = indptr[i + 1];
    touched.clear();
    for (int32_t p = lo; p < hi; ++p) {
      const int32_t col = indices[p];
      STIR_REQUIRE(col >= 0 && col < num_cols, "%s: column %d of row %d outside [0, %d)", who, col, i, num_cols);
      const int32_t part = col / psize;
      if (deg[part]++ == 0) touched.push_back(part);
    }
    for (int32_t part : touched) {
      const int d = deg[part];
      const int b = bucket_of(widths, nb, d);
      const int w = widths[b];
      const int64_t ell_rows = (d + w - 1) / w;
      const size_t k = size_t(part) * nb + b;
      base[part] = emitted[k];
      which[part] = b;
      emitted[k] += ell_rows;
      if (kFill) {
        for (int64_t j = 0; j < ell_rows; ++j) rows_out[k][base[part] + j] = i;
        for (int64_t s = base[part] * w + d; s < (base[part] + ell_rows) * w; ++s) {
          cols_out[k][s] = 0;
          mask_out[k][s] = 0;
        }
      }
    }
    if (kFill) {
      for (int32_t p = lo; p < hi; ++p) {
        const int32_t col = indices[p];
        const int32_t part = col / psize;
        const int b = which[part];
        const size_t k = size_t(part) * nb + b;
        const int64_t pos = base[part] * widths[b] + seen[part]++;
        cols_out[k][pos] = col;
        mask_out[k][pos] = 1;
      }
    }
    for (int32_t part : touched) {
      deg[part] = 0;
      seen[part] = 0;
    }
  }
  if (!kFill) std::copy(emitted.begin(), emitted.end(), nrows);
  return 0;
}

// Streams the (row, col) entries of one relation through the ELL rows of its bucket the way
// the reference's append loop does (format.cc:239-273): an ELL row ends when it is full or
// the row id changes.  Calls emit(bucket, ell_row_in_relation, slot, row, col).
template <typename Emit>
void stream_relation(int r, const int32_t* indptr0, const int32_t* indices0,
                     const int32_t* indptr1, const int32_t* indices1, const int32_t* cols_bkt,
                     int nb, std::vector<int64_t>& ell_rows, Emit emit) {
  std::vector<int32_t> fill(nb, 0), last_row(nb, -1);
  std::fill(ell_rows.begin(), ell_rows.end(), 0);
  for (int32_t i = indptr0[r]; i < indptr0[r + 1]; ++i) {
    const int32_t row = indices0[i];
    const int cnt = indptr1[i + 1] - indptr1[i];
    const int b = bucket_of(cols_bkt, nb, cnt);
    const int cb = cols_bkt[b];
    for (int32_t j = indptr1[i]; j < indptr1[i + 1]; ++j) {
      if (fill[b] == 0 || fill[b] == cb || last_row[b] != row) {
        ++ell_rows[b];
        fill[b] = 0;
        last_row[b] = row;
      }
      emit(b, ell_rows[b] - 1, fill[b], row, indices1[j]);
      ++fill[b];
    }
  }
}

int check_csf(const char* who, int32_t num_rels, const int32_t* indptr0, const int32_t* indptr1,
              const int32_t* rows_bkt, const int32_t* cols_bkt, int32_t nb) {
  STIR_REQUIRE(num_rels >= 0 && indptr0 && indptr1, "%s: bad CSF arguments", who);
  STIR_REQUIRE(nb > 0 && rows_bkt && cols_bkt, "%s: empty bucket list", who);
  for (int b = 0; b < nb; ++b)
    STIR_REQUIRE(rows_bkt[b] > 0 && cols_bkt[b] > 0, "%s: bucket sizes must be positive", who);
  for (int b = 1; b < nb; ++b)
    STIR_REQUIRE(cols_bkt[b - 1] < cols_bkt[b], "%s: The given nnz_cols_bkt should be ascending.", who);
  for (int r = 0; r < num_rels; ++r)
    STIR_REQUIRE(indptr0[r] <= indptr0[r + 1], "%s: indptr0 decreases at relation %d", who, r);
  for (int32_t i = indptr0[0]; i < indptr0[num_rels]; ++i)
    STIR_REQUIRE(indptr1[i] <= indptr1[i + 1], "%s: indptr1 decreases at stored row %d", who, i);
  return 0;
}

// groups_per_rel[b*num_rels + r] = whole groups of rows_bkt[b] ELL rows relation r needs.
void csf_count(int32_t num_rels, const int32_t* indptr0, const int32_t* indices0,
               const int32_t* indptr1, const int32_t* indices1, const int32_t* rows_bkt,
               const int32_t* cols_bkt, int32_t nb, std::vector<int64_t>& ell_rows_per_rel) {
  ell_rows_per_rel.assign(size_t(nb) * num_rels, 0);
  std::vector<int64_t> ell_rows(nb, 0);
  for (int r = 0; r < num_rels; ++r) {
    stream_relation(r, indptr0, indices0, indptr1, indices1, cols_bkt, nb, ell_rows,
                    [](int, int64_t, int, int32_t, int32_t) {});
    for (int b = 0; b < nb; ++b) ell_rows_per_rel[size_t(b) * num_rels + r] = ell_rows[b];
  }
  (void)rows_bkt;
}

}  // namespace

extern "C" {

int stir_column_part_hyb_sizes(int32_t num_rows, int32_t num_cols, const int32_t* indptr,
                               const int32_t* indices, int32_t num_col_parts,
                               const int32_t* buckets, int32_t num_buckets, int64_t* nrows) {
  STIR_REQUIRE(nrows, "ColumnPartHyb: nrows is null");
  return column_part_hyb_pass<false>(num_rows, num_cols, indptr, indices, num_col_parts, buckets,
                                     num_buckets, nrows, nullptr, nullptr, nullptr);
}

int stir_column_part_hyb_fill(int32_t num_rows, int32_t num_cols, const int32_t* indptr,
                              const int32_t* indices, int32_t num_col_parts,
                              const int32_t* buckets, int32_t num_buckets,
                              int32_t* const* row_indices, int32_t* const* col_indices,
                              int32_t* const* mask) {
  STIR_REQUIRE(row_indices && col_indices && mask, "ColumnPartHyb: null output table");
  return column_part_hyb_pass<true>(num_rows, num_cols, indptr, indices, num_col_parts, buckets,
                                    num_buckets, nullptr, row_indices, col_indices, mask);
}

int stir_csf_to_ell3d_sizes(int32_t num_rels, const int32_t* indptr0, const int32_t* indices0,
                            const int32_t* indptr1, const int32_t* indices1,
                            const int32_t* rows_bkt, const int32_t* cols_bkt,
                            int32_t num_buckets, int64_t* groups) {
  if (check_csf("CSFToELL3D", num_rels, indptr0, indptr1, rows_bkt, cols_bkt, num_buckets)) return -1;
  std::vector<int64_t> per_rel;
  csf_count(num_rels, indptr0, indices0, indptr1, indices1, rows_bkt, cols_bkt, num_buckets, per_rel);
  for (int b = 0; b < num_buckets; ++b) {
    int64_t g = 0;
    for (int r = 0; r < num_rels; ++r) g += stir::ceil_div(per_rel[size_t(b) * num_rels + r], rows_bkt[b]);
    groups[b] = g;
  }
  return 0;
}

int stir_csf_to_ell3d_fill(int32_t num_rels, const int32_t* indptr0, const int32_t* indices0,
                           const int32_t* indptr1, const int32_t* indices1,
                           const int32_t* rows_bkt, const int32_t* cols_bkt,
                           int32_t num_buckets, int32_t* const* indptr,
                           int32_t* const* row_indices, int32_t* const* col_indices,
                           int32_t* const* mask) {
  if (check_csf("CSFToELL3D", num_rels, indptr0, indptr1, rows_bkt, cols_bkt, num_buckets)) return -1;
  const int nb = num_buckets;
  std::vector<int64_t> per_rel;
  csf_count(num_rels, indptr0, indices0, indptr1, indices1, rows_bkt, cols_bkt, nb, per_rel);
  for (int b = 0; b < nb; ++b) {
    int64_t g = 0;
    indptr[b][0] = 0;
    for (int r = 0; r < num_rels; ++r) {
      g += stir::ceil_div(per_rel[size_t(b) * num_rels + r], rows_bkt[b]);
      indptr[b][r + 1] = int32_t(g);
    }
    const size_t slots = size_t(g) * rows_bkt[b] * cols_bkt[b];
    std::memset(col_indices[b], 0, slots * sizeof(int32_t));
    std::memset(mask[b], 0, slots * sizeof(int32_t));
  }
  std::vector<int64_t> ell_rows(nb, 0);
  for (int r = 0; r < num_rels; ++r) {
    stream_relation(r, indptr0, indices0, indptr1, indices1, cols_bkt, nb, ell_rows,
                    [&](int b, int64_t ell_row, int slot, int32_t row, int32_t col) {
                      const int64_t first = int64_t(indptr[b][r]) * rows_bkt[b];
                      row_indices[b][first + ell_row] = row;
                      const int64_t pos = (first + ell_row) * cols_bkt[b] + slot;
                      col_indices[b][pos] = col;
                      mask[b][pos] = 1;
                    });
    // pad the relation's ELL rows to whole groups by repeating its last row id
    for (int b = 0; b < nb; ++b) {
      const int64_t first = int64_t(indptr[b][r]) * rows_bkt[b];
      const int64_t end = int64_t(indptr[b][r + 1]) * rows_bkt[b];
      for (int64_t q = first + ell_rows[b]; q < end; ++q) row_indices[b][q] = row_indices[b][q - 1];
    }
  }
  return 0;
}

int stir_condense_sizes(int32_t n, const int32_t* indptr, const int32_t* indices, int32_t t,
                        int32_t g, int32_t* group_indptr, int64_t* num_groups) {
  if (check_csr("ConDense", n, indptr)) return -1;
  STIR_REQUIRE(t > 0 && g > 0, "ConDense: t=%d g=%d must be positive", t, g);
  STIR_REQUIRE(group_indptr && num_groups, "ConDense: null output");
  const int32_t tiles = (n + t - 1) / t;
  std::vector<int32_t> buf;
  int64_t groups = 0;
  group_indptr[0] = 0;
  for (int32_t tile = 0; tile < tiles; ++tile) {
    const int32_t r0 = tile * t, r1 = std::min(r0 + t, n);
    buf.assign(indices + indptr[r0], indices + indptr[r1]);
    std::sort(buf.begin(), buf.end());
    const int64_t uniq = std::unique(buf.begin(), buf.end()) - buf.begin();
    groups += stir::ceil_div(uniq, g);
    group_indptr[tile + 1] = int32_t(groups);
  }
  *num_groups = groups;
  return 0;
}

int stir_condense_fill(int32_t n, const int32_t* indptr, const int32_t* indices, int32_t t,
                       int32_t g, int32_t* tile_indices, int32_t* mask) {
  if (check_csr("ConDense", n, indptr)) return -1;
  STIR_REQUIRE(t > 0 && g > 0, "ConDense: t=%d g=%d must be positive", t, g);
  const int32_t tiles = (n + t - 1) / t;
  std::vector<int32_t> buf;
  int64_t groups = 0;
  for (int32_t tile = 0; tile < tiles; ++tile) {
    const int32_t r0 = tile * t, r1 = std::min(r0 + t, n);
    buf.assign(indices + indptr[r0], indices + indptr[r1]);
    std::sort(buf.begin(), buf.end());
    buf.erase(std::unique(buf.begin(), buf.end()), buf.end());
    const int64_t tile_groups = stir::ceil_div(int64_t(buf.size()), g);
    int32_t* ti = tile_indices + groups * g;
    int32_t* mk = mask + groups * t * g;
    std::fill(ti, ti + tile_groups * g, 0);
    std::fill(mk, mk + tile_groups * t * g, 0);
    std::copy(buf.begin(), buf.end(), ti);
    for (int32_t i = r0; i < r1; ++i)
      for (int32_t p = indptr[i]; p < indptr[i + 1]; ++p) {
        const int64_t u = std::lower_bound(buf.begin(), buf.end(), indices[p]) - buf.begin();
        mk[(u / g) * t * g + int64_t(i - r0) * g + u % g] = 1;
      }
    groups += tile_groups;
  }
  return 0;
}

}  // extern "C"
