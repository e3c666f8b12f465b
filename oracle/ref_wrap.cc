// TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
//
// extern "C" entry points around the reference's own host-only routines, which
// are compiled from where they lie under $(REFERENCE)/cc/cuda_lrm_npeff/src
// (nothing is copied).  They restate, for the LRM code base, the column
// compaction that the D-NPEFF path runs
// (cc/cuda_d_npeff/src/util/sparse_util.h:78-159 is the same sweep as
// cc/cuda_lrm_npeff/src/preprocess/column_pruning.h:14-82), and are used to
// check oracle/dnpeff_oracle.c on random inputs.  Built only where the
// reference tree is present; outputs go to oracle/_ref/.
#include <cstdint>
#include <cstring>
#include <memory>

#include <containers/conversions.h>
#include <containers/sparse_matrix.h>
#include <preprocess/column_pruning.h>
#include <util/array_util.h>

using npeff::CsrMatrix;
using npeff::DenseMatrix;

namespace {
template <typename T>
std::unique_ptr<T> copy_array(const T* src, int64_t n) {
  std::unique_ptr<T> p(new T[n > 0 ? n : 1]);
  if (n > 0) std::memcpy(p.get(), src, sizeof(T) * n);
  return p;
}
}  // namespace

extern "C" {

// prune_columns_in_place on int32 CSR arrays (row offsets int32, as the
// reference template uses one index type).  Arrays are updated in place;
// returns the new column count, *nnz_out the new nnz.
int64_t ref_prune_columns_i32(int64_t n_rows, int64_t n_cols, int64_t nnz, int32_t* row_offsets,
                              int32_t* col_indices, float* values, int64_t min_nnz_per_col,
                              int32_t* new_to_old, int64_t* nnz_out) {
  CsrMatrix<int32_t> mat(n_rows, n_cols, nnz, copy_array(values, nnz),
                         copy_array(row_offsets, n_rows + 1), copy_array(col_indices, nnz));
  std::unique_ptr<DenseMatrix<int32_t>> map;
  npeff::preprocessing::prune_columns_in_place(&mat, &map, min_nnz_per_col);
  std::memcpy(row_offsets, mat.row_offsets.get(), sizeof(int32_t) * (n_rows + 1));
  std::memcpy(col_indices, mat.col_indices.get(), sizeof(int32_t) * mat.nnz);
  std::memcpy(values, mat.values.get(), sizeof(float) * mat.nnz);
  std::memcpy(new_to_old, map->data.get(), sizeof(int32_t) * mat.n_cols);
  *nnz_out = mat.nnz;
  return mat.n_cols;
}

// csr_from_row_major_array; output arrays sized n_rows*n_cols by the caller.
int64_t ref_csr_from_row_major(const float* dense, int64_t n_rows, int64_t n_cols, float threshold,
                               int32_t* row_offsets, int32_t* col_indices, float* values) {
  std::unique_ptr<float> tmp = copy_array(dense, n_rows * n_cols);
  CsrMatrix<int32_t> mat =
      npeff::containers::csr_from_row_major_array<int32_t>(tmp.get(), n_rows, n_cols, threshold);
  std::memcpy(row_offsets, mat.row_offsets.get(), sizeof(int32_t) * (n_rows + 1));
  std::memcpy(col_indices, mat.col_indices.get(), sizeof(int32_t) * mat.nnz);
  std::memcpy(values, mat.values.get(), sizeof(float) * mat.nnz);
  return mat.nnz;
}

int ref_validate_indices(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t* row_offsets,
                         const int32_t* col_indices) {
  std::unique_ptr<float> vals(new float[nnz > 0 ? nnz : 1]);
  CsrMatrix<int32_t> mat(n_rows, n_cols, nnz, std::move(vals), copy_array(row_offsets, n_rows + 1),
                         copy_array(col_indices, nnz));
  return mat.validate_indices() ? 1 : 0;
}

// convert_numeric_arrays(dst, src, n): the direction pinned by
// cc/cuda_lrm_npeff/src/util/array_util_test.cc:7-19.
void ref_convert_i32_to_i64(int64_t* dst, int32_t* src, int64_t n) {
  npeff::util::convert_numeric_arrays(dst, src, (size_t)n);
}

}  // extern "C"
