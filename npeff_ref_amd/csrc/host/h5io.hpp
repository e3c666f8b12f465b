// hdf5 input and output of the two executables, field for field as the reference
// reads and writes them:
//   PEF input        cc/cuda_d_npeff/src/io/pef_fisher_h5.h:57-226
//                    (written by npeff/fishers/d_pefs_computer.py:235-251)
//   dense decomp     cc/cuda_d_npeff/src/io/nmf_decomp_h5.h:38-89
//                    (read by npeff/decomp/decomps.py:55-71)
//   sparse-H decomp  cc/cuda_d_npeff/src/io/nmf_decomp_h5.h:150-237,
//                    cc/cuda_d_npeff/src/util/h5_util.h:136-186
//                    (written by scripts/sparsify_d_npeff.py, npeff/decomp/decomps.py:113-140)
#pragma once

#include <hdf5.h>

#include <cstdint>
#include <string>
#include <vector>

#include "flags.hpp"

namespace h5io {

using hostutil::fatal;

inline hid_t check(hid_t id, const std::string& what) {
  if (id < 0) fatal("hdf5: " + what + " failed");
  return id;
}
inline void check_status(herr_t s, const std::string& what) {
  if (s < 0) fatal("hdf5: " + what + " failed");
}

struct PefDims {
  long n_rows = 0;
  long n_values_per_row = 0;
};

// Shape of data/fisher/values after the optional truncation flags
// (pef_fisher_h5.h:57-90,113-137).
inline PefDims pef_dims(const std::string& path, long n_examples, long n_fisher_values) {
  hid_t file = check(H5Fopen(path.c_str(), H5F_ACC_RDONLY, H5P_DEFAULT), "open " + path);
  hid_t ds = check(H5Dopen(file, "data/fisher/values", H5P_DEFAULT), "open data/fisher/values");
  hid_t sp = H5Dget_space(ds);
  if (H5Sget_simple_extent_ndims(sp) != 2) fatal("data/fisher/values must have rank 2");
  hsize_t dims[2];
  H5Sget_simple_extent_dims(sp, dims, nullptr);
  H5Sclose(sp);
  H5Dclose(ds);
  H5Fclose(file);
  PefDims d;
  d.n_rows = (long)dims[0];
  d.n_values_per_row = (long)dims[1];
  if (n_examples > 0) {
    if (n_examples > d.n_rows) fatal("n_examples exceeds the number of examples in the file");
    d.n_rows = n_examples;
  }
  if (n_fisher_values > 0) {
    if (n_fisher_values > d.n_values_per_row)
      fatal("n_fisher_values exceeds the number of values per example in the file");
    d.n_values_per_row = n_fisher_values;
  }
  return d;
}

struct Pef {
  long n_rows = 0, k = 0;
  long dense_fisher_size = 0;
  std::vector<float> values;    // [n_rows, k]
  std::vector<int32_t> indices; // [n_rows, k]
  std::vector<float> norms;     // [n_rows]
};

inline void read_hyperslab_2d(hid_t file, const char* name, hid_t mem_type, long n_rows, long n_cols,
                              void* out) {
  hid_t ds = check(H5Dopen(file, name, H5P_DEFAULT), std::string("open ") + name);
  hid_t sp = H5Dget_space(ds);
  hsize_t start[2] = {0, 0}, count[2] = {(hsize_t)n_rows, (hsize_t)n_cols};
  hid_t mem = H5Screate_simple(2, count, count);
  check_status(H5Sselect_hyperslab(sp, H5S_SELECT_SET, start, nullptr, count, nullptr), "hyperslab");
  check_status(H5Dread(ds, mem_type, mem, sp, H5P_DEFAULT, out), std::string("read ") + name);
  H5Sclose(mem);
  H5Sclose(sp);
  H5Dclose(ds);
}

// PefSparseFishers<IndT>::read (pef_fisher_h5.h:106-226).
inline Pef read_pef(const std::string& path, long n_examples, long n_fisher_values) {
  PefDims d = pef_dims(path, n_examples, n_fisher_values);
  Pef pef;
  pef.n_rows = d.n_rows;
  pef.k = d.n_values_per_row;
  hid_t file = check(H5Fopen(path.c_str(), H5F_ACC_RDONLY, H5P_DEFAULT), "open " + path);

  hid_t grp = check(H5Gopen(file, "data/fisher", H5P_DEFAULT), "open data/fisher");
  hid_t attr = check(H5Aopen_name(grp, "dense_fisher_size"), "open attribute dense_fisher_size");
  hid_t at = H5Aget_type(attr);
  // the reference insists on a 4-byte attribute (pef_fisher_h5.h:147-151)
  if (H5Tget_size(at) != 4) fatal("attribute dense_fisher_size must be a 4-byte integer");
  int n_cols = 0;
  check_status(H5Aread(attr, H5T_NATIVE_INT, &n_cols), "read dense_fisher_size");
  H5Tclose(at);
  H5Aclose(attr);
  H5Gclose(grp);
  pef.dense_fisher_size = n_cols;

  pef.values.resize((size_t)pef.n_rows * pef.k);
  pef.indices.resize((size_t)pef.n_rows * pef.k);
  pef.norms.resize((size_t)pef.n_rows);
  read_hyperslab_2d(file, "data/fisher/values", H5T_NATIVE_FLOAT, pef.n_rows, pef.k,
                    pef.values.data());
  read_hyperslab_2d(file, "data/fisher/indices", H5T_NATIVE_INT32, pef.n_rows, pef.k,
                    pef.indices.data());
  {
    hid_t ds = check(H5Dopen(file, "data/dense_fisher_norms", H5P_DEFAULT),
                     "open data/dense_fisher_norms");
    hid_t sp = H5Dget_space(ds);
    hsize_t start[1] = {0}, count[1] = {(hsize_t)pef.n_rows};
    hid_t mem = H5Screate_simple(1, count, count);
    check_status(H5Sselect_hyperslab(sp, H5S_SELECT_SET, start, nullptr, count, nullptr), "hyperslab");
    check_status(H5Dread(ds, H5T_NATIVE_FLOAT, mem, sp, H5P_DEFAULT, pef.norms.data()),
                 "read data/dense_fisher_norms");
    H5Sclose(mem);
    H5Sclose(sp);
    H5Dclose(ds);
  }
  H5Fclose(file);
  return pef;
}

// Writer of the PEF schema (what npeff/fishers/d_pefs_computer.py:235-251 produces),
// used by the synthetic-input tool and by tests.
inline void write_pef(const std::string& path, long n_rows, long k, int32_t dense_fisher_size,
                      const float* values, const int32_t* indices, const float* norms) {
  hid_t file = check(H5Fcreate(path.c_str(), H5F_ACC_TRUNC, H5P_DEFAULT, H5P_DEFAULT), "create " + path);
  hid_t data = check(H5Gcreate(file, "data", H5P_DEFAULT, H5P_DEFAULT, H5P_DEFAULT), "group data");
  hid_t fisher = check(H5Gcreate(data, "fisher", H5P_DEFAULT, H5P_DEFAULT, H5P_DEFAULT), "group fisher");
  {
    hid_t sp = H5Screate(H5S_SCALAR);
    hid_t a = check(H5Acreate(fisher, "dense_fisher_size", H5T_NATIVE_INT32, sp, H5P_DEFAULT, H5P_DEFAULT),
                    "attribute dense_fisher_size");
    check_status(H5Awrite(a, H5T_NATIVE_INT32, &dense_fisher_size), "write dense_fisher_size");
    H5Aclose(a);
    H5Sclose(sp);
  }
  hsize_t dims2[2] = {(hsize_t)n_rows, (hsize_t)k};
  {
    hid_t sp = H5Screate_simple(2, dims2, dims2);
    hid_t ds = check(H5Dcreate(fisher, "values", H5T_NATIVE_FLOAT, sp, H5P_DEFAULT, H5P_DEFAULT, H5P_DEFAULT), "values");
    check_status(H5Dwrite(ds, H5T_NATIVE_FLOAT, H5S_ALL, H5S_ALL, H5P_DEFAULT, values), "write values");
    H5Dclose(ds);
    ds = check(H5Dcreate(fisher, "indices", H5T_NATIVE_INT32, sp, H5P_DEFAULT, H5P_DEFAULT, H5P_DEFAULT), "indices");
    check_status(H5Dwrite(ds, H5T_NATIVE_INT32, H5S_ALL, H5S_ALL, H5P_DEFAULT, indices), "write indices");
    H5Dclose(ds);
    H5Sclose(sp);
  }
  {
    hsize_t dims1[1] = {(hsize_t)n_rows};
    hid_t sp = H5Screate_simple(1, dims1, dims1);
    hid_t ds = check(H5Dcreate(data, "dense_fisher_norms", H5T_NATIVE_FLOAT, sp, H5P_DEFAULT, H5P_DEFAULT, H5P_DEFAULT), "norms");
    check_status(H5Dwrite(ds, H5T_NATIVE_FLOAT, H5S_ALL, H5S_ALL, H5P_DEFAULT, norms), "write norms");
    H5Dclose(ds);
    H5Sclose(sp);
  }
  H5Gclose(fisher);
  H5Gclose(data);
  H5Fclose(file);
}

inline void write_matrix(hid_t grp, const char* name, long n_rows, long n_cols, const float* data) {
  hsize_t dims[2] = {(hsize_t)n_rows, (hsize_t)n_cols};
  hid_t sp = H5Screate_simple(2, dims, dims);
  hid_t ds = check(H5Dcreate(grp, name, H5T_NATIVE_FLOAT, sp, H5P_DEFAULT, H5P_DEFAULT, H5P_DEFAULT), name);
  check_status(H5Dwrite(ds, H5T_NATIVE_FLOAT, H5S_ALL, H5S_ALL, H5P_DEFAULT, data), std::string("write ") + name);
  H5Dclose(ds);
  H5Sclose(sp);
}

template <class T>
inline hid_t write_1d(hid_t grp, const char* name, hid_t type, const T* data, size_t n, bool close = true) {
  hsize_t dims[1] = {(hsize_t)n};
  hid_t sp = H5Screate_simple(1, dims, dims);
  hid_t ds = check(H5Dcreate(grp, name, type, sp, H5P_DEFAULT, H5P_DEFAULT, H5P_DEFAULT), name);
  check_status(H5Dwrite(ds, type, H5S_ALL, H5S_ALL, H5P_DEFAULT, data), std::string("write ") + name);
  H5Sclose(sp);
  if (close) H5Dclose(ds);
  return ds;
}

// NmfDecomposition<IndT>::save (nmf_decomp_h5.h:38-89): data/W [n, r], data/H [r, m],
// data/reduce_kept_indices [m] with attribute full_dense_size of shape (1,).  wide_indices:
// both are written as int64, as the reference's IndT = int64_t instantiation does (the main
// selects it when n_examples x n_fisher_values exceeds INT32_MAX, pef_fisher_h5.h:57-90).
inline void write_dense_decomposition(const std::string& path, long n, long r, long m, const float* W,
                                      const float* H, const int32_t* kept, int64_t full_dense_size,
                                      bool wide_indices = false) {
  hid_t file = check(H5Fcreate(path.c_str(), H5F_ACC_TRUNC, H5P_DEFAULT, H5P_DEFAULT), "create " + path);
  hid_t data = check(H5Gcreate(file, "data", H5P_DEFAULT, H5P_DEFAULT, H5P_DEFAULT), "group data");
  write_matrix(data, "W", n, r, W);
  write_matrix(data, "H", r, m, H);
  hid_t ds;
  hsize_t one[1] = {1};
  hid_t sp = H5Screate_simple(1, one, one);
  hid_t a;
  if (wide_indices) {
    std::vector<int64_t> kept64(kept, kept + m);
    ds = write_1d(data, "reduce_kept_indices", H5T_NATIVE_INT64, kept64.data(), (size_t)m, false);
    a = check(H5Acreate(ds, "full_dense_size", H5T_NATIVE_INT64, sp, H5P_DEFAULT, H5P_DEFAULT), "full_dense_size");
    check_status(H5Awrite(a, H5T_NATIVE_INT64, &full_dense_size), "write full_dense_size");
  } else {
    const int32_t fds = (int32_t)full_dense_size;
    ds = write_1d(data, "reduce_kept_indices", H5T_NATIVE_INT32, kept, (size_t)m, false);
    a = check(H5Acreate(ds, "full_dense_size", H5T_NATIVE_INT32, sp, H5P_DEFAULT, H5P_DEFAULT), "full_dense_size");
    check_status(H5Awrite(a, H5T_NATIVE_INT32, &fds), "write full_dense_size");
  }
  H5Aclose(a);
  H5Sclose(sp);
  H5Dclose(ds);
  H5Gclose(data);
  H5Fclose(file);
}

struct DenseDecomposition {
  long n = 0, r = 0, m = 0;
  std::vector<float> W, H;
  std::vector<int32_t> kept;
  long full_dense_size = 0;
};

inline std::vector<hsize_t> dataset_dims(hid_t file, const char* name) {
  hid_t ds = check(H5Dopen(file, name, H5P_DEFAULT), std::string("open ") + name);
  hid_t sp = H5Dget_space(ds);
  int nd = H5Sget_simple_extent_ndims(sp);
  std::vector<hsize_t> dims((size_t)(nd > 0 ? nd : 0));
  if (nd > 0) H5Sget_simple_extent_dims(sp, dims.data(), nullptr);
  H5Sclose(sp);
  H5Dclose(ds);
  return dims;
}

inline void read_all(hid_t file, const char* name, hid_t mem_type, void* out) {
  hid_t ds = check(H5Dopen(file, name, H5P_DEFAULT), std::string("open ") + name);
  check_status(H5Dread(ds, mem_type, H5S_ALL, H5S_ALL, H5P_DEFAULT, out), std::string("read ") + name);
  H5Dclose(ds);
}

// Integer attribute of any width and of shape () or (1,), as a long.
inline long read_int_attr(hid_t obj, const char* name) {
  hid_t a = check(H5Aopen_name(obj, name), std::string("open attribute ") + name);
  int64_t v[1] = {0};
  check_status(H5Aread(a, H5T_NATIVE_INT64, v), std::string("read attribute ") + name);
  H5Aclose(a);
  return (long)v[0];
}

inline DenseDecomposition read_dense_decomposition(const std::string& path) {
  DenseDecomposition d;
  hid_t file = check(H5Fopen(path.c_str(), H5F_ACC_RDONLY, H5P_DEFAULT), "open " + path);
  auto wd = dataset_dims(file, "data/W"), hd = dataset_dims(file, "data/H");
  if (wd.size() != 2 || hd.size() != 2) fatal("data/W and data/H must have rank 2");
  d.n = (long)wd[0]; d.r = (long)wd[1]; d.m = (long)hd[1];
  if ((long)hd[0] != d.r) fatal("data/W and data/H disagree on the number of components");
  d.W.resize((size_t)d.n * d.r);
  d.H.resize((size_t)d.r * d.m);
  d.kept.resize((size_t)d.m);
  read_all(file, "data/W", H5T_NATIVE_FLOAT, d.W.data());
  read_all(file, "data/H", H5T_NATIVE_FLOAT, d.H.data());
  read_all(file, "data/reduce_kept_indices", H5T_NATIVE_INT32, d.kept.data());
  hid_t ds = check(H5Dopen(file, "data/reduce_kept_indices", H5P_DEFAULT), "open reduce_kept_indices");
  d.full_dense_size = read_int_attr(ds, "full_dense_size");
  H5Dclose(ds);
  H5Fclose(file);
  return d;
}

// Rows [row0, row0 + n_rows) of a 2-D float dataset.
inline void read_rows_2d(hid_t file, const char* name, long row0, long n_rows, long n_cols, float* out) {
  hid_t ds = check(H5Dopen(file, name, H5P_DEFAULT), std::string("open ") + name);
  hid_t sp = H5Dget_space(ds);
  hsize_t start[2] = {(hsize_t)row0, 0}, count[2] = {(hsize_t)n_rows, (hsize_t)n_cols};
  hid_t mem = H5Screate_simple(2, count, count);
  check_status(H5Sselect_hyperslab(sp, H5S_SELECT_SET, start, nullptr, count, nullptr), "hyperslab");
  check_status(H5Dread(ds, H5T_NATIVE_FLOAT, mem, sp, H5P_DEFAULT, out), std::string("read ") + name);
  H5Sclose(mem);
  H5Sclose(sp);
  H5Dclose(ds);
}

struct SparseDecomposition {
  long n = 0, r = 0, m = 0;            // W [n, r]; H [r, m] CSR
  std::vector<float> W;
  std::vector<float> H_values;
  std::vector<int64_t> H_row_offsets;  // [r + 1]
  std::vector<int32_t> H_col_indices;
  std::vector<int32_t> kept;           // [m]
  long full_dense_size = 0;
};

// SparseNmfDecomposition<IndT>::read (nmf_decomp_h5.h:178-237).
inline SparseDecomposition read_sparse_decomposition(const std::string& path) {
  SparseDecomposition d;
  hid_t file = check(H5Fopen(path.c_str(), H5F_ACC_RDONLY, H5P_DEFAULT), "open " + path);
  auto wd = dataset_dims(file, "data/W");
  if (wd.size() != 2) fatal("data/W must have rank 2");
  d.n = (long)wd[0];
  d.W.resize((size_t)wd[0] * wd[1]);
  read_all(file, "data/W", H5T_NATIVE_FLOAT, d.W.data());
  hid_t hg = check(H5Gopen(file, "data/H", H5P_DEFAULT), "open data/H");
  {
    hid_t a = check(H5Aopen_name(hg, "shape"), "open attribute shape");
    int64_t shape[2] = {0, 0};
    check_status(H5Aread(a, H5T_NATIVE_INT64, shape), "read attribute shape");
    H5Aclose(a);
    d.r = (long)shape[0];
    d.m = (long)shape[1];
  }
  H5Gclose(hg);
  auto vd = dataset_dims(file, "data/H/values");
  size_t nnz = vd.empty() ? 0 : (size_t)vd[0];
  d.H_values.resize(nnz);
  d.H_col_indices.resize(nnz);
  d.H_row_offsets.resize((size_t)d.r + 1);
  auto rd = dataset_dims(file, "data/H/row_indices");
  if (rd.size() != 1 || (long)rd[0] != d.r + 1) fatal("data/H/row_indices must have r + 1 entries");
  if (nnz) read_all(file, "data/H/values", H5T_NATIVE_FLOAT, d.H_values.data());
  read_all(file, "data/H/row_indices", H5T_NATIVE_INT64, d.H_row_offsets.data());
  if (nnz) read_all(file, "data/H/column_indices", H5T_NATIVE_INT32, d.H_col_indices.data());
  auto kd = dataset_dims(file, "data/reduce_kept_indices");
  d.kept.resize(kd.empty() ? 0 : (size_t)kd[0]);
  if (!d.kept.empty()) read_all(file, "data/reduce_kept_indices", H5T_NATIVE_INT32, d.kept.data());
  hid_t ds = check(H5Dopen(file, "data/reduce_kept_indices", H5P_DEFAULT), "open reduce_kept_indices");
  d.full_dense_size = read_int_attr(ds, "full_dense_size");
  H5Dclose(ds);
  H5Fclose(file);
  return d;
}

// SparseNmfDecomposition<int32_t>::save (nmf_decomp_h5.h:150-170): group data/H with values,
// row_indices, column_indices and attribute shape (int64[2]); full_dense_size is a scalar
// attribute here (h5_util.h:157-170).  row_indices are written as int64, the width
// scripts/sparsify_d_npeff.py:46 uses.
inline void write_sparse_decomposition(const std::string& path, const SparseDecomposition& d) {
  hid_t file = check(H5Fcreate(path.c_str(), H5F_ACC_TRUNC, H5P_DEFAULT, H5P_DEFAULT), "create " + path);
  hid_t data = check(H5Gcreate(file, "data", H5P_DEFAULT, H5P_DEFAULT, H5P_DEFAULT), "group data");
  write_matrix(data, "W", d.n, d.r, d.W.data());
  hid_t hg = check(H5Gcreate(data, "H", H5P_DEFAULT, H5P_DEFAULT, H5P_DEFAULT), "group H");
  write_1d(hg, "values", H5T_NATIVE_FLOAT, d.H_values.data(), d.H_values.size());
  write_1d(hg, "row_indices", H5T_NATIVE_INT64, d.H_row_offsets.data(), d.H_row_offsets.size());
  write_1d(hg, "column_indices", H5T_NATIVE_INT32, d.H_col_indices.data(), d.H_col_indices.size());
  {
    int64_t shape[2] = {d.r, d.m};
    hsize_t two[1] = {2};
    hid_t sp = H5Screate_simple(1, two, two);
    hid_t a = check(H5Acreate(hg, "shape", H5T_NATIVE_INT64, sp, H5P_DEFAULT, H5P_DEFAULT), "shape");
    check_status(H5Awrite(a, H5T_NATIVE_INT64, shape), "write shape");
    H5Aclose(a);
    H5Sclose(sp);
  }
  H5Gclose(hg);
  hid_t ds = write_1d(data, "reduce_kept_indices", H5T_NATIVE_INT32, d.kept.data(), d.kept.size(), false);
  {
    int32_t fds = (int32_t)d.full_dense_size;
    hid_t sp = H5Screate(H5S_SCALAR);
    hid_t a = check(H5Acreate(ds, "full_dense_size", H5T_NATIVE_INT32, sp, H5P_DEFAULT, H5P_DEFAULT), "full_dense_size");
    check_status(H5Awrite(a, H5T_NATIVE_INT32, &fds), "write full_dense_size");
    H5Aclose(a);
    H5Sclose(sp);
  }
  H5Dclose(ds);
  H5Gclose(data);
  H5Fclose(file);
}

}  // namespace h5io
