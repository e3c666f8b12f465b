// sparsify_d_npeff: dense D-NPEFF decomposition -> decomposition with a CSR H, the input format
// of fit_coeffs_to_sparse_H.  Same flags and output schema as the reference's
// scripts/sparsify_d_npeff.py:18-73 (SparseDNpeffDecomposition.save, npeff/decomp/decomps.py:114-127).
//
// The script first calls normalize_components_to_unit_norm(), which the decomposition class does
// not define (decomps.py:24-71); what is built here is what the name says: every row of H is
// scaled to unit L2 norm and the matching column of W is multiplied by that norm, so W H is
// unchanged.  A row of zeros is left alone.  Then, per row, the entries >= H_threshold are kept
// in ascending column order (to_csr, :27-49).
//
// H is read one component at a time (the dense H of a full-size fit does not fit in host
// memory next to its sparse copy) and reduced on the GPU: fp64 sum of squares, then the
// threshold compaction.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "../../../include/dnpeff.h"
#include "flags.hpp"
#include "h5io.hpp"

using hostutil::fatal;

static void ok(int status) {
  if (status) fatal(std::string("Error: ") + dnpeff_last_error());
}

int main(int argc, char** argv) {
  hostutil::Flags flags(argc, argv);
  std::string in_path, out_path;
  float threshold = 0.0f;
  flags.read("decomposition_filepath", &in_path);
  flags.read("output_filepath", &out_path);
  flags.read("H_threshold", &threshold);  // the script asserts that it is given (:53)
  flags.verify_no_unread();

  hid_t file = h5io::check(H5Fopen(in_path.c_str(), H5F_ACC_RDONLY, H5P_DEFAULT), "open " + in_path);
  auto wd = h5io::dataset_dims(file, "data/W"), hd = h5io::dataset_dims(file, "data/H");
  if (wd.size() != 2 || hd.size() != 2) fatal("data/W and data/H must have rank 2");
  h5io::SparseDecomposition out;
  out.n = (long)wd[0];
  out.r = (long)wd[1];
  out.m = (long)hd[1];
  if ((long)hd[0] != out.r) fatal("data/W and data/H disagree on the number of components");
  if (out.m > (long)INT32_MAX) fatal("more than 2^31 - 1 features");
  out.W.resize((size_t)out.n * out.r);
  out.kept.resize((size_t)out.m);
  h5io::read_all(file, "data/W", H5T_NATIVE_FLOAT, out.W.data());
  h5io::read_all(file, "data/reduce_kept_indices", H5T_NATIVE_INT32, out.kept.data());
  {
    hid_t ds = h5io::check(H5Dopen(file, "data/reduce_kept_indices", H5P_DEFAULT), "open reduce_kept_indices");
    out.full_dense_size = h5io::read_int_attr(ds, "full_dense_size");
    H5Dclose(ds);
  }
  std::printf("Dense size: %ld\n", out.r * out.m);

  int n_dev = 0;
  ok(dnpeff_device_count(&n_dev));
  if (n_dev < 1) fatal("Error: no GPU visible.");
  void *x = nullptr, *idx = nullptr, *val = nullptr;
  const size_t m = (size_t)out.m;
  ok(dnpeff_dev_malloc(m * 4 + 4, &x));
  ok(dnpeff_dev_malloc(m * 4 + 4, &idx));
  ok(dnpeff_dev_malloc(m * 4 + 4, &val));
  std::vector<float> row(m);
  out.H_row_offsets.assign(1, 0);
  for (long k = 0; k < out.r; k++) {
    h5io::read_rows_2d(file, "data/H", k, 1, out.m, row.data());
    ok(dnpeff_dev_upload(x, row.data(), m * 4));
    double sq = 0.0;
    ok(dnpeff_op_dot(out.m, (const float*)x, (const float*)x, &sq));
    const float norm = (float)std::sqrt(sq);
    const float divisor = norm > 0.0f ? norm : 1.0f;
    int64_t kept = 0;
    ok(dnpeff_op_threshold_compact(out.m, (const float*)x, divisor, threshold, (int32_t*)idx,
                                   (float*)val, &kept));
    const size_t at = out.H_values.size();
    out.H_values.resize(at + (size_t)kept);
    out.H_col_indices.resize(at + (size_t)kept);
    if (kept) {
      ok(dnpeff_dev_download(out.H_values.data() + at, val, (size_t)kept * 4));
      ok(dnpeff_dev_download(out.H_col_indices.data() + at, idx, (size_t)kept * 4));
    }
    out.H_row_offsets.push_back((int64_t)out.H_values.size());
    for (long i = 0; i < out.n; i++) out.W[(size_t)i * out.r + k] *= divisor;
  }
  H5Fclose(file);
  dnpeff_dev_free(x);
  dnpeff_dev_free(idx);
  dnpeff_dev_free(val);
  std::printf("Sparse NNZ: %zu\n", out.H_values.size());
  h5io::write_sparse_decomposition(out_path, out);
  return 0;
}
