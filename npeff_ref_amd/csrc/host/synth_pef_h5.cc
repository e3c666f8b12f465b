// synth_pef_h5: writes a synthetic D-PEF hdf5 file in the layout that
// npeff/fishers/d_pefs_computer.py:235-251 produces, for tests and benchmarks of the two
// executables: per example k distinct parameter ids by successive Zipf(s) draws (draw order
// kept), log-normal values and the row's L2 norm as dense_fisher_norms.  Optionally also a
// random sparse-H decomposition file for fit_coeffs_to_sparse_H.
#include <cmath>
#include <iostream>
#include <string>
#include <vector>

#include "../../../include/dnpeff.h"
#include "flags.hpp"
#include "h5io.hpp"

using hostutil::fatal;

int main(int argc, char** argv) {
  hostutil::Flags f(argc, argv);
  std::string out, sparse_h_out;
  int n_examples = 0, n_values = 0, rank = 0;
  long n_parameters = 0, seed = 1;
  float zipf_s = 1.1f, mu = -8.0f, sigma = 2.0f, h_density = 0.01f;
  f.read("output_path", &out);
  f.read("n_examples", &n_examples);
  f.read("n_parameters", &n_parameters);
  f.read("n_fisher_values", &n_values);
  f.read("zipf_s", &zipf_s, false);
  f.read("mu", &mu, false);
  f.read("sigma", &sigma, false);
  f.read("seed", &seed, false);
  f.read("sparse_H_output_path", &sparse_h_out, false);
  f.read("rank", &rank, false);
  f.read("H_density", &h_density, false);
  int on_device = 0;  // 1: the device generator (same bits, far faster for files of gigabytes)
  f.read("on_device", &on_device, false);
  f.verify_no_unread();

  const size_t z = (size_t)n_examples * (size_t)n_values;
  std::vector<int64_t> rowptr((size_t)n_examples + 1);
  std::vector<int32_t> indices(z);
  std::vector<float> values(z), norms((size_t)n_examples);
  if (on_device) {
    dnpeff_csr* A = nullptr;
    if (dnpeff_synth_pef(n_examples, n_parameters, n_values, 0, 0, zipf_s, mu, sigma, (uint64_t)seed,
                         norms.data(), &A) ||
        dnpeff_csr_download(A, rowptr.data(), indices.data(), values.data()))
      fatal(std::string("Error: ") + dnpeff_last_error());
    dnpeff_csr_destroy(A);
  } else if (dnpeff_synth_pef_host(n_examples, n_parameters, n_values, 0, 0, zipf_s, mu, sigma,
                                   (uint64_t)seed, rowptr.data(), indices.data(), values.data(),
                                   norms.data())) {
    fatal(std::string("Error: ") + dnpeff_last_error());
  }
  h5io::write_pef(out, n_examples, n_values, (int32_t)n_parameters, values.data(), indices.data(),
                  norms.data());
  std::cout << "wrote " << out << ": " << n_examples << " x " << n_values << " of " << n_parameters
            << " parameters\n";

  if (!sparse_h_out.empty()) {
    if (rank < 1) fatal("Missing flag: rank");
    // H over all parameters (reduce_kept_indices = identity): entry (c, j) present with
    // probability H_density, value U[0,1) from the seeded generator of the library.
    h5io::SparseDecomposition sp;
    sp.n = 1; sp.r = rank; sp.m = n_parameters; sp.full_dense_size = n_parameters;
    sp.W.assign((size_t)rank, 0.0f);
    sp.H_row_offsets.push_back(0);
    for (int c = 0; c < rank; c++) {
      for (long j = 0; j < n_parameters; j++) {
        float u = dnpeff_uniform_at((uint64_t)seed + 17, 2, c, j, n_parameters);
        if (u < h_density) {
          sp.H_col_indices.push_back((int32_t)j);
          sp.H_values.push_back(dnpeff_uniform_at((uint64_t)seed + 17, 3, c, j, n_parameters) + 1e-3f);
        }
      }
      sp.H_row_offsets.push_back((int64_t)sp.H_values.size());
    }
    sp.kept.resize((size_t)n_parameters);
    for (long j = 0; j < n_parameters; j++) sp.kept[(size_t)j] = (int32_t)j;
    h5io::write_sparse_decomposition(sparse_h_out, sp);
    std::cout << "wrote " << sparse_h_out << ": H " << rank << " x " << n_parameters << ", nnz "
              << sp.H_values.size() << "\n";
  }
  return 0;
}
