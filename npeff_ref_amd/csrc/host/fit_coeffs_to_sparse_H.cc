// fit_coeffs_to_sparse_H: learns W for new examples against a fixed sparse H on one MI355X
// through the C ABI of dnpeff.h.  Flags, checks, order of steps and stdout lines follow
// cc/cuda_d_npeff/mains/fit_coeffs_to_sparse_H.cu:26-226; the two stages follow
// cc/cuda_d_npeff/src/nmf/sparse2/nmf_sparse_H.h:116-345.
#include <chrono>
#include <climits>
#include <iostream>
#include <numeric>
#include <string>
#include <vector>

#include "../../../include/dnpeff.h"
#include "flags.hpp"
#include "h5io.hpp"

using hostutil::fatal;

static void ck(int status) {
  if (status) fatal(std::string("Error: ") + dnpeff_last_error());
}

struct ProgramFlags {
  std::string output_path, pef_path, nmf_path;
  int n_splits_sparse_matmul = 0;  // memory knob of the reference's partitioned SpGEMM; the
                                   // single sparse x sparse kernel here needs no partitions
  int n_row_splits_pefs = 0;
  int max_iters = 0;
  int n_examples = -1, n_fisher_values = -1;
  int main_device = 0;
  int DEV_n_cols = -1;
  // additions (optional): the reference hard-codes eps at fit_coeffs_to_sparse_H.cu:185, logs
  // every 25 steps (only_W_learner_params.h:35) and leaves the seed unset
  float eps = 1e-7f;
  long seed = 43190432042L;
  int log_every = 25;
};

static ProgramFlags read_flags(int argc, char** argv) {
  hostutil::Flags f(argc, argv);
  ProgramFlags p;
  f.read("output_path", &p.output_path);
  f.read("pef_path", &p.pef_path);
  f.read("H_path", &p.nmf_path);
  f.read("n_splits_sparse_matmul", &p.n_splits_sparse_matmul);
  f.read("n_row_splits_pefs", &p.n_row_splits_pefs);
  f.read("nmf_max_iter", &p.max_iters);
  f.read("n_examples", &p.n_examples, false);
  f.read("n_fisher_values", &p.n_fisher_values, false);
  f.read("main_device", &p.main_device, false);
  f.read("DEV_n_cols", &p.DEV_n_cols, false);
  f.read("eps", &p.eps, false);
  f.read("seed", &p.seed, false);
  f.read("log_every", &p.log_every, false);
  f.verify_no_unread();
  return p;
}

int main(int argc, char** argv) {
  ProgramFlags flags = read_flags(argc, argv);

  int n_devices = 0;
  ck(dnpeff_device_count(&n_devices));
  if (n_devices != 1) fatal("Only single GPU is supported.");
  if (flags.n_row_splits_pefs < 1) fatal("Error: n_row_splits_pefs must be at least 1.");

  std::cout << "Starting to read in H.\n";
  h5io::SparseDecomposition sp = h5io::read_sparse_decomposition(flags.nmf_path);
  std::cout << "H read in.\n";
  dnpeff_csr* H = nullptr;
  ck(dnpeff_csr_from_host(sp.r, sp.m, (int64_t)sp.H_values.size(), sp.H_row_offsets.data(),
                          sp.H_col_indices.data(), sp.H_values.data(), &H));

  std::cout << "Starting to read in PEFs.\n";
  h5io::Pef pef = h5io::read_pef(flags.pef_path, flags.n_examples, flags.n_fisher_values);
  std::cout << "PEFS read in.\n";
  dnpeff_csr* A = nullptr;
  ck(dnpeff_csr_from_pef(pef.n_rows, pef.k, pef.dense_fisher_size, pef.indices.data(),
                         pef.values.data(), &A));
  pef.values = std::vector<float>();
  pef.indices = std::vector<int32_t>();
  ck(dnpeff_csr_normalize_rows(A, pef.norms.data(), 1e-9f));

  if ((long)sp.kept.size() < sp.m) fatal("Error: reduce_kept_indices is shorter than H has columns.");
  ck(dnpeff_csr_retain_columns(A, sp.kept.data(), sp.m));

  if (flags.DEV_n_cols >= 0) {
    std::cout << "NOTE: Using flag intended only for development purposes.\n";
    std::vector<int32_t> v((size_t)flags.DEV_n_cols);
    std::iota(v.begin(), v.end(), 0);
    ck(dnpeff_csr_retain_columns(A, v.data(), (int64_t)v.size()));
    ck(dnpeff_csr_retain_columns(H, v.data(), (int64_t)v.size()));
  }

  // The reference splits the rows and insists that every split can be indexed with 32 bits
  // (fit_coeffs_to_sparse_H.cu:150-166); the check is kept, the split itself is not needed.
  int64_t n = 0, m = 0, nnz = 0;
  ck(dnpeff_csr_shape(A, &n, &m, &nnz));
  {
    std::vector<int64_t> rowptr((size_t)n + 1);
    ck(dnpeff_csr_download(A, rowptr.data(), nullptr, nullptr));
    int64_t start_row = 0;
    for (int s = 0; s < flags.n_row_splits_pefs; s++) {
      int64_t end_row = start_row + dnpeff_size_of_split(n, flags.n_row_splits_pefs, s);
      int64_t split_nnz = rowptr[end_row] - rowptr[start_row];
      if (!(split_nnz < (int64_t)INT32_MAX)) {
        std::cout << "Row split of PEFs cannot use int32 indices [nnz = " << split_nnz << "].\n";
        fatal("Error: increase n_row_splits_pefs.");
      }
      start_row = end_row;
    }
  }

  dnpeff_fit* fit = nullptr;
  ck(dnpeff_fit_create(A, H, flags.eps, flags.seed, &fit));
  ck(dnpeff_sync());
  std::cout << "Finished running first stage.\n";
  dnpeff_csr_destroy(A);

  ck(dnpeff_fit_init_W(fit));
  ck(dnpeff_sync());
  auto t_start = std::chrono::high_resolution_clock::now();
  // the steps up to the next logged one in one call (the library then prepares H H^T once for all
  // of them); the sequence of updates is the loop's, one step at a time
  for (long i = 0; i < flags.max_iters;) {
    long run = flags.max_iters - i;
    if (flags.log_every > 0 && run > flags.log_every - i % flags.log_every) run = flags.log_every - i % flags.log_every;
    if (run > 1000000) run = 1000000;
    ck(dnpeff_fit_step(fit, (int)run));
    i += run - 1;
    if (flags.log_every > 0 && ((i + 1) % flags.log_every) == 0) {
      ck(dnpeff_sync());
      auto t_end = std::chrono::high_resolution_clock::now();
      double elapsed_ms = std::chrono::duration<double, std::milli>(t_end - t_start).count();
      double ref_loss = 0.0;
      ck(dnpeff_fit_loss(fit, &ref_loss, nullptr));
      std::cout << "step " << i + 1 << ": " << (float)ref_loss << " ["
                << elapsed_ms / (double)flags.log_every << " ms/step]\n";
      t_start = std::chrono::high_resolution_clock::now();
    }
    i++;
  }
  ck(dnpeff_sync());
  std::cout << "Finished running second stage.\n";

  // New W, unchanged sparse H (after DEV_n_cols, if given, as the reference does).
  h5io::SparseDecomposition out;
  int64_t hr = 0, hm = 0, hnnz = 0;
  ck(dnpeff_csr_shape(H, &hr, &hm, &hnnz));
  out.n = n; out.r = hr; out.m = hm;
  out.W.resize((size_t)n * hr);
  ck(dnpeff_fit_get_W(fit, out.W.data()));
  out.H_row_offsets.resize((size_t)hr + 1);
  out.H_col_indices.resize((size_t)hnnz);
  out.H_values.resize((size_t)hnnz);
  ck(dnpeff_csr_download(H, out.H_row_offsets.data(), out.H_col_indices.data(), out.H_values.data()));
  out.kept.assign(sp.kept.begin(), sp.kept.begin() + hm);
  out.full_dense_size = sp.full_dense_size;
  h5io::write_sparse_decomposition(flags.output_path, out);

  dnpeff_fit_destroy(fit);
  dnpeff_csr_destroy(H);
  return 0;
}
