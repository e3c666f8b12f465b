// run_nmf_on_pefs: reads a D-PEF hdf5 file, normalises the rows, drops sparse columns and runs
// multiplicative-update NMF with dense W and H on one MI355X through the C ABI of dnpeff.h;
// writes W, H and the kept-column map.  Flags, order of steps, defaults and stdout lines follow
// cc/cuda_d_npeff/mains/run_nmf_on_pefs.cu:15-259; the loop and its timer follow
// cc/cuda_d_npeff/src/nmf/sparse/multi_mu_dense_factors_nmf1.h:152-205.
#include <chrono>
#include <climits>
#include <cmath>
#include <iostream>
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
  std::string output_path, pef_path;
  int n_components = 0, max_iters = 0;
  int n_examples = -1, n_fisher_values = -1;
  float sparsity_W = -1.0f;            // accepted, without effect on the run (as in the reference, which
                                       // never calls its projection; dnpeff_nmf_sparsify_W is that call)
  int min_values_per_parameter = 1;
  std::string initial_H_path, initial_W_path;  // accepted, without effect (as in the reference)
  // additions (optional): the reference hard-codes these at run_nmf_on_pefs.cu:189-192
  float eps = 1e-8f;
  long seed = 43190432042L;
  int log_every = 10;
  int index_width = 0;  // 0: the reference's rule (64 when n_examples x n_fisher_values exceeds INT32_MAX)
};

static ProgramFlags parse_flags(int argc, char** argv) {
  hostutil::Flags f(argc, argv);
  ProgramFlags p;
  f.read("output_path", &p.output_path);
  f.read("per_example_fishers", &p.pef_path);
  f.read("nmf_n_components", &p.n_components);
  f.read("nmf_max_iter", &p.max_iters);
  f.read("n_examples", &p.n_examples, false);
  f.read("n_fisher_values", &p.n_fisher_values, false);
  f.read("min_values_per_parameter", &p.min_values_per_parameter, false);
  f.read("sparsity_W", &p.sparsity_W, false);
  f.read("initial_H_path", &p.initial_H_path, false);
  f.read("initial_W_path", &p.initial_W_path, false);
  f.read("eps", &p.eps, false);
  f.read("seed", &p.seed, false);
  f.read("log_every", &p.log_every, false);
  f.read("index_width", &p.index_width, false);
  return p;  // unknown flags are ignored, as in the reference
}

int main(int argc, char** argv) {
  ProgramFlags flags = parse_flags(argc, argv);

  h5io::PefDims dims = h5io::pef_dims(flags.pef_path, flags.n_examples, flags.n_fisher_values);
  const long nnz_in = dims.n_rows * dims.n_values_per_row;
  // Row offsets are always 64-bit and column ids 32-bit inside the library; the reference's
  // choice of index type still decides the log lines and the type of reduce_kept_indices /
  // full_dense_size in the output file (nmf_decomp_h5.h:58-75).  The reference chooses in two
  // steps (run_nmf_on_pefs.cu:236-254): it reads with 64-bit indices when n_examples x
  // n_fisher_values exceeds INT32_MAX, and then runs and saves with 32-bit ones when
  // canReindexWithInt32() says so, which (matrices.h:219-224) is when the pruned matrix still holds
  // more than INT32_MAX entries; only a matrix that pruning brought under INT32_MAX is run and
  // saved with 64-bit indices.  The same file types come out here; --index_width overrides.
  if (flags.index_width != 0 && flags.index_width != 32 && flags.index_width != 64)
    fatal("Error: --index_width must be 32 or 64.");
  const bool read_wide = nnz_in > (long)INT32_MAX;
  if (read_wide)
    std::cout << "Reading in PEFs using 64 bit indices.\n";
  else
    std::cout << "Using 32 bit indices.\n";

  int n_devices = 0;
  ck(dnpeff_device_count(&n_devices));
  if (n_devices < 1) fatal("Error: no GPU visible.");

  std::cout << "Starting to read in PEFs.\n";
  h5io::Pef pef = h5io::read_pef(flags.pef_path, flags.n_examples, flags.n_fisher_values);
  std::cout << "PEFS read in.\n";

  dnpeff_csr* A = nullptr;
  ck(dnpeff_csr_from_pef(pef.n_rows, pef.k, pef.dense_fisher_size, pef.indices.data(),
                         pef.values.data(), &A));
  pef.values = std::vector<float>();
  pef.indices = std::vector<int32_t>();
  ck(dnpeff_csr_normalize_rows(A, pef.norms.data(), 1e-9f));

  int64_t n = 0, m = 0, nnz = 0;
  ck(dnpeff_csr_shape(A, &n, &m, &nnz));
  std::cout << "n_cols before reduction: " << m << "\n";
  ck(dnpeff_csr_compact_columns(A, flags.min_values_per_parameter));
  ck(dnpeff_csr_shape(A, &n, &m, &nnz));
  std::cout << "n_cols after reduction: " << m << " [density=" << (double)nnz / (double)(n * m)
            << "]\n";

  bool wide_indices = read_wide && !(nnz > (int64_t)INT32_MAX);
  if (flags.index_width) wide_indices = flags.index_width == 64;
  std::cout << (wide_indices ? "Running NMF using 64 bit indices.\n" : "Running NMF using 32 bit indices.\n");

  std::cout << "Initializing NMF.\n";
  dnpeff_nmf* nmf = nullptr;
  // the matrix is only asked for its column map afterwards: the context may take its arrays
  ck(dnpeff_nmf_create_ex(A, flags.n_components, flags.eps, flags.seed, DNPEFF_NMF_CONSUME_MATRIX, &nmf));
  ck(dnpeff_nmf_init_factors(nmf));
  ck(dnpeff_sync());

  std::cout << "Running NMF.\n";
  auto t_start = std::chrono::high_resolution_clock::now();
  for (int step = 0; step < flags.max_iters; step++) {
    ck(dnpeff_nmf_step(nmf, 1));
    if (flags.log_every > 0 && (step + 1) % flags.log_every == 0) {
      ck(dnpeff_sync());
      auto t_end = std::chrono::high_resolution_clock::now();
      double elapsed_ms = std::chrono::duration<double, std::milli>(t_end - t_start).count();
      double loss = 0.0;
      ck(dnpeff_nmf_loss(nmf, &loss));
      // the ms/step figure ignores the time spent on the loss
      std::cout << "step " << step + 1 << ": " << (float)loss << " ["
                << elapsed_ms / (double)flags.log_every << " ms/step]\n";
      t_start = std::chrono::high_resolution_clock::now();
    }
  }
  ck(dnpeff_sync());

  const int r = flags.n_components;
  std::vector<float> W((size_t)n * r), H((size_t)r * m);
  std::vector<int32_t> kept((size_t)m);
  ck(dnpeff_nmf_get_W(nmf, W.data()));
  ck(dnpeff_nmf_get_H(nmf, H.data()));
  ck(dnpeff_csr_kept_indices(A, kept.data()));
  int64_t full = 0;
  ck(dnpeff_csr_full_dense_size(A, &full));

  std::cout << "Saving decomposition to file.\n";
  h5io::write_dense_decomposition(flags.output_path, n, r, m, W.data(), H.data(), kept.data(), full,
                                  wide_indices);
  dnpeff_nmf_destroy(nmf);
  dnpeff_csr_destroy(A);
  return 0;
}
