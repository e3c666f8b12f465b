// Sparseness projection of the columns of W (Hoyer 2004, "Non-negative matrix factorization with
// sparseness constraints", the projection operator of its section 3.3) in the form that
// DenseFactorSparsityContext::sparsifyF gives it
// (cc/cuda_d_npeff/src/nmf/sparse/dense_factor_sparsity_constraints.h:205-237, kernels
// cc/cuda_d_npeff/src/nmf/sparse/sparsity_constraint_kernels.h:16-141).  The reference builds the
// context when --sparsity_W is positive and never runs it: the one call is commented out
// (multi_mu_dense_factors_nmf1.h:161-162).  Here it is an entry point of its own that no loop calls.
//
// Every column x of W (n entries) is moved to s with sum(s) = l1, s >= 0:
//   s = x + (l1 - sum x) / n;  Y = all ones (the entries not yet fixed at zero)
//   repeat:  m = Y l1 / |Y|;  alpha from s.s, s.Y, |Y|;  s = m + alpha (s - m)
//            done when no column holds a negative entry
//            Y = 0 and s = 0 where s < 0;  s -= (sum s - l1) / |Y| on Y
// alpha is the reference's expression (sparsity_constraint_kernels.h:51-65), which differs from
// the root of Hoyer's quadratic by the term m.m under the square root: the columns end with
// ||s||^2 = l2^2 + l1^2 / |Y| instead of l2^2.  It is kept as the reference has it.
//
// The reference holds W column-major and takes the sums with cublasSgemv / strided-batched
// cublasSgemm in fp32, in an order it does not state.  W is row-major here; the per-column sums
// are accumulated in fp64 in a fixed order (row blocks, then blocks in ascending order) and
// rounded to fp32, everything else is the reference's fp32 arithmetic.  Columns that are no longer
// active keep their values, as in the reference (a column's mask is the number of negative
// entries its last step produced).
#include "dnpeff_internal.hpp"

namespace dn {

constexpr int HOYER_ROWS = 32;      // rows of W per workgroup in the passes that sum, at least
constexpr int HOYER_BLOCKS = 4096;  // and at most this many workgroups (partial sums per column)

// part[b][q][c] = sums over the rows of block b:  MODE 0: q0 = sum S
// MODE 1: q0 = sum Y, q1 = sum S S, q2 = sum S Y
// MODE 3 (after fixing the negative entries of active columns at zero): q0 = sum S, q1 = sum Y
template <int MODE>
__global__ void __launch_bounds__(256)
    k_hoyer_sums(int64_t n, int r, int64_t per, float* __restrict__ S, unsigned char* __restrict__ Y,
                 const float* __restrict__ active, double* __restrict__ part) {
  const int64_t row0 = (int64_t)blockIdx.x * per;
  const int64_t row1 = row0 + per < n ? row0 + per : n;
  for (int c = threadIdx.x; c < r; c += 256) {
    double q0 = 0.0, q1 = 0.0, q2 = 0.0;
    const bool act = MODE == 3 ? active[c] != 0.0f : true;
    for (int64_t i = row0; i < row1; i++) {
      const int64_t e = i * r + c;
      float s = S[e];
      if (MODE == 0) {
        q0 += (double)s;
      } else if (MODE == 1) {
        const float y = (float)Y[e];
        q0 += (double)y;
        q1 += (double)(s * s);
        q2 += (double)(s * y);
      } else {
        unsigned char y = Y[e];
        if (act) {  // kernel_updateYAndS, sparsity_constraint_kernels.h:91-113
          if (y && s < 0.0f) {
            y = 0;
            Y[e] = 0;
          }
          if (!y) {
            s = 0.0f;
            S[e] = 0.0f;
          }
        }
        q0 += (double)s;
        q1 += (double)y;
      }
    }
    double* p = part + (int64_t)blockIdx.x * 3 * r + c;
    p[0] = q0;
    p[r] = q1;
    p[2 * r] = q2;
  }
}

__device__ inline double hoyer_total(const double* part, int64_t blocks, int r, int q, int c) {
  double s = 0.0;
  for (int64_t b = 0; b < blocks; b++) s += part[(b * 3 + q) * r + c];
  return s;
}

// coef[c] after the pass of MODE:
//   0: (l1 - sum S) / n                       (kernel_computeInitialS, :16-27)
//   1: alpha; yy[c] = |Y|                     (kernel_computeAlpha, :41-66)
//   3: (sum S - l1) / |Y|                     (kernel_updateSLastStep, :116-141)
template <int MODE>
__global__ void __launch_bounds__(256)
    k_hoyer_coef(int64_t n, int r, int64_t blocks, const double* __restrict__ part, float l1, float l2,
                 float* __restrict__ coef, float* __restrict__ yy) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= r) return;
  if (MODE == 0) {
    const float sum = (float)hoyer_total(part, blocks, r, 0, c);
    coef[c] = (l1 - sum) / (float)n;
  } else if (MODE == 1) {
    const float YY = (float)hoyer_total(part, blocks, r, 0, c);
    const float SS = (float)hoyer_total(part, blocks, r, 1, c);
    const float SY = (float)hoyer_total(part, blocks, r, 2, c);
    const float L2 = sqrtf(l2 * l2);
    const float beta = l1 / YY;
    const float m2 = beta * beta * YY;
    const float ms = beta * SY;
    const float m_s_2 = fmaxf(1e-9f, beta * beta * YY + SS - 2.0f * beta * SY);
    coef[c] = (L2 * sqrtf(m_s_2) + m2 - ms) / m_s_2;
    yy[c] = YY;
  } else {
    const float sum_s = (float)hoyer_total(part, blocks, r, 0, c);
    const float sum_y = (float)hoyer_total(part, blocks, r, 1, c);
    coef[c] = (sum_s - l1) / sum_y;
  }
}

// S += coef[c], Y = 1
__global__ void __launch_bounds__(256)
    k_hoyer_start(int64_t total, int r, float* __restrict__ S, unsigned char* __restrict__ Y,
                  const float* __restrict__ coef) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    S[e] += coef[e % r];
    Y[e] = 1;
  }
}

// kernel_updateSAfterAlpha (:69-88) on the active columns, and the number of negative entries
// that it leaves in the rows of this block: neg[b][c] (0 for a column that is not active)
__global__ void __launch_bounds__(256)
    k_hoyer_step(int64_t n, int r, int64_t per, float* __restrict__ S, const unsigned char* __restrict__ Y,
                 const float* __restrict__ alpha, const float* __restrict__ yy,
                 const float* __restrict__ active, float l1, int* __restrict__ neg) {
  const int64_t row0 = (int64_t)blockIdx.x * per;
  const int64_t row1 = row0 + per < n ? row0 + per : n;
  for (int c = threadIdx.x; c < r; c += 256) {
    int count = 0;
    if (active[c] != 0.0f) {
      const float a = alpha[c], YY = yy[c];
      for (int64_t i = row0; i < row1; i++) {
        const int64_t e = i * r + c;
        const float m = (float)Y[e] * l1 / YY;
        const float s = m + a * (S[e] - m);
        S[e] = s;
        count += s < 0.0f;
      }
    }
    neg[(int64_t)blockIdx.x * r + c] = count;
  }
}

// active[c] = number of negative entries of column c; *any = 1 if there is one anywhere
// (updateAndReadActiveMask / isFinishedSync, dense_factor_sparsity_constraints.h:352-374)
__global__ void __launch_bounds__(256)
    k_hoyer_mask(int r, int64_t blocks, const int* __restrict__ neg, float* __restrict__ active,
                 int* __restrict__ any) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= r) return;
  int64_t count = 0;
  for (int64_t b = 0; b < blocks; b++) count += neg[b * r + c];
  active[c] = (float)count;
  if (count != 0) atomicOr(any, 1);
}

// kernel_updateSLastStep (:116-141): S -= coef[c] on the entries of active columns still in Y
__global__ void __launch_bounds__(256)
    k_hoyer_shift(int64_t total, int r, float* __restrict__ S, const unsigned char* __restrict__ Y,
                  const float* __restrict__ coef, const float* __restrict__ active) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    const int c = (int)(e % r);
    if (active[c] != 0.0f && Y[e]) S[e] -= coef[c];
  }
}

__global__ void k_hoyer_fill(int r, float* active, int* any) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c < r) active[c] = 1.0f;
  if (c == 0) *any = 0;
}

int sparsify_columns(int64_t n, int r, float* W, float l1, float l2, int* rounds_out) {
  DN_CHECK(n >= 1 && r >= 1 && r <= (1 << 20), "sparsify: %lld rows, rank %d", (long long)n, r);
  DN_CHECK(l1 > 0.0f, "sparsify: l1 norm %g is not positive (a null constraint)", (double)l1);
  const int64_t per = std::max<int64_t>(HOYER_ROWS, ceil_div(n, HOYER_BLOCKS));
  const int64_t blocks = ceil_div(n, per), total = n * r;
  dbuf<unsigned char> Y;
  dbuf<double> part;
  dbuf<float> coef, yy, active;
  dbuf<int> neg, any;
  DN_TRY(Y.alloc(total));
  DN_TRY(part.alloc(blocks * 3 * r));
  DN_TRY(coef.alloc(r));
  DN_TRY(yy.alloc(r));
  DN_TRY(active.alloc(r));
  DN_TRY(neg.alloc(blocks * r));
  DN_TRY(any.alloc(1));
  const dim3 b256(256), g_rows((unsigned)blocks), g_r((unsigned)ceil_div(r, 256));
  const dim3 g_flat((unsigned)std::min<int64_t>(ceil_div(total, 256), 65536));
  hipStream_t st = stream();
  hipLaunchKernelGGL(k_hoyer_fill, g_r, b256, 0, st, r, active.p, any.p);
  hipLaunchKernelGGL(k_hoyer_sums<0>, g_rows, b256, 0, st, n, r, per, W, Y.p, active.p, part.p);
  hipLaunchKernelGGL(k_hoyer_coef<0>, g_r, b256, 0, st, n, r, blocks, part.p, l1, l2, coef.p, yy.p);
  hipLaunchKernelGGL(k_hoyer_start, g_flat, b256, 0, st, total, r, W, Y.p, coef.p);
  DN_LAUNCH_CHECK();
  // every round that does not end the loop fixes at least one more entry of a column at zero
  int rounds = 0;
  for (;; rounds++) {
    DN_CHECK(rounds <= n, "sparsify: no end after %d rounds", rounds);
    hipLaunchKernelGGL(k_hoyer_sums<1>, g_rows, b256, 0, st, n, r, per, W, Y.p, active.p, part.p);
    hipLaunchKernelGGL(k_hoyer_coef<1>, g_r, b256, 0, st, n, r, blocks, part.p, l1, l2, coef.p, yy.p);
    hipLaunchKernelGGL(k_hoyer_step, g_rows, b256, 0, st, n, r, per, W, Y.p, coef.p, yy.p, active.p, l1, neg.p);
    hipLaunchKernelGGL(k_hoyer_mask, g_r, b256, 0, st, r, blocks, neg.p, active.p, any.p);
    DN_LAUNCH_CHECK();
    int host_any = 0;
    DN_HIP(hipMemcpyAsync(&host_any, any.p, sizeof(int), hipMemcpyDeviceToHost, st));
    DN_HIP(hipStreamSynchronize(st));
    if (!host_any) break;
    hipLaunchKernelGGL(k_hoyer_fill, dim3(1), dim3(1), 0, st, 0, active.p, any.p);  // any = 0
    hipLaunchKernelGGL(k_hoyer_sums<3>, g_rows, b256, 0, st, n, r, per, W, Y.p, active.p, part.p);
    hipLaunchKernelGGL(k_hoyer_coef<3>, g_r, b256, 0, st, n, r, blocks, part.p, l1, l2, coef.p, yy.p);
    hipLaunchKernelGGL(k_hoyer_shift, g_flat, b256, 0, st, total, r, W, Y.p, coef.p, active.p);
    DN_LAUNCH_CHECK();
  }
  if (rounds_out) *rounds_out = rounds + 1;
  return 0;
}

}  // namespace dn

DN_API int dnpeff_op_sparsify_columns(int64_t n_rows, int rank, float* W_nr, float l1_norm, float l2_norm,
                                      int* rounds) {
  DN_CHECK(W_nr != nullptr, "sparsify: null factor");
  return dn::sparsify_columns(n_rows, rank, W_nr, l1_norm, l2_norm, rounds);
}
