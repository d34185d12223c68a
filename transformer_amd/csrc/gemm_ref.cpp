// Plain twin of the matrix products (gemm_simple.hip, gemm_skinny.hip, gemm_mid.hip):
// C[M, N] = A[M, K] . W[N, K]^T (+ bias), sums in double; with swiglu, W holds gate rows then
// up rows and C[M, N] = silu(A . gate^T + b_gate) * (A . up^T + b_up).
#include "ref_common.h"

#include <cmath>

// The weights are stored [rows out, k] and multiplied transposed, as the reference's
// mat_mul calls are set up (models/llama/common/src/compute.rs:425-455); gate and up are
// the two halves of the merged matrix's rows (lib.rs:154-157, compute.rs:286).
extern "C" int ta_ref_gemm(const float* a, int lda, const float* w, int ldw, const float* bias, float* c,
                           int ldc, int M, int n_out, int K, int swiglu) {
  TA_REF_REQUIRE(M >= 0 && n_out > 0 && K > 0 && lda >= K && ldw >= K && ldc >= n_out, "ta_ref_gemm: bad sizes");
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < n_out; ++n) {
      double g = 0.0, u = 0.0;
      for (int k = 0; k < K; ++k) {
        g += (double)a[(size_t)m * lda + k] * w[(size_t)n * ldw + k];
        if (swiglu) u += (double)a[(size_t)m * lda + k] * w[(size_t)(n_out + n) * ldw + k];
      }
      if (bias) {
        g += bias[n];
        if (swiglu) u += bias[n_out + n];
      }
      c[(size_t)m * ldc + n] = (float)(swiglu ? g / (1.0 + std::exp(-g)) * u : g);
    }
  return 0;
}
