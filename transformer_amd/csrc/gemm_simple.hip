// C[M,N] = A[M,K] * W[N,K]^T (+ bias[N]) with float32 accumulation on the vector
// ALU: the matrix product of the true 32-bit path, and the fallback for storage
// types and shapes that no faster kernel takes.
//
// Every output element is one chain of fused multiply-adds over k = 0..K-1 in
// ascending order, whatever M, N or the tiling: a row of A gives the same bits
// alone or inside any batch.
#include "common.h"

#define BM 64
#define BN 64
#define BK 16

template <typename T, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_simple_kernel(const T* __restrict__ A, int lda,
                                                          const TW* __restrict__ W, int ldw,
                                                          const float* __restrict__ bias,
                                                          TC* __restrict__ C, int ldc, int M,
                                                          int N, int K) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  // each thread stages 4 elements of A and 4 of W per k-slab: row = tid / 4, k = (tid % 4) * 4 ..
  const int lr = threadIdx.x / 4, lk = (threadIdx.x % 4) * 4;
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      const int am = m0 + lr, wn = n0 + lr;
      As[lk + e][lr] = (am < M && k < K) ? to_f32(A[(size_t)am * lda + k]) : 0.f;
      Ws[lk + e][lr] = (wn < N && k < K) ? to_f32(W[(size_t)wn * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += bias[n];
      C[(size_t)m * ldc + n] = from_f32<TC>(v);
    }
  }
}

// in_dtype: type of A; w_dtype: type of W (a bfloat16 engine keeps a matrix that its file
// stores in 32 bits as it is: bfloat16 A with float32 W); out_dtype: type of C.
extern "C" int ta_gemm_simple(hipStream_t stream, int in_dtype, int w_dtype, int out_dtype,
                              const void* A, int lda, const void* W, int ldw, const float* bias,
                              void* C, int ldc, int M, int N, int K) {
  TA_REQUIRE(M >= 0 && N > 0 && K > 0, "ta_gemm_simple: bad sizes M=%d N=%d K=%d", M, N, K);
  TA_REQUIRE(lda >= K && ldw >= K && ldc >= N, "ta_gemm_simple: leading dimensions too small");
  if (M == 0) return 0;
  dim3 g((N + BN - 1) / BN, (M + BM - 1) / BM), b(256);
  TA_REQUIRE(g.y <= 65535, "ta_gemm_simple: M=%d too large for one launch", M);
#define LAUNCH(T, TW, TC)                                                                        \
  gemm_simple_kernel<T, TW, TC><<<g, b, 0, stream>>>((const T*)A, lda, (const TW*)W, ldw, bias,   \
                                                     (TC*)C, ldc, M, N, K)
  if (in_dtype == TA_F32 && w_dtype == TA_F32 && out_dtype == TA_F32) LAUNCH(float, float, float);
  else if (in_dtype == TA_BF16 && w_dtype == TA_BF16 && out_dtype == TA_BF16) LAUNCH(bf16_t, bf16_t, bf16_t);
  else if (in_dtype == TA_BF16 && w_dtype == TA_BF16 && out_dtype == TA_F32) LAUNCH(bf16_t, bf16_t, float);
  else if (in_dtype == TA_BF16 && w_dtype == TA_F32 && out_dtype == TA_BF16) LAUNCH(bf16_t, float, bf16_t);
  else if (in_dtype == TA_BF16 && w_dtype == TA_F32 && out_dtype == TA_F32) LAUNCH(bf16_t, float, float);
  else return ta_fail("ta_gemm_simple: unsupported dtypes a=%d w=%d out=%d", in_dtype, w_dtype, out_dtype);
#undef LAUNCH
  return ta_check_launch("ta_gemm_simple");
}
