// C[M,N] = A[M,K] * W[N,K]^T for few rows (M <= 64), bfloat16 in, float32 accumulate:
// the matrix products of a decode step, which are bound by reading W once from HBM.
//
// A workgroup owns 16 rows of W (16 output columns). Its four waves split K into
// quarters, so a wave streams 16 contiguous row segments; partial tiles are summed
// through LDS. The product runs on v_mfma_f32_16x16x32_bf16 with W as the first
// operand: a lane holds row (lane % 16) of the tile and 8 consecutive k, which is a
// 16-byte load straight from the row-major weight. The instruction sums over its 32
// k-slots whatever k they stand for, as long as both operands agree, so a lane takes
// 64 contiguous bytes of its row per 128-k chunk (slot (t, lane/16, e) = k0 +
// 32*(lane/16) + 8*t + e) and the activations are gathered the same way.
//
// SWIGLU: W holds gate rows then up rows (N = 2*di); the workgroup computes both
// tiles for its 16 columns and writes silu(gate) * up, so the [M, 2*di] product never
// reaches memory.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

union Frag16 {
  bf16x8 v;
  uint4 q;
};

__device__ __forceinline__ uint4 load16_or_zero(const bf16_t* p, bool ok) {
  return ok ? *reinterpret_cast<const uint4*>(p) : make_uint4(0, 0, 0, 0);
}

template <int MT, bool SWIGLU, typename TC>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16_t* __restrict__ A, int lda,
                                                          const bf16_t* __restrict__ W, int ldw,
                                                          const float* __restrict__ bias,
                                                          TC* __restrict__ C, int ldc, int M,
                                                          int n_out, int K) {
  constexpr int NT = SWIGLU ? 2 : 1;
  __shared__ float red[4][NT][MT][256];
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int r = lane % 16, kb = lane / 16;
  const int n0 = blockIdx.x * 16;
  const bool row_ok = n0 + r < n_out;
  const bf16_t* wrow[NT];
  wrow[0] = W + (size_t)(row_ok ? n0 + r : 0) * ldw;
  if (SWIGLU) wrow[NT - 1] = W + (size_t)(n_out + (row_ok ? n0 + r : 0)) * ldw;
  const bf16_t* arow[MT];
  bool a_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    a_ok[mt] = mt * 16 + r < M;
    arow[mt] = A + (size_t)(a_ok[mt] ? mt * 16 + r : 0) * lda;
  }
  floatx4 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int chunks = (K + 127) / 128;
  const int per_wave = (chunks + 3) / 4;
  const int c_lo = wave * per_wave;
  const int c_hi = (c_lo + per_wave < chunks) ? c_lo + per_wave : chunks;
#pragma unroll 2
  for (int c = c_lo; c < c_hi; ++c) {
    const int k0 = c * 128 + kb * 32;
    Frag16 wf[NT][4], af[MT][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const bool k_ok = k0 + t * 8 < K;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) wf[nt][t].q = load16_or_zero(wrow[nt] + k0 + t * 8, row_ok && k_ok);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) af[mt][t].q = load16_or_zero(arow[mt] + k0 + t * 8, a_ok[mt] && k_ok);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[nt][t].v, af[mt][t].v, acc[nt][mt], 0, 0, 0);
  }
  // accumulator: register i of a lane is W row 4*(lane/16) + i, activation row lane % 16
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][nt][mt][r * 16 + 4 * kb + i] = acc[nt][mt][i];
  __syncthreads();
  const int ml = threadIdx.x / 16, nl = threadIdx.x % 16;
  const int n = n0 + nl;
  if (n >= n_out) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + ml;
    if (m >= M) continue;
    float v[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      v[nt] = (red[0][nt][mt][threadIdx.x] + red[1][nt][mt][threadIdx.x]) +
              (red[2][nt][mt][threadIdx.x] + red[3][nt][mt][threadIdx.x]);
      // the unfused path stores the product in the output type before bias and activation
      if (SWIGLU && sizeof(TC) == 2) v[nt] = to_f32(from_f32<bf16_t>(v[nt]));
      if (bias) v[nt] += bias[nt * n_out + n];
    }
    float o = v[0];
    if (SWIGLU) o = v[0] / (1.0f + expf(-v[0])) * v[NT - 1];
    C[(size_t)m * ldc + n] = from_f32<TC>(o);
  }
}

// out_dtype TA_BF16 or TA_F32. swiglu != 0: W is [2*n_out, K] (gate rows, then up rows),
// C is [M, n_out] and bias, if given, has 2*n_out entries. Otherwise W is [n_out, K].
extern "C" int ta_gemm_skinny_bf16(hipStream_t stream, int out_dtype, int swiglu, const void* A,
                                   int lda, const void* W, int ldw, const float* bias, void* C,
                                   int ldc, int M, int n_out, int K) {
  TA_REQUIRE(M >= 0 && M <= 64, "ta_gemm_skinny_bf16: M=%d outside [0, 64]", M);
  TA_REQUIRE(n_out > 0 && K > 0, "ta_gemm_skinny_bf16: bad sizes N=%d K=%d", n_out, K);
  TA_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldc >= n_out,
             "ta_gemm_skinny_bf16: K and the row strides must be multiples of 8 (16-byte rows)");
  TA_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "ta_gemm_skinny_bf16: operands must be 16-byte aligned");
  TA_REQUIRE(out_dtype == TA_BF16 || out_dtype == TA_F32, "ta_gemm_skinny_bf16: unknown output dtype %d", out_dtype);
  if (M == 0) return 0;
  dim3 g((n_out + 15) / 16), b(256);
  const int mt = (M + 15) / 16;
#define LAUNCH(MTV, SW, TC)                                                                    \
  gemm_skinny_kernel<MTV, SW, TC><<<g, b, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, ldw, \
                                                       bias, (TC*)C, ldc, M, n_out, K)
#define BY_MT(SW, TC)                        \
  switch (mt) {                              \
    case 1: LAUNCH(1, SW, TC); break;        \
    case 2: LAUNCH(2, SW, TC); break;        \
    case 3: LAUNCH(3, SW, TC); break;        \
    default: LAUNCH(4, SW, TC); break;       \
  }
  if (swiglu) {
    if (out_dtype == TA_BF16) BY_MT(true, bf16_t) else BY_MT(true, float)
  } else {
    if (out_dtype == TA_BF16) BY_MT(false, bf16_t) else BY_MT(false, float)
  }
#undef BY_MT
#undef LAUNCH
  return ta_check_launch("ta_gemm_skinny_bf16");
}
