// C[M,N] = A[M,K] * W[N,K]^T for few rows (M <= 16), bfloat16 in, float32 accumulate:
// the matrix products of a decode step, which are bound by reading W once from HBM.
//
// A workgroup owns 16 rows of W (16 output columns). Its WAVES waves split K among
// them, so a wave streams 16 contiguous row segments; the partial tiles are summed
// through LDS in wave order. The product runs on v_mfma_f32_16x16x32_bf16 with W as the first
// operand: a lane holds row (lane % 16) of the tile and 8 consecutive k, which is a
// 16-byte load straight from the row-major weight. The instruction sums over its 32
// k-slots whatever k they stand for, as long as both operands agree. The four lanes of
// a row read 64 contiguous bytes in one instruction (slot (t, lane/16, e) = k0 + 32*t +
// 8*(lane/16) + e), so an instruction touches 16 half cache lines instead of 64 separate
// 16-byte pieces: a CU is bound by the lines it can request long before HBM is. For the
// same reason the activations, which every workgroup reads again in the same pattern,
// are what the time grows with: one row costs nothing, sixteen rows half as much again.
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

template <int WAVES, bool SWIGLU, typename TC>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ A, int lda,
                                                                 const bf16_t* __restrict__ W, int ldw,
                                                                 const float* __restrict__ bias,
                                                                 TC* __restrict__ C, int ldc, int M,
                                                                 int n_out, int K) {
  constexpr int NT = SWIGLU ? 2 : 1;
  __shared__ float red[WAVES][NT][256];
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int r = lane % 16, kb = lane / 16;
  const int n0 = blockIdx.x * 16;
  const bool row_ok = n0 + r < n_out;
  const bf16_t* wrow[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) wrow[nt] = W + (size_t)(nt * n_out + (row_ok ? n0 + r : 0)) * ldw;
  const bool a_ok = r < M;
  const bf16_t* arow = A + (size_t)(a_ok ? r : 0) * lda;
  floatx4 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int chunks = (K + 127) / 128;
  const int per_wave = (chunks + WAVES - 1) / WAVES;
  const int c_lo = wave * per_wave;
  const int c_hi = (c_lo + per_wave < chunks) ? c_lo + per_wave : chunks;
#pragma unroll 2
  for (int c = c_lo; c < c_hi; ++c) {
    const int k0 = c * 128 + kb * 8;
    Frag16 wf[NT][4], af[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const bool k_ok = k0 + t * 32 < K;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) wf[nt][t].q = load16_or_zero(wrow[nt] + k0 + t * 32, row_ok && k_ok);
      af[t].q = load16_or_zero(arow + k0 + t * 32, a_ok && k_ok);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[nt][t].v, af[t].v, acc[nt], 0, 0, 0);
  }
  // accumulator: register i of a lane is W row 4*(lane/16) + i, activation row lane % 16
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][nt][r * 16 + 4 * kb + i] = acc[nt][i];
  __syncthreads();
  if (threadIdx.x >= 256) return;
  const int m = threadIdx.x / 16, n = n0 + threadIdx.x % 16;
  if (m >= M || n >= n_out) return;
  float v[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    float sum = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) sum += red[wv][nt][threadIdx.x];
    v[nt] = sum;
    // the unfused path stores the product in the output type before bias and activation
    if (SWIGLU && sizeof(TC) == 2) v[nt] = to_f32(from_f32<bf16_t>(v[nt]));
    if (bias) v[nt] += bias[nt * n_out + n];
  }
  float o = v[0];
  if (SWIGLU) o = v[0] / (1.0f + expf(-v[0])) * v[NT - 1];
  C[(size_t)m * ldc + n] = from_f32<TC>(o);
}

// Waves per workgroup for a product with n_out columns over K. It depends on the weight's
// shape alone, so a row's result does not depend on what else is in the batch. Measured:
// sixteen waves keep enough loads in flight per CU at every width; a narrow weight (one
// workgroup per CU or fewer) does as well with eight.
static int skinny_waves(int n_out, int K) {
  const int tiles = (n_out + 15) / 16;
  const int chunks = (K + 127) / 128;
  int w = tiles > 256 ? 16 : 8;
  while (w > 4 && chunks < 2 * w) w /= 2;     // at least two chunks per wave
  return w;
}

// out_dtype TA_BF16 or TA_F32. swiglu != 0: W is [2*n_out, K] (gate rows, then up rows),
// C is [M, n_out] and bias, if given, has 2*n_out entries. Otherwise W is [n_out, K].
// waves (4, 8 or 16) per workgroup; 0: chosen by the weight's shape.
extern "C" int ta_gemm_skinny_bf16(hipStream_t stream, int out_dtype, int swiglu, const void* A,
                                   int lda, const void* W, int ldw, const float* bias, void* C,
                                   int ldc, int M, int n_out, int K, int waves) {
  TA_REQUIRE(M >= 0 && M <= 16, "ta_gemm_skinny_bf16: M=%d outside [0, 16]", M);
  TA_REQUIRE(n_out > 0 && K > 0, "ta_gemm_skinny_bf16: bad sizes N=%d K=%d", n_out, K);
  TA_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldc >= n_out,
             "ta_gemm_skinny_bf16: K and the row strides must be multiples of 8 (16-byte rows)");
  TA_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "ta_gemm_skinny_bf16: operands must be 16-byte aligned");
  TA_REQUIRE(out_dtype == TA_BF16 || out_dtype == TA_F32, "ta_gemm_skinny_bf16: unknown output dtype %d", out_dtype);
  if (M == 0) return 0;
  if (waves == 0) waves = skinny_waves(n_out, K);
  TA_REQUIRE(waves == 4 || waves == 8 || waves == 16, "ta_gemm_skinny_bf16: waves must be 4, 8 or 16, got %d", waves);
  dim3 g((n_out + 15) / 16), b(waves * 64);
#define LAUNCH(WV, SW, TC)                                                                      \
  gemm_skinny_kernel<WV, SW, TC><<<g, b, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, ldw, \
                                                      bias, (TC*)C, ldc, M, n_out, K)
#define BY_WAVES(SW, TC)                 \
  switch (waves) {                       \
    case 4: LAUNCH(4, SW, TC); break;    \
    case 8: LAUNCH(8, SW, TC); break;    \
    default: LAUNCH(16, SW, TC); break;  \
  }
  if (swiglu) {
    if (out_dtype == TA_BF16) { BY_WAVES(true, bf16_t) } else { BY_WAVES(true, float) }
  } else {
    if (out_dtype == TA_BF16) { BY_WAVES(false, bf16_t) } else { BY_WAVES(false, float) }
  }
#undef BY_WAVES
#undef LAUNCH
  return ta_check_launch("ta_gemm_skinny_bf16");
}
