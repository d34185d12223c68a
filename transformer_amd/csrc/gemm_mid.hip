// C[M,N] = A[M,K] * W[N,K]^T for 17 to 64 rows (and for 9 to 16 over a long K), bfloat16 in,
// float32 accumulate: the matrix products of a decode step with a larger batch, still bound
// by reading W once from HBM, but with activations that are too large to be read again by
// every 16 columns.
//
// A workgroup of 8 waves owns 64 rows of W (64 output columns) and a range of K. Wave w
// takes the 16 rows (w % 4) of the tile and the half (w / 4) of the range: the four waves of a
// half share their chunk of the activations (up to 64 rows x 128 k) through LDS, which the
// workgroup fills with loads that cover whole cache lines, one chunk ahead, with one barrier
// per chunk. W comes in as in gemm_skinny.hip: whole lines, through 4 KB of LDS that belong
// to the wave alone, into the operand layout of v_mfma_f32_16x16x32_bf16; the 16-byte pieces
// of a row are permuted by the row number on the way in, so that operand reads meet no bank
// twice. The two halves are added through LDS at the end.
//
// With few column tiles (a square matrix has 64) the range of K is cut further among
// `splits` workgroups; each writes its partial result to its own [M, N] float32 plane and
// the reader adds the planes in order (the residual add of the next norm does).
//
// SWIGLU: W holds gate rows then up rows (N = 2*di); a workgroup takes 32 gate rows and the
// 32 up rows of the same columns and writes silu(gate) * up.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

union MidFrag {
  bf16x8 v;
  u32x4 q;
};

// what a load reads that has nothing to bring: a chunk past the end, k past K. Choosing the
// address costs nothing; choosing between the loaded value and zero would make every load
// be waited for where it is issued.
__device__ u32x4 mid_zeros = {0, 0, 0, 0};     // not const: a constant would make the loads generic

template <int MR, bool SWIGLU, bool TAIL, typename TC>
__global__ __launch_bounds__(512) void gemm_mid_kernel(const bf16_t* __restrict__ A, int lda,
                                                       const bf16_t* __restrict__ W, int ldw,
                                                       const float* __restrict__ bias,
                                                       TC* __restrict__ C, int ldc, size_t c_plane,
                                                       int M, int n_out, int K, int chunks_per_split) {
  constexpr int COLS = SWIGLU ? 32 : 64;
  // activations: [buffer][half of K][row][256 bytes]; afterwards the partial sums of the waves
  __shared__ __attribute__((aligned(16))) uint32_t a_lds[2][2][MR * 16 * 64];
  __shared__ __attribute__((aligned(16))) uint32_t w_stage[8][1024];
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int r = lane % 16, kb = lane / 16;
  const int sub = wave % 4, kh = wave / 4;
  const int n0 = blockIdx.x * COLS;

  // W: instruction t brings rows 4t + lane/16 of the wave's 16, 16 lanes per 256 bytes of a row
  const int lrow = lane / 16, lpiece = lane % 16;
  const bf16_t* wsrc[4];
  int gpiece[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int row = 4 * t + lrow;
    gpiece[t] = lpiece ^ row;
    int col, wrow;                       // output column and row of W
    if (SWIGLU) {
      col = n0 + 16 * (sub % 2) + row;
      wrow = (sub >= 2 ? n_out : 0) + col;
    } else {
      col = n0 + 16 * sub + row;
      wrow = col;
    }
    wsrc[t] = W + (size_t)(col < n_out ? wrow : 0) * ldw + gpiece[t] * 8;
  }
  // activations: the 256 threads of a half bring 16 rows per instruction, 16 threads per row
  const int th = threadIdx.x % 256;
  const int arow = th / 16, apiece = th % 16;
  const int agp = apiece ^ arow;
  const bf16_t* asrc[MR];
#pragma unroll
  for (int j = 0; j < MR; ++j) {
    const int row = 16 * j + arow;
    asrc[j] = A + (size_t)(row < M ? row : 0) * lda + agp * 8;
  }

  const int chunks = (K + 127) / 128;
  const int c_begin = blockIdx.y * chunks_per_split;
  const int c_end = c_begin + chunks_per_split < chunks ? c_begin + chunks_per_split : chunks;
  const int iters = (c_end - c_begin + 1) / 2;           // chunks of the longer half
  const int my_begin = c_begin + kh * iters;
  const int my_end = my_begin + iters < c_end ? my_begin + iters : c_end;

  floatx4 acc[MR];
#pragma unroll
  for (int j = 0; j < MR; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
  // Loads run well ahead of their use, because a workgroup is alone on its CU and only what
  // it has asked for hides the memory's latency: rows of W four chunks ahead (four register
  // sets), activations three chunks ahead (two register sets, then one of two LDS buffers).
  u32x4 areg[2][MR], wreg[4][4];
  // Every load is issued unconditionally, so that the waits can count loads. A chunk past the
  // half's last one and k past K (TAIL only) read zeros in both operands; rows past M or
  // n_out read row 0 and feed outputs that are never stored.
#define LOAD_A(aset, it_)                                                                     \
  do {                                                                                        \
    const int c_ = my_begin + (it_);                                                          \
    const bool ok_ = c_ < my_end && (!TAIL || c_ * 128 + agp * 8 < K);                        \
    _Pragma("unroll") for (int j = 0; j < MR; ++j)                                            \
        areg[aset][j] = *(ok_ ? reinterpret_cast<const u32x4*>(asrc[j] + c_ * 128) : &mid_zeros); \
  } while (0)
#define LOAD_W(set, it_)                                                                      \
  do {                                                                                        \
    const int c_ = my_begin + (it_);                                                          \
    _Pragma("unroll") for (int t = 0; t < 4; ++t) {                                           \
      const bool ok_ = c_ < my_end && (!TAIL || c_ * 128 + gpiece[t] * 8 < K);                \
      wreg[set][t] = __builtin_nontemporal_load(ok_ ? reinterpret_cast<const u32x4*>(wsrc[t] + c_ * 128) : (const u32x4*)&mid_zeros); \
    }                                                                                         \
  } while (0)
#define STORE_A(aset, buf)                                                                    \
  do {                                                                                        \
    _Pragma("unroll") for (int j = 0; j < MR; ++j)                                            \
        *reinterpret_cast<u32x4*>(&a_lds[buf][kh][(16 * j + arow) * 64 + apiece * 4]) = areg[aset][j]; \
  } while (0)
  // the chunk `it_` of both halves: its activations lie in LDS buffer it_ % 2, its rows of W
  // in register set it_ % 4; chunk it_ + 1's activations (register set (it_ + 1) % 2) go to
  // the other buffer meanwhile
#define STEP(S4, it_)                                                                         \
  do {                                                                                        \
    __syncthreads();                                                                          \
    STORE_A((S4 + 1) % 2, (S4 + 1) % 2);                                                      \
    __builtin_amdgcn_sched_barrier(0);                                                        \
    LOAD_A((S4 + 1) % 2, (it_) + 3);                                                          \
    _Pragma("unroll") for (int t = 0; t < 4; ++t)                                             \
        *reinterpret_cast<u32x4*>(&w_stage[wave][(4 * t + lrow) * 64 + lpiece * 4]) = wreg[S4][t]; \
    __builtin_amdgcn_sched_barrier(0);                                                        \
    LOAD_W(S4, (it_) + 4);                                                                    \
    __builtin_amdgcn_sched_barrier(0);                                                        \
    __builtin_amdgcn_wave_barrier();                                                          \
    _Pragma("unroll") for (int t = 0; t < 4; ++t) {                                           \
      MidFrag wf_;                                                                            \
      wf_.q = *reinterpret_cast<const u32x4*>(&w_stage[wave][r * 64 + ((4 * t + kb) ^ r) * 4]); \
      _Pragma("unroll") for (int j = 0; j < MR; ++j) {                                        \
        MidFrag af_;                                                                          \
        af_.q = *reinterpret_cast<const u32x4*>(&a_lds[S4 % 2][kh][(16 * j + r) * 64 + ((4 * t + kb) ^ r) * 4]); \
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf_.v, af_.v, acc[j], 0, 0, 0);      \
      }                                                                                       \
    }                                                                                         \
    __builtin_amdgcn_wave_barrier();                                                          \
  } while (0)

  LOAD_A(0, 0);
  LOAD_W(0, 0);
  LOAD_A(1, 1);
  LOAD_W(1, 1);
  LOAD_W(2, 2);
  LOAD_W(3, 3);
  STORE_A(0, 0);
  __builtin_amdgcn_sched_barrier(0);
  LOAD_A(0, 2);
  // four steps without a branch between them (a join would wait for every load in flight);
  // steps past the last chunk multiply zeros
  for (int it = 0; it < iters; it += 4) {
    STEP(0, it);
    STEP(1, it + 1);
    STEP(2, it + 2);
    STEP(3, it + 3);
  }
#undef STEP
#undef STORE_A
#undef LOAD_W
#undef LOAD_A

  // accumulator: register i of a lane is W row 4*(lane/16) + i of the wave's 16, activation
  // row lane % 16 of row tile j
  __syncthreads();
  float* red = reinterpret_cast<float*>(&a_lds[0][0][0]);          // [wave][row tile][256]
#pragma unroll
  for (int j = 0; j < MR; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[(wave * MR + j) * 256 + r * 16 + 4 * kb + i] = acc[j][i];
  __syncthreads();
  TC* cplane = C + (size_t)blockIdx.y * c_plane;
  for (int idx = threadIdx.x; idx < MR * 16 * COLS; idx += 512) {
    const int m = idx / COLS, col = idx % COLS;
    const int n = n0 + col;
    if (m >= M || n >= n_out) continue;
    const int s16 = col / 16, at = (m % 16) * 16 + col % 16, j = m / 16;
    if (SWIGLU) {
      float g = red[(s16 * MR + j) * 256 + at] + red[((s16 + 4) * MR + j) * 256 + at];
      float u = red[((s16 + 2) * MR + j) * 256 + at] + red[((s16 + 6) * MR + j) * 256 + at];
      // the unfused path stores the product in the output type before bias and activation
      if (sizeof(TC) == 2) {
        g = to_f32(from_f32<bf16_t>(g));
        u = to_f32(from_f32<bf16_t>(u));
      }
      if (bias) {
        g += bias[n];
        u += bias[n_out + n];
      }
      cplane[(size_t)m * ldc + n] = from_f32<TC>(g / (1.0f + expf(-g)) * u);
    } else {
      float v = red[(s16 * MR + j) * 256 + at] + red[((s16 + 4) * MR + j) * 256 + at];
      if (bias && blockIdx.y == 0) v += bias[n];
      cplane[(size_t)m * ldc + n] = from_f32<TC>(v);
    }
  }
}

// Workgroups that share a column tile's K. It depends on the weight's shape alone, so a
// row's result does not depend on what else is in the batch: about one workgroup per CU,
// at least four chunks of 128 each.
extern "C" int ta_gemm_mid_splits(int n_out, int K) {
  const int tiles = (n_out + 63) / 64, chunks = (K + 127) / 128;
  int s = 256 / tiles;
  if (s > 8) s = 8;
  if (s < 1) s = 1;
  // at least four chunks each, and none left empty by the rounding up of the others
  while (s > 1 && (chunks < 4 * s || (s - 1) * ((chunks + s - 1) / s) >= chunks)) --s;
  return s;
}

// out_dtype TA_BF16 or TA_F32. swiglu != 0: W is [2*n_out, K] (gate rows, then up rows), C is
// [M, n_out], bias has 2*n_out entries, splits must be 1. Otherwise W is [n_out, K] and, with
// splits > 1, C holds `splits` planes of c_plane elements each (float32), whose sum is the
// product (the bias is in plane 0).
extern "C" int ta_gemm_mid_bf16(hipStream_t stream, int out_dtype, int swiglu, const void* A, int lda,
                                const void* W, int ldw, const float* bias, void* C, int ldc,
                                long long c_plane, int M, int n_out, int K, int splits) {
  TA_REQUIRE(M >= 0 && M <= 64, "ta_gemm_mid_bf16: M=%d outside [0, 64]", M);
  TA_REQUIRE(n_out > 0 && K > 0, "ta_gemm_mid_bf16: bad sizes N=%d K=%d", n_out, K);
  TA_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && ldc >= n_out,
             "ta_gemm_mid_bf16: K and the row strides must be multiples of 8 (16-byte rows)");
  TA_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "ta_gemm_mid_bf16: operands must be 16-byte aligned");
  TA_REQUIRE(out_dtype == TA_BF16 || out_dtype == TA_F32, "ta_gemm_mid_bf16: unknown output dtype %d", out_dtype);
  const int chunks = (K + 127) / 128;
  TA_REQUIRE(splits >= 1 && splits <= chunks, "ta_gemm_mid_bf16: %d splits of %d chunks", splits, chunks);
  TA_REQUIRE(splits == 1 || (!swiglu && out_dtype == TA_F32 && c_plane >= (long long)(M - 1) * ldc + n_out),
             "ta_gemm_mid_bf16: partial planes need float32 output without activation and room for [M, N] each");
  if (M == 0) return 0;
  const int per = (chunks + splits - 1) / splits;
  TA_REQUIRE((splits - 1) * per < chunks, "ta_gemm_mid_bf16: %d splits leave one without work", splits);
  const int cols = swiglu ? 32 : 64;
  dim3 g((n_out + cols - 1) / cols, splits), b(512);
  const int mr = (M + 15) / 16;
  const bool tail = K % 128 != 0;
#define LAUNCH_T(MRV, SW, TL, TC)                                                                     \
  gemm_mid_kernel<MRV, SW, TL, TC><<<g, b, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, ldw,  \
                                                        bias, (TC*)C, ldc, (size_t)c_plane, M, n_out, K, per)
#define LAUNCH_TL(MRV, SW, TC) \
  if (tail) LAUNCH_T(MRV, SW, true, TC); else LAUNCH_T(MRV, SW, false, TC)
#define LAUNCH_MR(SW, TC)                      \
  switch (mr) {                                \
    case 1: LAUNCH_TL(1, SW, TC); break;       \
    case 2: LAUNCH_TL(2, SW, TC); break;       \
    case 3: LAUNCH_TL(3, SW, TC); break;       \
    default: LAUNCH_TL(4, SW, TC); break;      \
  }
  if (swiglu) {
    if (out_dtype == TA_BF16) { LAUNCH_MR(true, bf16_t) } else { LAUNCH_MR(true, float) }
  } else {
    if (out_dtype == TA_BF16) { LAUNCH_MR(false, bf16_t) } else { LAUNCH_MR(false, float) }
  }
#undef LAUNCH_MR
#undef LAUNCH_TL
#undef LAUNCH_T
  return ta_check_launch("ta_gemm_mid_bf16");
}
