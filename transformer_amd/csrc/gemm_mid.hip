// C[M,N] = A[M,K] * W[N,K]^T for 17 to 64 rows (and for 9 to 16 over a long K), bfloat16 in,
// float32 accumulate: the matrix products of a decode step with a larger batch, still bound
// by reading W once from HBM, but with activations that are too large to be read again by
// every 16 columns.
//
// A workgroup of 8 waves owns 64 rows of W (64 output columns) and a range of K. Wave w
// takes the 16 rows (w % 4) of the tile and the half (w / 4) of the range (or, for a product
// in one plane with few column tiles, 32 columns with two waves side by side and four
// quarters of K): the four waves of a
// half share their chunk of the activations (up to 64 rows x 64 k) through LDS, which the
// workgroup fills with loads that cover whole cache lines, with one barrier per chunk. W
// comes in with loads that cover whole lines too (8 lanes per 128 bytes of a row, 8 rows per
// instruction) and goes through 2 KB of LDS that belong to the wave alone into the operand
// layout of v_mfma_f32_16x16x32_bf16; the 16-byte pieces are permuted by the row number on the
// way in, so that operand reads meet no bank twice. The two halves are added through LDS at
// the end, and the waves of the first half write the result from their registers.
//
// What decides the speed is how many workgroups a CU holds at once: one workgroup's waves
// stand still together at its start, its barriers and its end, and only other workgroups'
// loads fill that time. Chunks of 64 k (instead of 128) and short register queues keep a
// workgroup at 24 to 48 KB of LDS and under 128 registers, so that two to four fit; with
// 96 KB and 200 registers (one workgroup per CU) the same kernel took 30 % longer.
//
// With few column tiles (a square matrix has 64) the range of K is cut further among
// `splits` workgroups; each writes its partial result to its own [M, N] float32 plane and
// the reader adds the planes in order (the residual add of the next norm does).
//
// SWIGLU: W holds gate rows then up rows (N = 2*di) and the kernel writes silu(gate) * up.
// Up to 48 rows a workgroup owns 32 columns: waves 0, 1 of a half take their gate tiles, waves
// 2, 3 the up tiles, which they hand over through LDS at the end. At 49 to 64 rows a wave takes
// the gate tile and the up tile of its 16 columns (two tiles per wave: it reads each piece of
// the activations from LDS once for both) and a workgroup owns 64 columns: every workgroup
// reads all of the activations from L2 once, 512 KB at 64 rows, which costs as much as W
// when there are 448 workgroups.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

union MidFrag {
  bf16x8 v;
  u32x4 q;
};

// what a load reads that has nothing to bring: a chunk past the end, k past K. Choosing the
// address costs nothing; choosing between the loaded value and zero would make every load
// be waited for where it is issued.
__device__ u32x4 mid_zeros = {0, 0, 0, 0};     // not const: a constant would make the loads generic

#ifndef MID_DEPTH1
#define MID_DEPTH1 4      // chunks of W and of the activations that a wave asks for ahead
#endif
#ifndef MID_DEPTH2
#define MID_DEPTH2 2      // the same with two tiles per wave
#endif

// where piece `piece` (16 bytes = 8 k) of row `row` of a tile of 16 rows x 64 k lies in LDS, in
// 32-bit words: rows r and r + 8 share a line of 16 pieces, and the piece number is permuted
// by the line number, so that the 16 lanes that read one piece of all 16 rows meet 16 bank
// groups, as do the 8 lanes that write the 8 pieces of a row
__device__ __forceinline__ int mid_slot(int row, int piece) {
  const int q = row % 8;
  return (q * 16 + ((((row / 8) % 2) * 8 + piece) ^ q)) * 4;
}

template <int MR, int NTW, bool SWIGLU, bool TAIL, typename TC, int KW>
__global__ __launch_bounds__(512) void gemm_mid_kernel(const bf16_t* __restrict__ A, int lda,
                                                       const bf16_t* __restrict__ W, int ldw,
                                                       const float* __restrict__ bias,
                                                       TC* __restrict__ C, int ldc, size_t c_plane,
                                                       int M, int n_out, int K, int chunks_per_split,
                                                       int vec_ok) {
  static_assert(NTW == 1 || SWIGLU, "two tiles per wave are the gate and the up tile of its columns");
  static_assert(KW == 2 || (KW == 4 && !SWIGLU), "the range of K is halved, or quartered for a plain product");
  constexpr int CW = 8 / KW;                     // waves side by side along the columns
  constexpr int TP = 512 / KW;                   // threads that share a part of K
  constexpr int COLS = SWIGLU && NTW == 1 ? 32 : 16 * CW;   // output columns of a workgroup
  constexpr int AL = (MR * 128 + TP - 1) / TP;   // 16-byte loads of activations per thread and chunk
  constexpr int A_WORDS = 2 * KW * MR * 512;     // [buffer][part of K][row tile][512]
  constexpr int W_WORDS = 8 * NTW * 512;         // [wave][tile][512]
  constexpr int RED_WORDS = (KW - 1) * CW * NTW * MR * 256;  // partial sums of the later parts of K
  __shared__ __attribute__((aligned(16))) uint32_t lds[A_WORDS + W_WORDS > RED_WORDS ? A_WORDS + W_WORDS : RED_WORDS];
  uint32_t* const a_lds = lds;
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  uint32_t* const w_stage = lds + A_WORDS + wave * NTW * 512;
  const int r = lane % 16, kb = lane / 16;
  const int sub = wave % CW, kh = wave / CW;
  const int n0 = blockIdx.x * COLS;

  // W: instruction t brings rows 8t + lane/8 of the wave's 16, 8 lanes per 128 bytes of a row
  const int lrow = lane / 8, lpiece = lane % 8;
  const bf16_t* wsrc[NTW][2];
  int w_st[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int row = 8 * t + lrow;
    w_st[t] = mid_slot(row, lpiece);
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
      // output column and row of W; with SWIGLU the up row of a column lies n_out rows on,
      // in the wave's second tile or, with one tile per wave, in the tile of wave sub + 2
      const int col = n0 + 16 * (SWIGLU && NTW == 1 ? sub % 2 : sub) + row;
      const int wrow = (SWIGLU && NTW == 1 ? sub / 2 : nt) * n_out + col;
      wsrc[nt][t] = W + (size_t)(col < n_out ? wrow : 0) * ldw + lpiece * 8;
    }
  }
  // activations: the threads of a part of K bring TP / 8 rows per instruction, 8 threads per row
  const int th = threadIdx.x % TP;
  const bf16_t* asrc[AL];
  int a_st[AL];
  bool a_has[AL];
#pragma unroll
  for (int i = 0; i < AL; ++i) {
    const int row = th / 8 + (TP / 8) * i;
    a_has[i] = row < MR * 16;
    asrc[i] = A + (size_t)(row < M ? row : 0) * lda + lpiece * 8;
    a_st[i] = (row / 16) * 512 + mid_slot(row % 16, lpiece);
  }
  // operand reads: lane (r, kb) of multiplication t takes piece 4t + kb of row r
  int rd[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) rd[t] = mid_slot(r, 4 * t + kb);

  const int chunks = (K + 63) / 64;
  const int c_begin = blockIdx.y * chunks_per_split;
  const int c_end = c_begin + chunks_per_split < chunks ? c_begin + chunks_per_split : chunks;
  const int iters = (c_end - c_begin + KW - 1) / KW;     // chunks of the longest part
  const int my_begin = c_begin + kh * iters;
  const int my_end = my_begin + iters < c_end ? my_begin + iters : c_end;

  floatx4 acc[NTW][MR];
#pragma unroll
  for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
    for (int j = 0; j < MR; ++j) acc[nt][j] = floatx4{0.f, 0.f, 0.f, 0.f};
  // WD register sets each for the rows of W and for the activations hold the chunks after the
  // current one; a step first asks for the chunk WD steps ahead (into the set that the end of
  // the step before has emptied), then multiplies the current chunk out of LDS, and at its end
  // moves the next chunk from registers to LDS (the wave's own staging area for W, the other
  // of the two shared buffers for the activations). Loads complete in order, so both
  // operands are asked for equally far ahead: a wait for activations that were asked for late
  // would wait for all rows of W that were asked for before them.
  constexpr int WD = NTW == 2 ? MID_DEPTH2 : MID_DEPTH1;
  constexpr int UNR = WD % 2 ? 2 * WD : WD;             // steps until sets and buffers repeat
  u32x4 areg[WD][AL], wreg[WD][NTW][2];
  // Every load is issued unconditionally, so that the waits can count loads. A chunk past the
  // half's last one and k past K (TAIL only) read zeros in both operands; rows past M or
  // n_out read row 0 and feed outputs that are never stored.
#define LOAD_A(set, it_)                                                                      \
  do {                                                                                        \
    const int c_ = my_begin + (it_);                                                          \
    const bool ok_ = c_ < my_end && (!TAIL || c_ * 64 + lpiece * 8 < K);                      \
    _Pragma("unroll") for (int i = 0; i < AL; ++i)                                            \
        areg[set][i] = *(ok_ ? reinterpret_cast<const u32x4*>(asrc[i] + c_ * 64) : &mid_zeros); \
  } while (0)
#define LOAD_W(set, it_)                                                                      \
  do {                                                                                        \
    const int c_ = my_begin + (it_);                                                          \
    const bool ok_ = c_ < my_end && (!TAIL || c_ * 64 + lpiece * 8 < K);                      \
    _Pragma("unroll") for (int t = 0; t < 2; ++t)                                             \
        _Pragma("unroll") for (int nt = 0; nt < NTW; ++nt)                                    \
            wreg[set][nt][t] = __builtin_nontemporal_load(ok_ ? reinterpret_cast<const u32x4*>(wsrc[nt][t] + c_ * 64) : (const u32x4*)&mid_zeros); \
  } while (0)
#define STORE_A(set, buf)                                                                     \
  do {                                                                                        \
    _Pragma("unroll") for (int i = 0; i < AL; ++i)                                            \
        if ((MR * 128) % TP == 0 || i + 1 < AL || a_has[i])                                   \
          *reinterpret_cast<u32x4*>(&a_lds[((buf) * KW + kh) * MR * 512 + a_st[i]]) = areg[set][i]; \
  } while (0)
  // the wave reads what its other lanes wrote: LDS serves a wave's requests in order, so the
  // staging area can take the next chunk as soon as the reads of this one have been issued
#define STORE_W(set)                                                                          \
  do {                                                                                        \
    _Pragma("unroll") for (int nt = 0; nt < NTW; ++nt)                                        \
        _Pragma("unroll") for (int t = 0; t < 2; ++t)                                         \
            *reinterpret_cast<u32x4*>(&w_stage[nt * 512 + w_st[t]]) = wreg[set][nt][t];       \
  } while (0)
  // step it_ of both halves: chunk it_ lies in LDS (activations in buffer SA), register sets
  // SW + 1 .. hold the chunks behind it, set SW is free
#define STEP(SW, SA, it_)                                                                     \
  do {                                                                                        \
    __syncthreads();                                                                          \
    LOAD_A(SW, (it_) + WD);                                                                   \
    LOAD_W(SW, (it_) + WD);                                                                   \
    __builtin_amdgcn_sched_barrier(0);                                                        \
    _Pragma("unroll") for (int t = 0; t < 2; ++t) {                                           \
      MidFrag wf_[NTW];                                                                       \
      _Pragma("unroll") for (int nt = 0; nt < NTW; ++nt)                                      \
          wf_[nt].q = *reinterpret_cast<const u32x4*>(&w_stage[nt * 512 + rd[t]]);            \
      _Pragma("unroll") for (int j = 0; j < MR; ++j) {                                        \
        MidFrag af_;                                                                          \
        af_.q = *reinterpret_cast<const u32x4*>(&a_lds[(((SA) * KW + kh) * MR + j) * 512 + rd[t]]); \
        _Pragma("unroll") for (int nt = 0; nt < NTW; ++nt)                                    \
            acc[nt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf_[nt].v, af_.v, acc[nt][j], 0, 0, 0); \
      }                                                                                       \
    }                                                                                         \
    __builtin_amdgcn_sched_barrier(0);                                                        \
    __builtin_amdgcn_wave_barrier();                                                          \
    STORE_A((SW + 1) % WD, (SA + 1) % 2);                                                     \
    STORE_W((SW + 1) % WD);                                                                   \
    __builtin_amdgcn_wave_barrier();                                                          \
  } while (0)

#pragma unroll
  for (int d = 0; d < WD; ++d) {
    LOAD_A(d, d);
    LOAD_W(d, d);
  }
  STORE_A(0, 0);
  STORE_W(0);
  __builtin_amdgcn_wave_barrier();
  // UNR steps without a branch between them (a join would wait for every load in flight);
  // steps past the last chunk multiply zeros
  for (int it = 0; it < iters; it += UNR) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) STEP(u % WD, u % 2, it + u);
  }
#undef STEP
#undef STORE_W
#undef STORE_A
#undef LOAD_W
#undef LOAD_A

  // accumulator: register i of a lane is W row 4*(lane/16) + i of the wave's tile, activation
  // row lane % 16 of row tile j. The waves of the later parts of K hand theirs over.
  __syncthreads();
  floatx4* red = reinterpret_cast<floatx4*>(lds);          // [part - 1][column wave][tile][row tile][lane]
  if (kh > 0) {
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
      for (int j = 0; j < MR; ++j) red[((((kh - 1) * CW + sub) * NTW + nt) * MR + j) * 64 + lane] = acc[nt][j];
  }
  __syncthreads();
  if (SWIGLU && NTW == 1) {
    // the waves with the up tiles add the halves and hand the sums to the waves with the gates
    if (kh == 0 && sub >= 2) {
#pragma unroll
      for (int j = 0; j < MR; ++j) red[(sub * MR + j) * 64 + lane] += acc[0][j];
    }
    __syncthreads();
    if (kh == 1 || sub >= 2) return;
  }
  if (kh > 0) return;
  TC* cplane = C + (size_t)blockIdx.y * c_plane;
  const int n = n0 + 16 * sub + 4 * kb;                    // the lane's first of four columns
#pragma unroll
  for (int j = 0; j < MR; ++j) {
    const int m = 16 * j + r;
    float o[4];
    if (SWIGLU) {
      const floatx4 gs = acc[0][j] + red[((sub * NTW + 0) * MR + j) * 64 + lane];
      const floatx4 us = NTW == 2 ? acc[NTW - 1][j] + red[((sub * NTW + NTW - 1) * MR + j) * 64 + lane]
                                  : red[((sub + 2) * MR + j) * 64 + lane];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float g = gs[i], u = us[i];
        // the unfused path stores the product in the output type before bias and activation
        if (sizeof(TC) == 2) {
          g = to_f32(from_f32<bf16_t>(g));
          u = to_f32(from_f32<bf16_t>(u));
        }
        if (bias && n + i < n_out) {
          g += bias[n + i];
          u += bias[n_out + n + i];
        }
        o[i] = g / (1.0f + expf(-g)) * u;
      }
    } else {
      floatx4 vs = acc[0][j];                              // the parts are added in their order
#pragma unroll
      for (int part = 1; part < KW; ++part) vs += red[(((part - 1) * CW + sub) * MR + j) * 64 + lane];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        o[i] = vs[i];
        if (bias && blockIdx.y == 0 && n + i < n_out) o[i] += bias[n + i];
      }
    }
    if (m >= M) continue;
    TC* dst = cplane + (size_t)m * ldc + n;
    if (vec_ok && n + 3 < n_out) {
      if (sizeof(TC) == 4) {
        *reinterpret_cast<floatx4*>(dst) = floatx4{o[0], o[1], o[2], o[3]};
      } else {
        *reinterpret_cast<u32x2*>(dst) = u32x2{f32x2_to_bf16x2_bits(o[0], o[1]), f32x2_to_bf16x2_bits(o[2], o[3])};
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < n_out) dst[i] = from_f32<TC>(o[i]);
    }
  }
}

// Workgroups that share a column tile's K. It depends on the weight's shape alone, so a
// row's result does not depend on what else is in the batch: about one workgroup per CU,
// at least eight chunks of 64 each.
extern "C" int ta_gemm_mid_splits(int n_out, int K) {
  const int tiles = (n_out + 63) / 64, chunks = (K + 63) / 64;
  int s = 256 / tiles;
  if (s > TA_MAX_PLANES) s = TA_MAX_PLANES;
  if (s < 1) s = 1;
  // at least eight chunks each, and none left empty by the rounding up of the others
  while (s > 1 && (chunks < 8 * s || (s - 1) * ((chunks + s - 1) / s) >= chunks)) --s;
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
  const int chunks = (K + 63) / 64;
  TA_REQUIRE(splits >= 1 && splits <= (chunks + 1) / 2, "ta_gemm_mid_bf16: %d splits of %d chunks", splits, (chunks + 1) / 2);
  TA_REQUIRE(splits == 1 || (!swiglu && out_dtype == TA_F32 && c_plane >= (long long)(M - 1) * ldc + n_out),
             "ta_gemm_mid_bf16: partial planes need float32 output without activation and room for [M, N] each");
  if (M == 0) return 0;
  const int per = (chunks + splits - 1) / splits;
  TA_REQUIRE((splits - 1) * per < chunks, "ta_gemm_mid_bf16: %d splits leave one without work", splits);
  const int mr = (M + 15) / 16;
  // the activation: up to 48 rows one tile per wave and 32 columns per workgroup, so that
  // there are workgroups enough for several per CU; at 64 rows every workgroup reads 512 KB
  // of activations, and twice the columns per workgroup (two tiles per wave) halve that
  const int swt = mr == 4 ? 2 : 1;
  const int cols = (swiglu && swt == 1) ? 32 : 64;
  // a plain product in one plane with few column tiles (the qkv product: 96) quarters the range
  // of K inside a workgroup, which then owns 32 columns: twice the workgroups
  const int kw = (!swiglu && splits == 1 && (n_out + 63) / 64 <= 128) ? 4 : 2;
  dim3 g((n_out + cols - 1) / cols, splits), b(512);
  if (kw == 4) g.x = (n_out + 31) / 32;
  const bool tail = K % 64 != 0;
  // four columns of a lane go out in one store when every row and plane keeps them aligned
  const size_t esz = out_dtype == TA_F32 ? 4 : 2;
  const int vec_ok = ((uintptr_t)C % (4 * esz)) == 0 && ldc % 4 == 0 && (splits == 1 || c_plane % 4 == 0);
#define LAUNCH_K(MRV, SW, TL, TC, KWV)                                                                     \
  gemm_mid_kernel<MRV, (SW && MRV == 4 ? 2 : 1), SW, TL, TC, KWV><<<g, b, 0, stream>>>(                     \
      (const bf16_t*)A, lda, (const bf16_t*)W, ldw, bias, (TC*)C, ldc, (size_t)c_plane, M, n_out, K, per, vec_ok)
#define LAUNCH_T(MRV, SW, TL, TC) \
  if (!SW && kw == 4) LAUNCH_K(MRV, SW, TL, TC, (SW ? 2 : 4)); else LAUNCH_K(MRV, SW, TL, TC, 2)
#define LAUNCH_TL(MRV, SW, TC) \
  if (tail) { LAUNCH_T(MRV, SW, true, TC); } else { LAUNCH_T(MRV, SW, false, TC); }
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
#undef LAUNCH_K
  return ta_check_launch("ta_gemm_mid_bf16");
}
