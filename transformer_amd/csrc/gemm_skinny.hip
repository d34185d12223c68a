// C[M,N] = A[M,K] * W[N,K]^T for few rows (M <= 16), bfloat16 in, float32 accumulate:
// the matrix products of a decode step, which are bound by reading W once from HBM.
//
// A workgroup owns 16 rows of W (16 output columns). Its WAVES waves split K among
// them; the partial tiles are summed through LDS in wave order. The product runs on
// v_mfma_f32_16x16x32_bf16 with W as the first operand: a lane holds row (lane % 16) of
// the tile and 8 consecutive k. The instruction sums over its 32 k-slots whatever k they
// stand for, as long as both operands agree (slot (t, lane/16, e) = k0 + 32*t +
// 8*(lane/16) + e here).
//
// A CU is bound by the cache lines its loads touch long before HBM is: loading the
// operand layout directly touches 16 half lines per instruction, and the activations,
// which every workgroup reads again in that pattern, then cost half as much again as W
// at 8 rows. So W comes in with loads that cover whole lines (16 lanes per 256 bytes of a
// row, 4 rows per instruction) and goes through a 4 KB piece of LDS that belongs to the
// wave alone (no barrier) into the operand layout; the 16-byte pieces of a row are
// permuted by the row number on the way in, so the operand reads meet no bank twice.
//
// SWIGLU: W holds gate rows then up rows (N = 2*di); the workgroup computes both
// tiles for its 16 columns and writes silu(gate) * up, so the [M, 2*di] product never
// reaches memory.
//
// A product may also take over the RMS norm that stands between two products, so that a
// single-token step needs no kernel of its own for it. The product in front of the norm
// (SkinnyNorm::X set) adds its result to the float32 residual stream X, writes the new
// rows times the norm's weight as the next product's activations H, not yet scaled, and
// leaves the sum of squares of its 16 columns per row in out_parts[tile][16]. The product
// behind the norm (scale_parts set) sums these per row in tile order and multiplies its
// result by rsqrt(sum / size + eps): a row's scale factors out of the dot product.
#include "common.h"

struct SkinnyNorm {
  const float* scale_parts;   // [n_parts][16] sums of squares per row of A, or null
  int n_parts;
  float eps, inv_size;
  float* X;                   // [M][ldx] residual stream, or null
  int ldx;
  const float* norm_w;        // [n_out] weight of the norm that follows
  bf16_t* H;                  // [M][ldh] (X + product) * norm_w
  int ldh;
  float* out_parts;           // [tiles][16]
};

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

union Frag16 {
  bf16x8 v;
  u32x4 q;
};

// W is read once per step and is far larger than any cache: a non-temporal load streams it
// past the caches (a plain read-only stream reaches 7.2 TB/s on MI355X this way, 6.1 with
// ordinary loads). The activations, which every workgroup reads again, stay ordinary loads.
#define STREAM_LOAD(p) __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p))


template <int WAVES, bool SWIGLU, bool TAIL, typename TC, bool SCALE, bool FOLD>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ A, int lda,
                                                                 const bf16_t* __restrict__ W, int ldw,
                                                                 const float* __restrict__ bias,
                                                                 TC* __restrict__ C, int ldc, int M,
                                                                 int n_out, int K, SkinnyNorm nm) {
  constexpr int NT = SWIGLU ? 2 : 1;
  constexpr int SP = 16;       // partial sums of squares a thread asks for ahead of the product
  __shared__ float row_sq[WAVES][16];
  // per wave and tile: 16 rows x 128 k of W (4 KB) on their way from the coalesced load to
  // the operand layout; afterwards the same memory holds the partial sums
  __shared__ __attribute__((aligned(16))) uint32_t stage[WAVES][NT][1024];
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int r = lane % 16, kb = lane / 16;
  const int n0 = blockIdx.x * 16;
  // loading: instruction t brings rows 4t + lane/16; the 16 lanes of a row bring its 256
  // bytes, permuted by the row number so that the operand reads below meet no bank twice
  const int lrow = lane / 16, lpiece = lane % 16;
  const bf16_t* wsrc[NT][4];
  int gpiece[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int row = 4 * t + lrow;
    gpiece[t] = lpiece ^ row;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      wsrc[nt][t] = W + (size_t)(nt * n_out + (n0 + row < n_out ? n0 + row : 0)) * ldw + gpiece[t] * 8;
  }
  const bool a_ok = r < M;
  const bf16_t* arow = A + (size_t)(a_ok ? r : 0) * lda;
  // what the thread that stores output (m, n) adds to: asked for now, needed at the end
  // (dead threads and a product without a residual read a harmless address)
  const int em = (int)threadIdx.x / 16 < M ? threadIdx.x / 16 : 0;
  const int en = n0 + r < n_out ? n0 + r : 0;
  float x_old = 0.f, norm_w = 0.f;
  if (FOLD) {
    x_old = nm.X[(size_t)em * nm.ldx + en];
    norm_w = nm.norm_w[en];
  }
  floatx4 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int chunks = (K + 127) / 128;
  const int per_wave = (chunks + WAVES - 1) / WAVES;
  const int c_lo = wave * per_wave;
  const int c_hi = (c_lo + per_wave < chunks) ? c_lo + per_wave : chunks;
  // Two sets of staging registers take turns, and every load is issued unconditionally, so
  // that the waits can count loads: while one chunk is multiplied the next is in flight.
  // Rows past n_out or M read row 0 and only feed outputs that are never stored; k past K
  // (TAIL only) is zero in both operands; a load past the wave's last chunk, whose result
  // is not used, reads the same 16 bytes in every lane.
  u32x4 wreg[2][NT][4], areg[2][4];
#define LOAD_CHUNK(set, c_)                                                                   \
  do {                                                                                        \
    const int kc_ = (c_) * 128;                                                               \
    const bool live_ = (c_) < c_hi;      /* past the wave's last chunk: one cheap address */  \
    _Pragma("unroll") for (int t = 0; t < 4; ++t) {                                           \
      const bool wk_ = live_ && (!TAIL || kc_ + gpiece[t] * 8 < K);                           \
      const bool ak_ = live_ && (!TAIL || kc_ + t * 32 + kb * 8 < K);                         \
      _Pragma("unroll") for (int nt = 0; nt < NT; ++nt) {                                     \
        const u32x4 v_ = STREAM_LOAD(wk_ ? wsrc[nt][t] + kc_ : W);                            \
        wreg[set][nt][t] = (TAIL && !wk_) ? u32x4{0, 0, 0, 0} : v_;                           \
      }                                                                                       \
      const u32x4 a_ = *reinterpret_cast<const u32x4*>(ak_ ? arow + kc_ + t * 32 + kb * 8 : A); \
      areg[set][t] = (TAIL && !ak_) ? u32x4{0, 0, 0, 0} : a_;                                 \
    }                                                                                         \
  } while (0)
  // the wave reads what its other lanes wrote: LDS serves a wave's requests in order, and
  // the compiler may not move them across the wave barriers (a fence would also wait for
  // the loads in flight)
#define MUL_CHUNK(set)                                                                        \
  do {                                                                                        \
    _Pragma("unroll") for (int t = 0; t < 4; ++t)                                             \
        _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                     \
            *reinterpret_cast<u32x4*>(&stage[wave][nt][(4 * t + lrow) * 64 + lpiece * 4]) = wreg[set][nt][t]; \
    __builtin_amdgcn_wave_barrier();                                                          \
    _Pragma("unroll") for (int t = 0; t < 4; ++t)                                             \
        _Pragma("unroll") for (int nt = 0; nt < NT; ++nt) {                                   \
      Frag16 wf_, af_;                                                                        \
      wf_.q = *reinterpret_cast<const u32x4*>(&stage[wave][nt][r * 64 + ((4 * t + kb) ^ r) * 4]); \
      af_.q = areg[set][t];                                                                   \
      acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf_.v, af_.v, acc[nt], 0, 0, 0);      \
    }                                                                                         \
    __builtin_amdgcn_wave_barrier();                                                          \
  } while (0)
  // sums of squares of this thread's strip of tiles for row r: asked for now, before the
  // loads of W queue up behind them, and added up after the product (a wait in between
  // would hold the first chunks back); the order of the sum depends on the shapes alone
  float sqv[SCALE ? SP : 1];
  const int strip = threadIdx.x / 16;
  if (SCALE) {
#pragma unroll
    for (int i = 0; i < SP; ++i) {
      const int p = strip + i * WAVES * 4;
      const bool ok = a_ok && p < nm.n_parts;
      const float v = nm.scale_parts[ok ? p * 16 + r : 0];
      sqv[i] = ok ? v : 0.f;
    }
  }
  if (c_lo < c_hi) LOAD_CHUNK(0, c_lo);
  if (c_lo < c_hi) {
    int c = c_lo;
    // the body has no branch (a load whose only use is conditional gets moved into the
    // condition) and the scheduler may not reorder across the barriers, or it would sink
    // the loads below the products they should overlap
    for (; c + 1 < c_hi; c += 2) {
      LOAD_CHUNK(1, c + 1);
      __builtin_amdgcn_sched_barrier(0);
      MUL_CHUNK(0);
      __builtin_amdgcn_sched_barrier(0);
      LOAD_CHUNK(0, c + 2);
      __builtin_amdgcn_sched_barrier(0);
      MUL_CHUNK(1);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (c < c_hi) MUL_CHUNK(0);                  // an odd number of chunks: the last one
  }
#undef LOAD_CHUNK
#undef MUL_CHUNK
  if (SCALE) {
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < SP; ++i) sq += sqv[SCALE ? i : 0];
    if (a_ok)
      for (int p = strip + SP * WAVES * 4; p < nm.n_parts; p += WAVES * 4) sq += nm.scale_parts[p * 16 + r];
    sq += __shfl_xor(sq, 16, TA_WAVE);
    sq += __shfl_xor(sq, 32, TA_WAVE);
    if (lane < 16) row_sq[wave][r] = sq;
  }
  // accumulator: register i of a lane is W row 4*(lane/16) + i, activation row lane % 16
  float* red = reinterpret_cast<float*>(&stage[wave][0][0]);
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[nt * 1024 + r * 16 + 4 * kb + i] = acc[nt][i];
  __syncthreads();
  if (threadIdx.x >= 256) return;
  const int m = threadIdx.x / 16, n = n0 + threadIdx.x % 16;
  if (m >= M) return;                            // sixteen lanes of a row leave together
  const bool col_ok = n < n_out;
  float rs = 1.f;
  if (SCALE) {
    float sq = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) sq += row_sq[wv][m];
    rs = rsqrtf(sq * nm.inv_size + nm.eps);
  }
  float v[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    float sum = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) sum += reinterpret_cast<const float*>(&stage[wv][nt][0])[threadIdx.x];
    v[nt] = sum * rs;
    // the unfused path stores the product in the output type before bias and activation
    if (SWIGLU && sizeof(TC) == 2) v[nt] = to_f32(from_f32<bf16_t>(v[nt]));
    if (bias && col_ok) v[nt] += bias[nt * n_out + n];
  }
  float o = v[0];
  if (SWIGLU) o = v[0] / (1.0f + expf(-v[0])) * v[NT - 1];
  if (FOLD) {
    float xn = 0.f;
    if (col_ok) {
      xn = x_old + o;
      nm.X[(size_t)m * nm.ldx + n] = xn;
      nm.H[(size_t)m * nm.ldh + n] = from_f32<bf16_t>(xn * norm_w);
    }
    float sq = xn * xn;
    sq += __shfl_xor(sq, 8, 16);
    sq += __shfl_xor(sq, 4, 16);
    sq += __shfl_xor(sq, 2, 16);
    sq += __shfl_xor(sq, 1, 16);
    if (threadIdx.x % 16 == 0) nm.out_parts[(size_t)blockIdx.x * 16 + m] = sq;
    return;
  }
  if (col_ok) C[(size_t)m * ldc + n] = from_f32<TC>(o);
}

// Many output columns (from 640 tiles of 16 on, where it overtakes the kernel above) over a short
// K (at most 16 * CPW chunks of 128): sixteen waves split
// K, each keeps its slice of the activations in registers for the whole kernel, and the
// workgroup walks `tiles_per_wg` tiles of 16 rows of W one after the other. The
// activations are read once per workgroup instead of once per tile, and the fixed cost of a
// workgroup is spread over several tiles; the next tile's rows are in flight while the
// current one is multiplied. Partial sums of a tile go through one of two LDS buffers, so
// one barrier per tile is enough. SWIGLU: the walk alternates between the gate rows and the
// up rows of a tile's columns, and the threads that sum a tile keep the gate value until
// the up value arrives.
template <int CPW, bool TAIL, bool SWIGLU, typename TC>
__global__ __launch_bounds__(1024) void gemm_skinny_hold_kernel(const bf16_t* __restrict__ A, int lda,
                                                                const bf16_t* __restrict__ W, int ldw,
                                                                const float* __restrict__ bias,
                                                                TC* __restrict__ C, int ldc, int M,
                                                                int n_out, int K, int tiles_per_wg,
                                                                SkinnyNorm nm) {
  __shared__ __attribute__((aligned(16))) uint32_t stage[16][1024];
  __shared__ float red[2][16][256];
  __shared__ float row_sq[64][16];
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int r = lane % 16, kb = lane / 16;
  const int lrow = lane / 16, lpiece = lane % 16;
  const int tiles = (n_out + 15) / 16;
  const int tile0 = blockIdx.x * tiles_per_wg;
  const int ntile = tiles - tile0 < tiles_per_wg ? tiles - tile0 : tiles_per_wg;
  const int nstep = SWIGLU ? 2 * ntile : ntile;
  const int kbase = wave * CPW * 128;            // this wave's slice of K

  // activations: lane (r, kb), chunk cc, slot t holds A[r][kbase + cc*128 + t*32 + kb*8 ..+7]
  const bool a_ok = r < M;
  const bf16_t* arow = A + (size_t)(a_ok ? r : 0) * lda;
  u32x4 areg[CPW][4];
#pragma unroll
  for (int cc = 0; cc < CPW; ++cc)
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int k = kbase + cc * 128 + t * 32 + kb * 8;
      const bool ok = !TAIL || k < K;
      const u32x4 v = *reinterpret_cast<const u32x4*>(ok ? arow + k : A);
      areg[cc][t] = (TAIL && !ok) ? u32x4{0, 0, 0, 0} : v;
    }
  // W: instruction t brings rows 4t + lane/16 of the tile, 16 lanes per 256 bytes of a row
  int gpiece[4];
  bool wk[CPW][4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    gpiece[t] = lpiece ^ (4 * t + lrow);
#pragma unroll
    for (int cc = 0; cc < CPW; ++cc) wk[cc][t] = !TAIL || kbase + cc * 128 + gpiece[t] * 8 < K;
  }
  u32x4 wreg[CPW][4];
  // rows past n_out read row 0 and feed outputs that are never stored; a tile past the
  // workgroup's last reads the same 16 bytes in every lane (the loads stay unconditional
  // so that the waits can count them)
#define LOAD_TILE(i_, cc)                                                                     \
  do {                                                                                        \
    const bool live_ = (i_) < nstep;                                                          \
    _Pragma("unroll") for (int t = 0; t < 4; ++t) {                                           \
      const int it_ = SWIGLU ? (i_) >> 1 : (i_);                                              \
      const int row_ = (tile0 + it_) * 16 + 4 * t + lrow;                                     \
      const bf16_t* src_ = W + (size_t)((row_ < n_out ? row_ : 0) + ((SWIGLU && ((i_) & 1)) ? n_out : 0)) * ldw + \
                           kbase + (cc) * 128 + gpiece[t] * 8;                                \
      const u32x4 v_ = STREAM_LOAD((live_ && wk[cc][t]) ? src_ : W);                          \
      wreg[cc][t] = (TAIL && !wk[cc][t]) ? u32x4{0, 0, 0, 0} : v_;                            \
    }                                                                                         \
  } while (0)
#pragma unroll
  for (int cc = 0; cc < CPW; ++cc) LOAD_TILE(0, cc);
  if (nm.scale_parts) {
    // sums of squares of this thread's strip of tiles for row r; the first tile's barrier
    // stands between this and the threads that sum them up
    const int strip = threadIdx.x / 16;
    float sq = 0.f;
    if (a_ok)
      for (int p = strip; p < nm.n_parts; p += 64) sq += nm.scale_parts[p * 16 + r];
    row_sq[strip][r] = sq;
  }
  float gate = 0.f, rs = 1.f;
  for (int i = 0; i < nstep; ++i) {
    floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int cc = 0; cc < CPW; ++cc) {
#pragma unroll
      for (int t = 0; t < 4; ++t)
        *reinterpret_cast<u32x4*>(&stage[wave][(4 * t + lrow) * 64 + lpiece * 4]) = wreg[cc][t];
      __builtin_amdgcn_sched_barrier(0);
      LOAD_TILE(i + 1, cc);                      // in flight while this tile is multiplied
      __builtin_amdgcn_sched_barrier(0);
      // the wave reads what its other lanes wrote: LDS serves a wave's requests in order
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        Frag16 wf, af;
        wf.q = *reinterpret_cast<const u32x4*>(&stage[wave][r * 64 + ((4 * t + kb) ^ r) * 4]);
        af.q = areg[cc][t];
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf.v, af.v, acc, 0, 0, 0);
      }
      __builtin_amdgcn_wave_barrier();
    }
    // accumulator: register j of a lane is W row 4*(lane/16) + j, activation row lane % 16
    float* mine = &red[i & 1][wave][0];
#pragma unroll
    for (int j = 0; j < 4; ++j) mine[r * 16 + 4 * kb + j] = acc[j];
    __syncthreads();
    if (threadIdx.x < 256) {
      const int m = threadIdx.x / 16, n = (tile0 + (SWIGLU ? i >> 1 : i)) * 16 + threadIdx.x % 16;
      if (i == 0 && nm.scale_parts && m < M) {
        float sq = 0.f;
#pragma unroll
        for (int st = 0; st < 64; ++st) sq += row_sq[st][m];
        rs = rsqrtf(sq * nm.inv_size + nm.eps);
      }
      if (m < M && n < n_out) {
        float sum = 0.f;
#pragma unroll
        for (int wv = 0; wv < 16; ++wv) sum += red[i & 1][wv][threadIdx.x];
        sum *= rs;
        if (SWIGLU) {
          // the unfused path stores the product in the output type before bias and activation
          if (sizeof(TC) == 2) sum = to_f32(from_f32<bf16_t>(sum));
          if (bias) sum += bias[(i & 1) * n_out + n];
          if (i & 1)
            C[(size_t)m * ldc + n] = from_f32<TC>(gate / (1.0f + expf(-gate)) * sum);
          else
            gate = sum;
        } else {
          if (bias) sum += bias[n];
          C[(size_t)m * ldc + n] = from_f32<TC>(sum);
        }
      }
    }
  }
#undef LOAD_TILE
}

// Waves per workgroup for a product with n_out columns over K. It depends on the weight's
// shape alone, so a row's result does not depend on what else is in the batch. Measured on
// weights from 34 MB to 940 MB: with few tiles four waves with long runs of K each do
// best, with more tiles eight; sixteen never.
static int skinny_waves(int n_out, int K) {
  const int tiles = (n_out + 15) / 16;
  const int chunks = (K + 127) / 128;
  int w = tiles < 512 ? 4 : 8;
  while (w > 4 && chunks < 2 * w) w /= 2;     // at least two chunks per wave
  return w;
}

static int skinny_launch(hipStream_t stream, int out_dtype, int swiglu, const void* A, int lda,
                         const void* W, int ldw, const float* bias, void* C, int ldc, int M,
                         int n_out, int K, int waves, const SkinnyNorm& nm);

// out_dtype TA_BF16 or TA_F32. swiglu != 0: W is [2*n_out, K] (gate rows, then up rows),
// C is [M, n_out] and bias, if given, has 2*n_out entries. Otherwise W is [n_out, K].
// waves (4, 8 or 16) per workgroup; 0: chosen by the weight's shape.
extern "C" int ta_gemm_skinny_bf16(hipStream_t stream, int out_dtype, int swiglu, const void* A,
                                   int lda, const void* W, int ldw, const float* bias, void* C,
                                   int ldc, int M, int n_out, int K, int waves) {
  SkinnyNorm nm = {};
  return skinny_launch(stream, out_dtype, swiglu, A, lda, W, ldw, bias, C, ldc, M, n_out, K, waves, nm);
}

// The same product around an RMS norm (see the head of this file). scale_parts != null:
// A holds rows that are not yet scaled; [n_parts][16] sums of squares, `size` the norm's
// width. X != null (not with swiglu): the product (+ bias) is added to X [M][ldx] in place,
// H [M][ldh] gets the new rows times norm_w [n_out], out_parts [ceil(n_out/16)][16] their
// sums of squares; C is not written.
extern "C" int ta_gemm_skinny_norm_bf16(hipStream_t stream, int out_dtype, int swiglu, const void* A,
                                        int lda, const void* W, int ldw, const float* bias, void* C,
                                        int ldc, int M, int n_out, int K, int waves,
                                        const float* scale_parts, int n_parts, float eps, int size,
                                        float* X, int ldx, const float* norm_w, void* H, int ldh,
                                        float* out_parts) {
  SkinnyNorm nm = {};
  if (scale_parts) {
    TA_REQUIRE(n_parts > 0 && size > 0, "ta_gemm_skinny_norm_bf16: %d partial sums over a width of %d", n_parts, size);
    nm.scale_parts = scale_parts; nm.n_parts = n_parts; nm.eps = eps; nm.inv_size = 1.0f / (float)size;
  }
  if (X) {
    TA_REQUIRE(!swiglu, "ta_gemm_skinny_norm_bf16: the activation cannot be followed by the residual");
    TA_REQUIRE(norm_w && H && out_parts, "ta_gemm_skinny_norm_bf16: norm weight, activations and partial sums are needed");
    TA_REQUIRE(ldx >= n_out && ldh >= n_out, "ta_gemm_skinny_norm_bf16: rows of X or H are shorter than %d", n_out);
    nm.X = X; nm.ldx = ldx; nm.norm_w = norm_w; nm.H = (bf16_t*)H; nm.ldh = ldh; nm.out_parts = out_parts;
  } else {
    TA_REQUIRE(C != nullptr, "ta_gemm_skinny_norm_bf16: no output");
  }
  return skinny_launch(stream, out_dtype, swiglu, A, lda, W, ldw, bias, C, ldc, M, n_out, K, waves, nm);
}

static int skinny_launch(hipStream_t stream, int out_dtype, int swiglu, const void* A, int lda,
                         const void* W, int ldw, const float* bias, void* C, int ldc, int M,
                         int n_out, int K, int waves, const SkinnyNorm& nm) {
  TA_REQUIRE(M >= 0 && M <= 16, "ta_gemm_skinny_bf16: M=%d outside [0, 16]", M);
  TA_REQUIRE(n_out > 0 && K > 0, "ta_gemm_skinny_bf16: bad sizes N=%d K=%d", n_out, K);
  TA_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K && (nm.X || ldc >= n_out),
             "ta_gemm_skinny_bf16: K and the row strides must be multiples of 8 (16-byte rows)");
  TA_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "ta_gemm_skinny_bf16: operands must be 16-byte aligned");
  TA_REQUIRE(out_dtype == TA_BF16 || out_dtype == TA_F32, "ta_gemm_skinny_bf16: unknown output dtype %d", out_dtype);
  if (M == 0) return 0;
  const int tiles = (n_out + 15) / 16, chunks = (K + 127) / 128;
  if (waves == 0 && !nm.X && (swiglu ? 2 : 1) * tiles >= 640 && chunks <= 32) {
    // about one workgroup per CU and round, at most eight tiles each
    const int steps = (swiglu ? 2 : 1) * tiles;
    const int rounds = (steps + 2047) / 2048;
    int per = (steps + 256 * rounds - 1) / (256 * rounds);
    if (swiglu) per = (per + 1) / 2;             // tiles of columns; each is two steps
    const int cpw = chunks <= 16 ? 1 : 2;
    const bool tail = K % 128 != 0 || chunks != 16 * cpw;
    dim3 g((tiles + per - 1) / per), b(1024);
#define HOLD_SW(CPW, TL, SW, TC)                                                                    \
  gemm_skinny_hold_kernel<CPW, TL, SW, TC><<<g, b, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, \
                                                                ldw, bias, (TC*)C, ldc, M, n_out, K, per, nm)
#define HOLD(CPW, TL, TC) \
  if (swiglu) HOLD_SW(CPW, TL, true, TC); else HOLD_SW(CPW, TL, false, TC)
#define HOLD_BY(TC)                                                  \
  if (cpw == 1) { if (tail) { HOLD(1, true, TC); } else { HOLD(1, false, TC); } } \
  else { if (tail) { HOLD(2, true, TC); } else { HOLD(2, false, TC); } }
    if (out_dtype == TA_BF16) { HOLD_BY(bf16_t) } else { HOLD_BY(float) }
#undef HOLD_BY
#undef HOLD
#undef HOLD_SW
    return ta_check_launch("ta_gemm_skinny_bf16 (many columns)");
  }
  if (waves == 0) waves = skinny_waves(n_out, K);
  if (swiglu && waves > 8) waves = 8;          // two tiles per wave: 8 KB of LDS each
  TA_REQUIRE(waves == 4 || waves == 8 || waves == 16, "ta_gemm_skinny_bf16: waves must be 4, 8 or 16, got %d", waves);
  dim3 g((n_out + 15) / 16), b(waves * 64);
#define LAUNCH_T(WV, SW, TL, TC, SC, FO)                                                           \
  gemm_skinny_kernel<WV, SW, TL, TC, SC, FO><<<g, b, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, \
                                                                  ldw, bias, (TC*)C, ldc, M, n_out, K, nm)
#define LAUNCH_S(WV, SW, TL, TC) \
  if (nm.scale_parts) LAUNCH_T(WV, SW, TL, TC, true, false); else LAUNCH_T(WV, SW, TL, TC, false, false)
#define LAUNCH(WV, SW, TC) \
  if (K % 128 == 0) { LAUNCH_S(WV, SW, false, TC); } else { LAUNCH_S(WV, SW, true, TC); }
#define LAUNCH_FOLD(WV)                                                                  \
  if (K % 128 == 0) {                                                                    \
    if (nm.scale_parts) LAUNCH_T(WV, false, false, float, true, true); else LAUNCH_T(WV, false, false, float, false, true); \
  } else {                                                                               \
    if (nm.scale_parts) LAUNCH_T(WV, false, true, float, true, true); else LAUNCH_T(WV, false, true, float, false, true);   \
  }
#define BY_WAVES(SW, TC)                 \
  switch (waves) {                       \
    case 4: LAUNCH(4, SW, TC); break;    \
    case 8: LAUNCH(8, SW, TC); break;    \
    default: LAUNCH(16, SW, TC); break;  \
  }
  if (nm.X) {
    switch (waves) {
      case 4: LAUNCH_FOLD(4); break;
      case 8: LAUNCH_FOLD(8); break;
      default: LAUNCH_FOLD(16); break;
    }
  } else if (swiglu) {
    if (out_dtype == TA_BF16) { BY_WAVES(true, bf16_t) } else { BY_WAVES(true, float) }
  } else {
    if (out_dtype == TA_BF16) { BY_WAVES(false, bf16_t) } else { BY_WAVES(false, float) }
  }
#undef BY_WAVES
#undef LAUNCH_FOLD
#undef LAUNCH
#undef LAUNCH_S
#undef LAUNCH_T
  return ta_check_launch("ta_gemm_skinny_bf16");
}
