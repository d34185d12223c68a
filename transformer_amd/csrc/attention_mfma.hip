// Causal grouped-query attention over the paged cache on the matrix cores
// (v_mfma_f32_32x32x16_bf16), bfloat16 storage, float32 softmax and accumulation.
//
// A wave owns 32 "rows" of one (sequence, kv head): row = (query token, query head
// inside the kv head's group). It works on transposed tiles so that every operand is
// read from memory in the register layout the instruction wants:
//
//   S^T[key, row] = sum_d K[key, d] * Q[row, d]      A = K page rows,   B = Q rows
//   O^T[d, row]  += sum_key V^T[d, key] * P^T[key, row]   A = V^T page rows, B = P^T
//
// A lane holds column `row = lane % 32` of S^T and of O^T, so the softmax of a row is
// a reduction inside a lane plus one exchange with lane ^ 32, and the rescaling of O^T
// is a per-lane multiply. The accumulator layout of the instruction puts keys
// 8*(r/4) + 4*(lane/32) + r%4 (r = register 0..15) of a 32-key tile into a lane; the
// value operand of the second product is gathered in that same order (two 8-byte runs
// of 4 consecutive keys), so no data is moved between lanes.
//
// Two kernels share this core. "rows": every wave has its own 32 rows and walks all
// their keys (prompts). "keys": the four waves of a workgroup share one tile of rows
// and walk different pages of a slice of the keys; slices are merged by a second
// kernel (single tokens, where the keys are the only parallelism there is). The merge
// is a kernel of its own on purpose: a device-wide fence inside the first kernel, which
// a last-workgroup-merges scheme needs, writes back the L2 of every XCD and cost far
// more than the second launch when it was tried.
#include <type_traits>
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

// a plain vector: arrays of it stay in registers where arrays of HIP's uint4 struct went to
// scratch memory and came back through it on every page
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

union Frag {
  bf16x8 v;
  uint4 q;
  uint2 h[2];
  uint32_t w[4];
};

// operands of the 16x16 matrix instructions
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef short short4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

union Frag16 {
  bf16x8 v;
  u32x4 q;
  u32x2 h[2];
  uint32_t w[4];
};
union Frag8 {
  short4v v;
  u32x2 q;
  uint32_t w[2];
};

__device__ __forceinline__ uint32_t pack2(float a, float b) { return f32x2_to_bf16x2_bits(a, b); }

// Maximum and sum over the lanes 16 or 32 apart, by the lane-swap instructions of gfx950 (one
// vector operation each; a shuffle goes through the LDS crossbar and costs over a hundred
// cycles in the middle of a chain). After the swap one register holds the values of the even
// rows of 16 lanes (lower 32 lanes) and the other those of the odd rows (upper lanes) in
// every lane, so both lanes of a pair combine the same two numbers in the same order.
__device__ __forceinline__ float max_xor16(float x) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float max_xor32(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_xor16(float x) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float sum_xor32(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// keys whose index is >= limit read as zero; `first` is the key of element 0 of a
// 4-key run held in a uint2
__device__ __forceinline__ uint2 zero_from(uint2 v, int first, int limit) {
  if (first + 0 >= limit) v.x &= 0xffff0000u;
  if (first + 1 >= limit) v.x &= 0x0000ffffu;
  if (first + 2 >= limit) v.y &= 0xffff0000u;
  if (first + 3 >= limit) v.y &= 0x0000ffffu;
  return v;
}

template <int DH>
struct WaveState {
  static constexpr int KS = DH / 16;   // k-steps of the first product
  static constexpr int MT = DH / 32;   // 32-row tiles of O^T
  Frag qf[KS];
  floatx16 o[MT];
  float m, l;                          // running maximum (log2 domain) and sum of this lane's row
};

// One page (64 keys) for one wave. kp: K page of the kv head [64][DH]; vp: V^T page
// [DH][64]. my_start/my_end: keys this lane's row may see. kv_len: keys written so far.
// KSTR / VSTR: elements between rows of the K tile / of the V^T tile (a page in global
// memory, or a padded copy in LDS). ZERO_TAIL: unwritten keys of the V^T tile still
// have to be read as zero (the LDS copy is cleaned when it is stored).
template <int DH, int KSTR, int VSTR, bool ZERO_TAIL, bool EARLY_V = false>
__device__ __forceinline__ void wave_page(WaveState<DH>& w, const bf16_t* __restrict__ kp,
                                          const bf16_t* __restrict__ vp, int key0, int my_start,
                                          int my_end, int kv_len, bool all_visible,
                                          float scale_log2, int j, int h) {
  constexpr int KS = DH / 16, MT = DH / 32;
  // EARLY_V: the value operands are requested before the first product, so that a wave
  // that has only a page or two to do waits for memory once, not twice
  Frag va[EARLY_V ? MT : 1][4];
  if (EARLY_V) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const bf16_t* vrow = vp + (mt * 32 + j) * VSTR + 4 * h + 32 * (t / 2) + 16 * (t % 2);
        va[mt][t].h[0] = *reinterpret_cast<const uint2*>(vrow);
        va[mt][t].h[1] = *reinterpret_cast<const uint2*>(vrow + 8);
      }
  }
  floatx16 s[2];
#pragma unroll
  for (int sub = 0; sub < 2; ++sub) {
    floatx16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const bf16_t* krow = kp + (sub * 32 + j) * KSTR + h * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Frag a;
      a.q = *reinterpret_cast<const uint4*>(krow + ks * 16);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, w.qf[ks].v, acc, 0, 0, 0);
    }
    s[sub] = acc;
  }
  // softmax of the lane's row over this page. Scores stay raw; the running maximum is
  // kept in the log2 domain (raw * scale * log2 e), so an exponent is one fma + exp2.
  float mx = -INFINITY;
  if (all_visible) {
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[sub][r]);
  } else {
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = key0 + sub * 32 + 8 * (r / 4) + 4 * h + (r % 4);
        const float t = (key >= my_start && key < my_end) ? s[sub][r] : -INFINITY;
        s[sub][r] = t;
        mx = fmaxf(mx, t);
      }
  }
  mx = max_xor32(mx);
  const float m_new = fmaxf(w.m, mx * scale_log2);     // -inf * positive stays -inf
  const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
  const float alpha = __builtin_amdgcn_exp2f(w.m - m_use);
  float rs = 0.f;
#pragma unroll
  for (int sub = 0; sub < 2; ++sub)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float p = __builtin_amdgcn_exp2f(fmaf(s[sub][r], scale_log2, -m_use));
      s[sub][r] = p;
      rs += p;
    }
  rs = sum_xor32(rs);
  w.l = w.l * alpha + rs;
  w.m = m_new;
  if (__any(alpha != 1.f)) {       // once the maxima have settled nothing needs rescaling
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) w.o[mt][r] *= alpha;
  }

  Frag pb[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e)
      pb[t].w[e] = pack2(s[t / 2][8 * (t % 2) + 2 * e], s[t / 2][8 * (t % 2) + 2 * e + 1]);

  const bool partial = ZERO_TAIL && key0 + TA_PAGE > kv_len;   // unwritten keys hold anything: read them as 0
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const bf16_t* vrow = vp + (mt * 32 + j) * VSTR + 4 * h;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int kb = 32 * (t / 2) + 16 * (t % 2);
      Frag a;
      if (EARLY_V) {
        a = va[EARLY_V ? mt : 0][t];
      } else {
        a.h[0] = *reinterpret_cast<const uint2*>(vrow + kb);
        a.h[1] = *reinterpret_cast<const uint2*>(vrow + kb + 8);
      }
      if (partial) {
        a.h[0] = zero_from(a.h[0], key0 + kb + 4 * h, kv_len);
        a.h[1] = zero_from(a.h[1], key0 + kb + 8 + 4 * h, kv_len);
      }
      w.o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, pb[t].v, w.o[mt], 0, 0, 0);
    }
  }
}

template <int DH>
__device__ __forceinline__ void wave_init(WaveState<DH>& w, const bf16_t* __restrict__ qrow,
                                          bool row_ok, int h) {
#pragma unroll
  for (int ks = 0; ks < DH / 16; ++ks) {
    if (row_ok)
      w.qf[ks].q = *reinterpret_cast<const uint4*>(qrow + ks * 16 + h * 8);
    else
      w.qf[ks].q = make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int mt = 0; mt < DH / 32; ++mt)
#pragma unroll
    for (int r = 0; r < 16; ++r) w.o[mt][r] = 0.f;
  w.m = -INFINITY;
  w.l = 0.f;
}

// ------------------------------------------------------------------ rows: prompts
template <int DH>
__global__ __launch_bounds__(256) void attn_rows_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
    const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ pos0, int nh, int nkv, float scale_log2, int window) {
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int j = lane % 32, h = lane / 32;
  const int b = blockIdx.z, kvh = blockIdx.y;
  const int group = nh / nkv;
  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0;
  const int nrows = qlen * group;
  const int row0 = (blockIdx.x * 4 + wave) * 32;
  if (row0 >= nrows) return;                       // no barrier is used in this kernel
  const int p0 = pos0[b];
  const int kv_len = p0 + qlen;
  const int row = row0 + j;
  const bool row_ok = row < nrows;
  const int qi = row_ok ? row / group : 0;
  const int head = kvh * group + (row_ok ? row % group : 0);

  WaveState<DH> w;
  wave_init<DH>(w, q + (size_t)(q0 + qi) * q_stride + (size_t)head * DH, row_ok, h);

  const int last_row = (row0 + 31 < nrows - 1) ? row0 + 31 : nrows - 1;
  const int tile_end = p0 + last_row / group + 1;          // largest my_end of the tile
  const int tile_min_end = p0 + row0 / group + 1;          // smallest my_end of the tile
  int tile_start = 0, tile_max_start = 0;
  if (window > 0) {
    tile_start = tile_min_end - window;
    if (tile_start < 0) tile_start = 0;
    tile_max_start = tile_end - window;
    if (tile_max_start < 0) tile_max_start = 0;
  }
  int my_end = row_ok ? p0 + qi + 1 : 0;
  int my_start = 0;
  if (window > 0 && row_ok) {
    my_start = my_end - window;
    if (my_start < 0) my_start = 0;
  }
  const bool all_rows = row0 + 32 <= nrows;

  const int* table = block_table + (size_t)b * max_blocks;
  for (int pg = tile_start / TA_PAGE; pg * TA_PAGE < tile_end; ++pg) {
    const int key0 = pg * TA_PAGE;
    const size_t page = (size_t)table[pg];
    const bf16_t* kp = kcache + (page * nkv + kvh) * (size_t)(TA_PAGE * DH);
    const bf16_t* vp = vcache + (page * nkv + kvh) * (size_t)(TA_PAGE * DH);
    const bool all_visible = all_rows && key0 + TA_PAGE <= tile_min_end && key0 >= tile_max_start;
    wave_page<DH, DH, TA_PAGE, true>(w, kp, vp, key0, my_start, my_end, kv_len, all_visible, scale_log2, j, h);
  }
  if (row_ok) {
    const float inv = w.l > 0.f ? 1.0f / w.l : 0.f;
    bf16_t* o = out + (size_t)(q0 + qi) * out_stride + (size_t)head * DH;
#pragma unroll
    for (int mt = 0; mt < DH / 32; ++mt)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int d = 32 * mt + 8 * g4 + 4 * h;
        uint2 v;
        v.x = pack2(w.o[mt][4 * g4 + 0] * inv, w.o[mt][4 * g4 + 1] * inv);
        v.y = pack2(w.o[mt][4 * g4 + 2] * inv, w.o[mt][4 * g4 + 3] * inv);
        *reinterpret_cast<uint2*>(o + d) = v;
      }
  }
}

// ------------------------------------------------------------------ rows through LDS
// The same work for long prompts: the four waves of a workgroup own 128 consecutive
// rows of one (sequence, kv head) and share every K and V^T page through LDS, so a page
// crosses the L2 once per 128 rows. The next page travels global -> registers while the
// current one is multiplied, and registers -> LDS between two barriers. Rows are padded
// (K by 16 bytes, V^T by 8) so that the operand reads of a wave spread over all banks.
template <int DH>
__global__ __launch_bounds__(256, 2) void attn_rows_lds_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
    const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ pos0, int nh, int nkv, float scale_log2, int window, int pair) {
  constexpr int KSTR = DH + 8, VSTR = TA_PAGE + 4;
  constexpr int PER = TA_PAGE * DH / 8 / 256;          // 16-byte pieces of a page per thread
  // two page buffers: the next page is stored while the current one is multiplied
  __shared__ __attribute__((aligned(16))) bf16_t Ks[2][TA_PAGE * KSTR];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[2][DH * VSTR];
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int j = lane % 32, h = lane / 32;
  const int b = blockIdx.z, kvh = blockIdx.x;   // kv heads vary fastest: see the launch
  const int group = nh / nkv;
  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0;
  const int nrows = qlen * group;
  // A block of 128 rows reads the keys up to its last token, so the blocks of a prompt are
  // a triangle of work. All workgroups are resident at once and nothing rebalances them, so
  // with `pair` a workgroup takes two blocks, the x-th from the end and then the x-th from
  // the start: every workgroup of a prompt walks the same number of pages. Without it the
  // late blocks, which see the most keys, are handed out first.
  const int nblk = (nrows + 127) / 128;
  if ((int)blockIdx.y >= (pair ? (nblk + 1) / 2 : nblk)) return;   // the whole workgroup leaves together
  const int p0 = pos0[b];
  for (int part = 0; part < 2; ++part) {
  const int blk = part == 0 ? nblk - 1 - (int)blockIdx.y : (int)blockIdx.y;
  if (part == 1 && (!pair || blk == nblk - 1 - (int)blockIdx.y)) break;   // the middle block of an odd count
  const int wg_row0 = blk * 128;
  const int kv_len = p0 + qlen;
  const int row0 = wg_row0 + wave * 32;
  const bool wave_ok = row0 < nrows;
  const int row = row0 + j;
  const bool row_ok = row < nrows;
  const int qi = row_ok ? row / group : 0;
  const int head = kvh * group + (row_ok ? row % group : 0);

  WaveState<DH> w;
  wave_init<DH>(w, q + (size_t)(q0 + qi) * q_stride + (size_t)head * DH, row_ok, h);

  // key ranges: of the workgroup (what is loaded) and of this wave (what it multiplies)
  const int wg_last = (wg_row0 + 127 < nrows - 1) ? wg_row0 + 127 : nrows - 1;
  const int wg_end = p0 + wg_last / group + 1;
  int wg_start = 0;
  if (window > 0) {
    wg_start = p0 + wg_row0 / group + 1 - window;
    if (wg_start < 0) wg_start = 0;
  }
  const int last_row = (row0 + 31 < nrows - 1) ? row0 + 31 : nrows - 1;
  const int tile_end = wave_ok ? p0 + last_row / group + 1 : 0;
  const int tile_min_end = p0 + row0 / group + 1;
  int tile_start = 0, tile_max_start = 0;
  if (window > 0 && wave_ok) {
    tile_start = tile_min_end - window;
    if (tile_start < 0) tile_start = 0;
    tile_max_start = tile_end - window;
    if (tile_max_start < 0) tile_max_start = 0;
  }
  const int my_end = row_ok ? p0 + qi + 1 : 0;
  int my_start = 0;
  if (window > 0 && row_ok) {
    my_start = my_end - window;
    if (my_start < 0) my_start = 0;
  }
  const bool all_rows = row0 + 32 <= nrows;

  const int* table = block_table + (size_t)b * max_blocks;
  const int pg_first = wg_start / TA_PAGE;
  const int pg_last = (wg_end - 1) / TA_PAGE;
  u32x4 kreg[PER], vreg[PER];
#define FETCH_PAGE(pg_)                                                              \
  do {                                                                               \
    const size_t page_ = (size_t)table[pg_];                                         \
    const bf16_t* kp_ = kcache + (page_ * nkv + kvh) * (size_t)(TA_PAGE * DH);       \
    const bf16_t* vp_ = vcache + (page_ * nkv + kvh) * (size_t)(TA_PAGE * DH);       \
    _Pragma("unroll") for (int i = 0; i < PER; ++i) {                                \
      const int piece = threadIdx.x + i * 256;                                       \
      kreg[i] = *reinterpret_cast<const u32x4*>(kp_ + (size_t)piece * 8);            \
      vreg[i] = *reinterpret_cast<const u32x4*>(vp_ + (size_t)piece * 8);            \
    }                                                                                \
  } while (0)

#define STORE_PAGE(buf_, pg_)                                                        \
  do {                                                                               \
    const int key0_ = (pg_) * TA_PAGE;                                               \
    _Pragma("unroll") for (int i = 0; i < PER; ++i) {                                \
      const int piece = threadIdx.x + i * 256;                                       \
      const int krow = piece / (DH / 8), kcol = (piece % (DH / 8)) * 8;              \
      *reinterpret_cast<u32x4*>(Ks[buf_] + krow * KSTR + kcol) = kreg[i];            \
      const int vrow = piece / (TA_PAGE / 8), vcol = (piece % (TA_PAGE / 8)) * 8;    \
      uint4 v = make_uint4(vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w);              \
      if (key0_ + vcol + 8 > kv_len) { /* keys that no step has written read as zero */ \
        uint2 lo = make_uint2(v.x, v.y), hi = make_uint2(v.z, v.w);                  \
        lo = zero_from(lo, key0_ + vcol, kv_len);                                    \
        hi = zero_from(hi, key0_ + vcol + 4, kv_len);                                \
        v = make_uint4(lo.x, lo.y, hi.x, hi.y);                                      \
      }                                                                              \
      /* rows of V^T are padded by 8 bytes, so a 16-byte piece is stored as two halves */ \
      *reinterpret_cast<uint2*>(Vs[buf_] + vrow * VSTR + vcol) = make_uint2(v.x, v.y);      \
      *reinterpret_cast<uint2*>(Vs[buf_] + vrow * VSTR + vcol + 4) = make_uint2(v.z, v.w);  \
    }                                                                                \
  } while (0)

  // K: [64][DH], V^T: [DH][64] in LDS. Page p is stored during the step of page p-1 and its
  // loads were issued a step before that, so a step waits neither for memory nor for the
  // store of its own page; one barrier per page separates the readers of a buffer from its
  // next writers. The barrier at the head of the loop also keeps the two parts of a
  // workgroup apart.
  __syncthreads();
  FETCH_PAGE(pg_first);
  STORE_PAGE(pg_first & 1, pg_first);
  if (pg_first < pg_last) FETCH_PAGE(pg_first + 1);
  for (int pg = pg_first; pg <= pg_last; ++pg) {
    const int key0 = pg * TA_PAGE;
    __syncthreads();
    if (pg < pg_last) {
      STORE_PAGE((pg + 1) & 1, pg + 1);
      if (pg + 1 < pg_last) FETCH_PAGE(pg + 2);
    }
    if (key0 < tile_end && key0 + TA_PAGE > tile_start) {
      const bool all_visible = all_rows && key0 + TA_PAGE <= tile_min_end && key0 >= tile_max_start;
      wave_page<DH, KSTR, VSTR, false>(w, Ks[pg & 1], Vs[pg & 1], key0, my_start, my_end, kv_len, all_visible,
                                       scale_log2, j, h);
    }
  }
#undef STORE_PAGE
#undef FETCH_PAGE
  if (row_ok) {
    const float inv = w.l > 0.f ? 1.0f / w.l : 0.f;
    bf16_t* o = out + (size_t)(q0 + qi) * out_stride + (size_t)head * DH;
#pragma unroll
    for (int mt = 0; mt < DH / 32; ++mt)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int d = 32 * mt + 8 * g4 + 4 * h;
        uint2 v;
        v.x = pack2(w.o[mt][4 * g4 + 0] * inv, w.o[mt][4 * g4 + 1] * inv);
        v.y = pack2(w.o[mt][4 * g4 + 2] * inv, w.o[mt][4 * g4 + 3] * inv);
        *reinterpret_cast<uint2*>(o + d) = v;
      }
  }
  }
}

// ------------------------------------------------------------------ rows, overlapped by half pages
// The same division of labour as attn_rows_lds_kernel (a workgroup's waves share every K and
// V^T page through LDS), with the three parts of the work taken apart so that a wave's matrix
// instructions and its softmax overlap. Work goes in half pages of 32 keys: in a half step the
// matrix cores form the scores of half page k and add the products of half page k - 2 to the
// output while the vector ALU turns the scores of half page k - 1 into probabilities (maximum,
// exponentials, sums, rounding); none of the three needs a result of the other two. A matrix
// instruction keeps its wave from issuing for about 19 cycles and its pipeline busy for 32, and
// some six vector instructions per matrix instruction fit beside it (measured: one wave alone
// on a SIMD 16 ns per matrix instruction with up to 6 of them, 31 ns with 8; two waves on the
// SIMD 15 and 19 ns), so the softmax, five instructions per matrix instruction at heads of 128,
// has to be dealt out between the matrix instructions, and a second wave on the SIMD takes
// what is left over. The output is rescaled by a half page's factor after the half page
// before it has been added, which is the same sum.
//
// A workgroup owns 128 rows, a wave one tile of 32, and a wave stays under 256 registers, so
// that two workgroups share a CU. (With 256 rows a workgroup and two tiles a wave every
// operand read from LDS feeds two matrix instructions, but a wave then needs nearly all 512
// registers and has its SIMD to itself: 2 % faster alone for one prompt of 4,096 tokens or
// more, 2 to 3 % slower than this inside the model, slower everywhere else.)
//
// Every wave walks all pages of its workgroup (the tokens of a workgroup's rows end in the same
// page or the next, so nothing is saved by stopping a wave early); pages that every row of the
// workgroup sees whole take steps without the mask. Keys and values come through two LDS
// buffers each: a page's step stores the keys of the next page and the values of this one
// (which the next step multiplies), asked for a step before, and asks for the ones after.

// The reference point of a row's exponentials (log2 domain). It need not be the running
// maximum: probabilities, their sum and the output are all relative to the same number, which
// cancels at the end, and the rounding of a probability to bfloat16 is relative. So the
// reference moves only when a half page's maximum lies more than REFERENCE_SLACK above it (a
// probability then stays below 2^REFERENCE_SLACK) or when the row has seen no key yet, and the
// output, which would have to be multiplied by the factor that this returns, is left alone on
// most pages.
#define REFERENCE_SLACK 8.0f
__device__ __forceinline__ float softmax_reference(float& m, float page_max) {
  if (!(page_max > m + REFERENCE_SLACK)) return 1.f;        // also when both are -inf
  const float alpha = __builtin_amdgcn_exp2f(m - page_max);        // 0 for a row's first keys
  m = page_max;
  return alpha;
}

template <int DH>
struct HalvesState {
  static constexpr int KS = DH / 16, MT = DH / 32;
  static constexpr int PER = TA_PAGE * DH / 8 / 256;   // 16-byte pieces of a page per thread
  Frag qf[KS];
  floatx16 o[MT];
  float m, l;                  // the row's reference (log2 domain) and sum
  floatx16 s[2];               // [half page's parity]
  Frag pb[2][2];               // [half page's parity][16 keys]
  u32x4 kreg[PER], vreg[PER];
};

// scores of the wave's rows for the 32 keys at krows (the wave's view: row j of the half page)
template <int DH, int KSTR>
__device__ __forceinline__ void halves_scores(const Frag (&qf)[DH / 16], const bf16_t* __restrict__ krows,
                                              floatx16& s) {
  s = floatx16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int k = 0; k < DH / 16; ++k) {
    Frag a;
    a.q = *reinterpret_cast<const uint4*>(krows + k * 16);
    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, qf[k].v, s, 0, 0, 0);
  }
}

// scores over 32 keys -> probabilities, packed; returns the factor for what is older
template <bool MASKED>
__device__ __forceinline__ float halves_softmax(floatx16& s, Frag (&pb)[2], float& m, float& l, int key0,
                                                int my_start, int my_end, float scale_log2, int h) {
  float mx = -INFINITY;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    if (MASKED) {
      const int key = key0 + 8 * (r / 4) + 4 * h + (r % 4);
      s[r] = (key >= my_start && key < my_end) ? s[r] : -INFINITY;
    }
    mx = fmaxf(mx, s[r]);
  }
  mx = max_xor32(mx);
  const float alpha = softmax_reference(m, mx * scale_log2);
  const float m_use = (m == -INFINITY) ? 0.f : m;
  float rs = 0.f;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float p = __builtin_amdgcn_exp2f(fmaf(s[r], scale_log2, -m_use));
    s[r] = p;
    rs += p;
  }
  rs = sum_xor32(rs);
  l = l * alpha + rs;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) pb[t].w[e] = pack2(s[8 * t + 2 * e], s[8 * t + 2 * e + 1]);
  return alpha;
}

// vrows: the wave's view of the half page's values (row j of V^T, first key of the half page)
template <int DH, int VSTR>
__device__ __forceinline__ void halves_values(floatx16 (&o)[DH / 32], const bf16_t* __restrict__ vrows,
                                              const Frag (&pb)[2]) {
#pragma unroll
  for (int mt = 0; mt < DH / 32; ++mt)
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      Frag a;
      a.h[0] = *reinterpret_cast<const uint2*>(vrows + mt * 32 * VSTR + 16 * t);
      a.h[1] = *reinterpret_cast<const uint2*>(vrows + mt * 32 * VSTR + 16 * t + 8);
      o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, pb[t].v, o[mt], 0, 0, 0);
    }
}

// A half step with all three parts, written out in the order in which it is to be issued: a
// unit is one operand from LDS, read three units before, and the matrix instruction it feeds
// (the scores of the next half page first, then the products of the one before), and behind
// it a slice of this half page's softmax: maxima of 8 scores, the row's reference and factor,
// 2 exponentials and their sum, the row's sum, 2 words of packed probabilities. The scheduler
// may reorder inside a unit but not across units (left alone it issues all matrix
// instructions first and the softmax behind them, and nothing overlaps). Returns the factor
// for what is older.
template <int DH, int KSTR, int VSTR, bool MASKED>
__device__ __forceinline__ float halves_full_half(const Frag (&qf)[DH / 16], floatx16 (&o)[DH / 32], float& m,
                                                  float& l, floatx16& s_nxt, floatx16& s_cur, Frag (&pb_cur)[2],
                                                  const Frag (&pb_prev)[2], const bf16_t* __restrict__ krows,
                                                  const bf16_t* __restrict__ vrows, int key0, int my_start,
                                                  int my_end, float scale_log2, int h) {
  constexpr int KS = DH / 16, NPV = (DH / 32) * 2, U = KS + NPV;
  constexpr int I_MAX = 2, I_REF = I_MAX, I_EXP = I_REF + 1, I_SUM = I_EXP + 8, I_PACK = I_SUM + 1;
  constexpr int ITEMS = I_PACK + 4;
  constexpr int AHEAD = 3;               // operands are read from LDS this many units before their use
  float mx = -INFINITY, m_use = 0.f, rs = 0.f, alpha = 1.f;
  Frag ring[AHEAD + 1];
#define HALVES_READ(u_)                                                                          \
  do {                                                                                         \
    if ((u_) < KS) {                                                                           \
      ring[(u_) % (AHEAD + 1)].q = *reinterpret_cast<const uint4*>(krows + (u_) * 16);          \
    } else if ((u_) < U) {                                                                     \
      const bf16_t* vrow_ = vrows + (((u_) - KS) / 2) * 32 * VSTR + 16 * (((u_) - KS) % 2);    \
      ring[(u_) % (AHEAD + 1)].h[0] = *reinterpret_cast<const uint2*>(vrow_);                  \
      ring[(u_) % (AHEAD + 1)].h[1] = *reinterpret_cast<const uint2*>(vrow_ + 8);              \
    }                                                                                          \
  } while (0)
#pragma unroll
  for (int u = 0; u < AHEAD; ++u) HALVES_READ(u);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    HALVES_READ(u + AHEAD);
    if (u < KS) {
      if (u == 0) s_nxt = floatx16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      s_nxt = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[u % (AHEAD + 1)].v, qf[u].v, s_nxt, 0, 0, 0);
    } else {
      const int mt = (u - KS) / 2, t = (u - KS) % 2;
      o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[u % (AHEAD + 1)].v, pb_prev[t].v, o[mt], 0, 0, 0);
    }
#pragma unroll
    for (int it = u * ITEMS / U; it < (u + 1) * ITEMS / U; ++it) {
      if (it < I_MAX) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int r = it * 8 + e;
          if (MASKED) {
            const int key = key0 + 8 * (r / 4) + 4 * h + (r % 4);
            s_cur[r] = (key >= my_start && key < my_end) ? s_cur[r] : -INFINITY;
          }
          mx = fmaxf(mx, s_cur[r]);
        }
      } else if (it == I_REF) {
        mx = max_xor32(mx);
        alpha = softmax_reference(m, mx * scale_log2);
        m_use = (m == -INFINITY) ? 0.f : m;
      } else if (it < I_SUM) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const int r = (it - I_EXP) * 2 + e;
          const float p = __builtin_amdgcn_exp2f(fmaf(s_cur[r], scale_log2, -m_use));
          s_cur[r] = p;
          rs += p;
        }
      } else if (it == I_SUM) {
        rs = sum_xor32(rs);
        l = l * alpha + rs;
      } else {
#pragma unroll
        for (int e2 = 0; e2 < 2; ++e2) {
          const int w2 = (it - I_PACK) * 2 + e2, t = w2 / 4, e = w2 % 4;
          pb_cur[t].w[e] = pack2(s_cur[8 * t + 2 * e], s_cur[8 * t + 2 * e + 1]);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#undef HALVES_READ
  return alpha;
}

template <int DH>
__global__ __launch_bounds__(256, 2) void attn_rows_halves_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
    const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ pos0, int nh, int nkv, float scale_log2, int window, int pair) {
  constexpr int KSTR = DH + 8, VSTR = TA_PAGE + 4;
  constexpr int PER = HalvesState<DH>::PER, MT = DH / 32;
  constexpr int ROWS = 128;
  __shared__ __attribute__((aligned(16))) bf16_t Ks[2][TA_PAGE * KSTR];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[2][DH * VSTR];
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int j = lane % 32, h = lane / 32;
  const int b = blockIdx.z, kvh = blockIdx.x;   // kv heads vary fastest: see the launch
  const int group = nh / nkv;
  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0;
  const int nrows = qlen * group;
  const int nblk = (nrows + ROWS - 1) / ROWS;
  if ((int)blockIdx.y >= (pair == 1 ? (nblk + 1) / 2 : nblk)) return;   // the whole workgroup leaves together
  const int p0 = pos0[b];
  const int kv_len = p0 + qlen;
  const int* table = block_table + (size_t)b * max_blocks;
  for (int part = 0; part < 2; ++part) {
    // with `pair` == 1 the x-th block from the end and then the x-th from the start (see
    // attn_rows_lds_kernel); otherwise one block each, the longest first
    int blk = part == 0 ? nblk - 1 - (int)blockIdx.y : (int)blockIdx.y;
    if (part == 1 && (pair != 1 || blk == nblk - 1 - (int)blockIdx.y)) break;
    if (pair == 2) {
      // Unpaired, two workgroups share a CU and all are on the CUs at once. They are placed in
      // the order of their index, the second round on the CUs in the order of the first: the
      // late half of the blocks from the end, then the early half from the start, so that the
      // longest block shares its CU with the shortest (2,048 tokens of the 8B shape fill the
      // CUs exactly twice: 63 -> 60 us). With more workgroups than that the ones that wait go
      // longest first.
      const int half = (nblk + 1) / 2;
      blk = (int)blockIdx.y < half ? nblk - 1 - (int)blockIdx.y : (int)blockIdx.y - half;
    }
    const int wg_row0 = blk * ROWS;
    HalvesState<DH> st;
    const int row = wg_row0 + wave * 32 + j;
    const bool row_ok = row < nrows;
    const int qi = row_ok ? row / group : 0;
    const int head = kvh * group + (row_ok ? row % group : 0);
    const int my_end = row_ok ? p0 + qi + 1 : 0;
    int my_start = 0;
    if (window > 0 && row_ok) {
      my_start = my_end - window;
      if (my_start < 0) my_start = 0;
    }
    {
      const bf16_t* qrow = q + (size_t)(q0 + qi) * q_stride + (size_t)head * DH;
#pragma unroll
      for (int k = 0; k < DH / 16; ++k) {
        if (row_ok)
          st.qf[k].q = *reinterpret_cast<const uint4*>(qrow + k * 16 + h * 8);
        else
          st.qf[k].q = make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) st.o[mt][r] = 0.f;
      st.m = -INFINITY;
      st.l = 0.f;
    }

    // keys of the workgroup (what is loaded and walked)
    const int wg_last = (wg_row0 + ROWS - 1 < nrows - 1) ? wg_row0 + ROWS - 1 : nrows - 1;
    const int wg_end = p0 + wg_last / group + 1;
    const int wg_min_end = p0 + wg_row0 / group + 1;     // what the workgroup's first row sees
    int wg_start = 0;
    if (window > 0) {
      wg_start = wg_min_end - window;
      if (wg_start < 0) wg_start = 0;
    }
    const int pg_first = wg_start / TA_PAGE;
    const int n = (wg_end - 1) / TA_PAGE - pg_first + 1;           // pages to walk, >= 1
    // leading pages that every row of the workgroup sees whole
    int n_full = 0;
    if (window == 0 && wg_last == wg_row0 + ROWS - 1) {
      n_full = wg_min_end / TA_PAGE - pg_first;
      if (n_full > n) n_full = n;
      if (n_full < 0) n_full = 0;
    }

    // the wave's views of a page in LDS: row j of the keys, row j of V^T
    const int koff = j * KSTR + h * 8, voff = j * VSTR + 4 * h;
#define HALVES_PAGE_NO(i_) table[pg_first + ((i_) < n ? (i_) : n - 1)]   /* one past the end: the last page again */
#define HALVES_FETCH(dst_, cache_, pgno_)                                              \
  do {                                                                               \
    const bf16_t* p_ = cache_ + ((size_t)(pgno_) * nkv + kvh) * (size_t)(TA_PAGE * DH); \
    _Pragma("unroll") for (int x = 0; x < PER; ++x)                                  \
        dst_[x] = *reinterpret_cast<const u32x4*>(p_ + (size_t)(threadIdx.x + x * 256) * 8); \
  } while (0)
#define HALVES_STORE_K(buf_, src_)                                                     \
  do {                                                                               \
    _Pragma("unroll") for (int x = 0; x < PER; ++x) {                                \
      const int piece = threadIdx.x + x * 256;                                       \
      const int krow = piece / (DH / 8), kcol = (piece % (DH / 8)) * 8;              \
      *reinterpret_cast<u32x4*>(Ks[buf_] + krow * KSTR + kcol) = src_[x];            \
    }                                                                                \
  } while (0)
#define HALVES_STORE_V(buf_, i_)                                                       \
  do {                                                                               \
    const int key0_ = (pg_first + (i_)) * TA_PAGE;                                   \
    _Pragma("unroll") for (int x = 0; x < PER; ++x) {                                \
      const int piece = threadIdx.x + x * 256;                                       \
      const int vrow = piece / (TA_PAGE / 8), vcol = (piece % (TA_PAGE / 8)) * 8;    \
      uint4 v = make_uint4(st.vreg[x].x, st.vreg[x].y, st.vreg[x].z, st.vreg[x].w);  \
      /* keys that no step has written read as zero; the page's test first, which is the same \
         for all lanes and fails for every page but a sequence's last */            \
      if (key0_ + TA_PAGE > kv_len && key0_ + vcol + 8 > kv_len) {                   \
        uint2 lo = make_uint2(v.x, v.y), hi = make_uint2(v.z, v.w);                  \
        lo = zero_from(lo, key0_ + vcol, kv_len);                                    \
        hi = zero_from(hi, key0_ + vcol + 4, kv_len);                                \
        v = make_uint4(lo.x, lo.y, hi.x, hi.y);                                      \
      }                                                                              \
      /* rows of V^T are padded by 8 bytes, so a 16-byte piece is stored as two halves */ \
      *reinterpret_cast<uint2*>(Vs[buf_] + vrow * VSTR + vcol) = make_uint2(v.x, v.y);      \
      *reinterpret_cast<uint2*>(Vs[buf_] + vrow * VSTR + vcol + 4) = make_uint2(v.z, v.w);  \
    }                                                                                \
  } while (0)
#define HALVES_RESCALE(alpha_)                                                       \
  do {                                                                               \
    if (__any((alpha_) != 1.f)) { /* the reference of some row has moved */          \
      _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                              \
          _Pragma("unroll") for (int r = 0; r < 16; ++r) st.o[mt][r] *= (alpha_);    \
    }                                                                                \
  } while (0)
    // Step i >= 1 after its barrier: the keys of page i and the values of page i - 1 are in
    // LDS, nobody reads the other two buffers any more. Half step a: scores of the first half
    // of page i, softmax of the second half of page i - 1, products of the first half of page
    // i - 1; half step b: scores of the second half of page i, softmax of its first half,
    // products of the second half of page i - 1.
#define HALVES_STEP(i_, MASKED)                                                      \
  do {                                                                               \
    const int cur_ = (i_) & 1;                                                       \
    __syncthreads();                                                                 \
    HALVES_STORE_K(1 - cur_, st.kreg);                                               \
    HALVES_STORE_V(cur_, (i_));                                                      \
    HALVES_FETCH(st.kreg, kcache, pgk_);                                             \
    HALVES_FETCH(st.vreg, vcache, pgv_);                                             \
    pgk_ = HALVES_PAGE_NO((i_) + 3);                                                 \
    pgv_ = HALVES_PAGE_NO((i_) + 2);                                                 \
    const int key0_ = (pg_first + (i_)) * TA_PAGE;                                   \
    __builtin_amdgcn_sched_barrier(0);                                               \
    const float alpha_a_ = halves_full_half<DH, KSTR, VSTR, MASKED>(                 \
        st.qf, st.o, st.m, st.l, st.s[0], st.s[1], st.pb[1], st.pb[0], Ks[cur_] + koff, Vs[1 - cur_] + voff, \
        key0_ - 32, my_start, my_end, scale_log2, h);                                \
    HALVES_RESCALE(alpha_a_);                                                        \
    __builtin_amdgcn_sched_barrier(0);                                               \
    const float alpha_b_ = halves_full_half<DH, KSTR, VSTR, MASKED>(                 \
        st.qf, st.o, st.m, st.l, st.s[1], st.s[0], st.pb[0], st.pb[1], Ks[cur_] + koff + 32 * KSTR,  \
        Vs[1 - cur_] + voff + 32, key0_, my_start, my_end, scale_log2, h);           \
    HALVES_RESCALE(alpha_b_);                                                        \
  } while (0)

    __syncthreads();                       // the readers of the part before are done
    {
      // the first two pages' keys and the first page's values are asked for at once
      u32x4 k1[PER];
      const int pg0_ = table[pg_first], pg1_ = HALVES_PAGE_NO(1);
      HALVES_FETCH(st.kreg, kcache, pg0_);
      HALVES_FETCH(k1, kcache, pg1_);
      HALVES_FETCH(st.vreg, vcache, pg0_);
      HALVES_STORE_K(0, st.kreg);
#pragma unroll
      for (int x = 0; x < PER; ++x) st.kreg[x] = k1[x];
    }
    int pgk_ = HALVES_PAGE_NO(2), pgv_ = HALVES_PAGE_NO(1);
    {
      // step 0: nothing older to finish
      __syncthreads();
      HALVES_STORE_K(1, st.kreg);
      HALVES_STORE_V(0, 0);
      HALVES_FETCH(st.kreg, kcache, pgk_);
      HALVES_FETCH(st.vreg, vcache, pgv_);
      pgk_ = HALVES_PAGE_NO(3);
      pgv_ = HALVES_PAGE_NO(2);
      const int key0_ = pg_first * TA_PAGE;
      halves_scores<DH, KSTR>(st.qf, Ks[0] + koff, st.s[0]);
      halves_scores<DH, KSTR>(st.qf, Ks[0] + koff + 32 * KSTR, st.s[1]);
      // the factor it returns has nothing to multiply: the output is still zero
      if (n_full > 0)
        halves_softmax<false>(st.s[0], st.pb[0], st.m, st.l, key0_, my_start, my_end, scale_log2, h);
      else
        halves_softmax<true>(st.s[0], st.pb[0], st.m, st.l, key0_, my_start, my_end, scale_log2, h);
    }
    int i = 1;
    for (; i < n_full && i < n; ++i) HALVES_STEP(i, false);
    for (; i < n; ++i) HALVES_STEP(i, true);
    {
      // what is left of the last page: the softmax of its second half and both products
      const int last_ = n - 1, cur_ = last_ & 1;
      __syncthreads();
      const float alpha_ = halves_softmax<true>(st.s[1], st.pb[1], st.m, st.l, (pg_first + last_) * TA_PAGE + 32,
                                                my_start, my_end, scale_log2, h);
      halves_values<DH, VSTR>(st.o, Vs[cur_] + voff, st.pb[0]);
      HALVES_RESCALE(alpha_);
      halves_values<DH, VSTR>(st.o, Vs[cur_] + voff + 32, st.pb[1]);
    }
#undef HALVES_STEP
#undef HALVES_RESCALE
#undef HALVES_STORE_V
#undef HALVES_STORE_K
#undef HALVES_FETCH
#undef HALVES_PAGE_NO
    if (row_ok) {
      const float inv = st.l > 0.f ? 1.0f / st.l : 0.f;
      bf16_t* o = out + (size_t)(q0 + qi) * out_stride + (size_t)head * DH;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int d = 32 * mt + 8 * g4 + 4 * h;
          uint2 v;
          v.x = pack2(st.o[mt][4 * g4 + 0] * inv, st.o[mt][4 * g4 + 1] * inv);
          v.y = pack2(st.o[mt][4 * g4 + 2] * inv, st.o[mt][4 * g4 + 3] * inv);
          *reinterpret_cast<uint2*>(o + d) = v;
        }
    }
  }
}

// ------------------------------------------------------------------ keys: single tokens
// grid (nkv * head_chunks, units), WAVES waves per workgroup. Every sequence brings exactly
// one token (row b of qkv). A workgroup takes one unit of work, a run of pages of one
// sequence named by the host's table, one page per wave in turn, merges its waves through
// LDS and writes either the final rows (the sequence has this one unit) or an unnormalised
// partial row with its (max, sum) for the merge kernel. The host cuts the sequences into
// units of about equal length, because what a CU can ask of the memory in a given time is
// limited and the longest walk sets the kernel's time.
//
// The step's rotation and cache write can ride along (cs / dest not null): the raw
// projections are read from qkv = [q heads | k heads | v heads], q is rotated in
// registers, and the workgroup whose slice holds the sequence's last page first
// rotates and stores the new key and stores the new value, then waits at a barrier:
// that page is read by this workgroup only, and a barrier makes a workgroup's global
// writes visible to itself.
template <int DH, int WAVES>
__global__ __launch_bounds__(WAVES * 64, 2) void attn_keys_kernel(
    const bf16_t* __restrict__ qkv, int q_stride, const float* __restrict__ bias,
    const float2* __restrict__ cs, int style, const int* __restrict__ dest,
    bf16_t* __restrict__ out, int out_stride, bf16_t* __restrict__ kcache,
    bf16_t* __restrict__ vcache, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ pos0, int nh, int nkv, float scale_log2, int window,
    const int* __restrict__ units, const int* __restrict__ seq_units, float* __restrict__ partial) {
  extern __shared__ float lds[];
  constexpr int KS = DH / 16, HALF = DH / 2;
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int j = lane % 32, h = lane / 32;
  // blockIdx.y names a unit of work: pages [unit_first, unit_first + unit_count) of sequence b
  const int* unit = units + TA_UNIT_INTS * blockIdx.y;
  const int b = unit[0], unit_first = unit[1], unit_count = unit[2];
  if (unit_count == 0) return;                   // a spare unit (every thread leaves here)
  const int splits = unit[6];                    // units that share this sequence
  const int group = nh / nkv;
  const int chunks = (group + 31) / 32;
  const int kvh = blockIdx.x / chunks, chunk = blockIdx.x % chunks;
  const int hg0 = chunk * 32;
  const int nrows = (group - hg0 < 32) ? group - hg0 : 32;
  const int p0 = pos0[b];
  const int kv_len = p0 + 1;
  const bool row_ok = j < nrows;
  const int head = kvh * group + hg0 + (row_ok ? j : 0);
  const bf16_t* tokrow = qkv + (size_t)b * q_stride;

  // ---- the new key and value of this kv head go to the cache (one workgroup does it)
  if (dest != nullptr && p0 / TA_PAGE >= unit_first && p0 / TA_PAGE < unit_first + unit_count) {
    // every head chunk of the kv head stores the same bits: each workgroup must see the
    // write before its own reads, and only its own barrier gives it that
    const int slot = dest[b];
    const size_t page = (size_t)(slot / TA_PAGE);
    const int off = slot % TA_PAGE;
    const bf16_t* kraw = tokrow + (size_t)(nh + kvh) * DH;
    const bf16_t* vraw = tokrow + (size_t)(nh + nkv + kvh) * DH;
    const float* kb = bias ? bias + (size_t)(nh + kvh) * DH : nullptr;
    const float* vb = bias ? bias + (size_t)(nh + nkv + kvh) * DH : nullptr;
    bf16_t* kc = kcache + ((page * nkv + kvh) * TA_PAGE + off) * (size_t)DH;
    bf16_t* vc = vcache + (page * nkv + kvh) * (size_t)(DH * TA_PAGE) + off;
    for (int i = threadIdx.x; i < HALF; i += WAVES * 64) {
      const int i0 = style == 0 ? i : 2 * i;
      const int i1 = style == 0 ? i + HALF : 2 * i + 1;
      float a = to_f32(kraw[i0]), c = to_f32(kraw[i1]);
      if (kb) {
        a += kb[i0];
        c += kb[i1];
      }
      float r0 = a, r1 = c;
      if (cs) {
        const float2 k = cs[(size_t)b * HALF + i];
        r0 = a * k.x - c * k.y;
        r1 = a * k.y + c * k.x;
      }
      kc[i0] = from_f32<bf16_t>(r0);
      kc[i1] = from_f32<bf16_t>(r1);
    }
    for (int i = threadIdx.x; i < DH; i += WAVES * 64) {
      float v = to_f32(vraw[i]);
      if (vb) v += vb[i];
      vc[(size_t)i * TA_PAGE] = from_f32<bf16_t>(v);
    }
    __syncthreads();     // the condition above is the same for every thread of the workgroup
  }

  // ---- this lane's row of q, rotated if asked for
  WaveState<DH> w;
  wave_init<DH>(w, tokrow + (size_t)head * DH, row_ok, h);
  if ((cs != nullptr || bias != nullptr) && row_ok) {
    const float* qb = bias ? bias + (size_t)head * DH : nullptr;
    const float2* ct = cs ? cs + (size_t)b * HALF : nullptr;
    if (style == 0) {
#pragma unroll
      for (int ks = 0; ks < KS / 2; ++ks) {
        Frag lo = w.qf[ks], hi = w.qf[ks + KS / 2];
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          float a[2], c[2];
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const int e = 2 * e2 + u;
            const int d = ks * 16 + h * 8 + e;
            const uint32_t wl = lo.w[e2], wh = hi.w[e2];
            a[u] = __uint_as_float(u ? (wl & 0xffff0000u) : (wl << 16));
            c[u] = __uint_as_float(u ? (wh & 0xffff0000u) : (wh << 16));
            if (qb) {
              a[u] += qb[d];
              c[u] += qb[d + HALF];
            }
            if (ct) {
              const float2 k = ct[d];
              const float r0 = a[u] * k.x - c[u] * k.y, r1 = a[u] * k.y + c[u] * k.x;
              a[u] = r0;
              c[u] = r1;
            }
          }
          lo.w[e2] = pack2(a[0], a[1]);
          hi.w[e2] = pack2(c[0], c[1]);
        }
        w.qf[ks] = lo;
        w.qf[ks + KS / 2] = hi;
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        Frag f = w.qf[ks];
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          const int d = ks * 16 + h * 8 + 2 * e2;
          float a = __uint_as_float(f.w[e2] << 16), c = __uint_as_float(f.w[e2] & 0xffff0000u);
          if (qb) {
            a += qb[d];
            c += qb[d + 1];
          }
          if (ct) {
            const float2 k = ct[d / 2];
            const float r0 = a * k.x - c * k.y, r1 = a * k.y + c * k.x;
            a = r0;
            c = r1;
          }
          f.w[e2] = pack2(a, c);
        }
        w.qf[ks] = f;
      }
    }
  }

  const int my_end = row_ok ? kv_len : 0;
  int my_start = 0;
  if (window > 0 && row_ok) {
    my_start = my_end - window;
    if (my_start < 0) my_start = 0;
  }
  const int vis_start = (window > 0 && kv_len > window) ? kv_len - window : 0;
  const int n_pages = (kv_len + TA_PAGE - 1) / TA_PAGE;
  int pg_lo = unit_first;
  int pg_hi = unit_first + unit_count;
  if (pg_hi > n_pages) pg_hi = n_pages;
  if (vis_start / TA_PAGE > pg_lo) pg_lo = vis_start / TA_PAGE;
  // keep every wave on its own residue so that a page is always taken by the same wave
  const int first = pg_lo + ((wave - pg_lo % WAVES) + WAVES) % WAVES;
  const int* table = block_table + (size_t)b * max_blocks;
  for (int pg = first; pg < pg_hi; pg += WAVES) {
    const int key0 = pg * TA_PAGE;
    const size_t page = (size_t)table[pg];
    const bf16_t* kp = kcache + (page * nkv + kvh) * (size_t)(TA_PAGE * DH);
    const bf16_t* vp = vcache + (page * nkv + kvh) * (size_t)(TA_PAGE * DH);
    const bool all_visible = key0 + TA_PAGE <= kv_len && key0 >= vis_start;   // rows beyond nrows are never written
    wave_page<DH, DH, TA_PAGE, true, true>(w, kp, vp, key0, my_start, my_end, kv_len, all_visible, scale_log2, j, h);
  }

  // ---- merge the waves: lds = ml[WAVES][32][2] then o[WAVES][nrows][DH]
  float* ml = lds;
  float* os = lds + WAVES * 32 * 2;
  if (h == 0) {
    ml[(wave * 32 + j) * 2 + 0] = w.m;
    ml[(wave * 32 + j) * 2 + 1] = w.l;
  }
  if (row_ok) {
    float* dst = os + ((size_t)wave * nrows + j) * DH;
#pragma unroll
    for (int mt = 0; mt < DH / 32; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) dst[32 * mt + 8 * (r / 4) + 4 * h + (r % 4)] = w.o[mt][r];
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < nrows * DH; idx += WAVES * 64) {
    const int r = idx / DH, d = idx - r * DH;
    float mm = -INFINITY;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) mm = fmaxf(mm, ml[(wv * 32 + r) * 2]);
    const float m_use = (mm == -INFINITY) ? 0.f : mm;
    float acc = 0.f, ll = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) {
      const float f = __builtin_amdgcn_exp2f(ml[(wv * 32 + r) * 2] - m_use);
      acc += f * os[((size_t)wv * nrows + r) * DH + d];
      ll += f * ml[(wv * 32 + r) * 2 + 1];
    }
    const int hd = kvh * group + hg0 + r;
    if (splits == 1) {
      const float inv = ll > 0.f ? 1.0f / ll : 0.f;
      out[(size_t)b * out_stride + (size_t)hd * DH + d] = from_f32<bf16_t>(acc * inv);
    } else {
      float* pr = partial + ((size_t)blockIdx.y * nh + hd) * (DH + 2);
      pr[d] = acc;
      if (d == 0) {
        pr[DH] = mm;
        pr[DH + 1] = ll;
      }
    }
  }
}

// ------------------------------------------------------------------ keys through LDS
// The same job as attn_keys_kernel with a different division of labour, made for the
// way a CU reads memory: reading a page straight into operand registers asks the
// texture unit for 32-byte and 8-byte pieces of many cache lines, and a CU with eight
// waves doing that is bound by its line requests, not by HBM. Here the four waves of a
// workgroup walk the pages of their slice together: a page comes in with full-width
// coalesced loads, through registers into LDS (as in attn_rows_lds_kernel); every wave
// then forms all scores of the page (the same 32 rows in every wave, so the softmax
// state is identical and nothing has to be merged) and multiplies the values of its own
// quarter of the head dimension.
template <int DH>
__global__ __launch_bounds__(256, 2) void attn_keys_lds_kernel(
    const bf16_t* __restrict__ qkv, int q_stride, const float* __restrict__ bias,
    const float2* __restrict__ cs, int style, const int* __restrict__ dest,
    bf16_t* __restrict__ out, int out_stride, bf16_t* __restrict__ kcache,
    bf16_t* __restrict__ vcache, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ pos0, int nh, int nkv, float scale_log2, int window,
    const int* __restrict__ units, const int* __restrict__ seq_units, float* __restrict__ partial) {
  constexpr int KS = DH / 16, MT = DH / 32, HALF = DH / 2;
  constexpr int MYT = (MT + 3) / 4;                    // 32-row tiles of O^T per wave
  constexpr int KSTR = DH + 8, VSTR = TA_PAGE + 4;
  constexpr int PER = TA_PAGE * DH / 8 / 256;
  __shared__ __attribute__((aligned(16))) bf16_t Ks[TA_PAGE * KSTR];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[DH * VSTR];
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int j = lane % 32, h = lane / 32;
  // blockIdx.y names a unit of work: pages [unit_first, unit_first + unit_count) of sequence b
  const int* unit = units + TA_UNIT_INTS * blockIdx.y;
  const int b = unit[0], unit_first = unit[1], unit_count = unit[2];
  if (unit_count == 0) return;                   // a spare unit (every thread leaves here)
  const int splits = unit[6];                    // units that share this sequence
  const int group = nh / nkv;
  const int chunks = (group + 31) / 32;
  const int kvh = blockIdx.x / chunks, chunk = blockIdx.x % chunks;
  const int hg0 = chunk * 32;
  const int nrows = (group - hg0 < 32) ? group - hg0 : 32;
  const int p0 = pos0[b];
  const int kv_len = p0 + 1;
  const bool row_ok = j < nrows;
  const int head = kvh * group + hg0 + (row_ok ? j : 0);
  const bf16_t* tokrow = qkv + (size_t)b * q_stride;

  if (dest != nullptr && p0 / TA_PAGE >= unit_first && p0 / TA_PAGE < unit_first + unit_count) {
    // every head chunk of the kv head stores the same bits: each workgroup must see the
    // write before its own reads, and only its own barrier gives it that
    const int slot = dest[b];
    const size_t page = (size_t)(slot / TA_PAGE);
    const int off = slot % TA_PAGE;
    const bf16_t* kraw = tokrow + (size_t)(nh + kvh) * DH;
    const bf16_t* vraw = tokrow + (size_t)(nh + nkv + kvh) * DH;
    const float* kb = bias ? bias + (size_t)(nh + kvh) * DH : nullptr;
    const float* vb = bias ? bias + (size_t)(nh + nkv + kvh) * DH : nullptr;
    bf16_t* kc = kcache + ((page * nkv + kvh) * TA_PAGE + off) * (size_t)DH;
    bf16_t* vc = vcache + (page * nkv + kvh) * (size_t)(DH * TA_PAGE) + off;
    for (int i = threadIdx.x; i < HALF; i += 256) {
      const int i0 = style == 0 ? i : 2 * i;
      const int i1 = style == 0 ? i + HALF : 2 * i + 1;
      float a = to_f32(kraw[i0]), c = to_f32(kraw[i1]);
      if (kb) {
        a += kb[i0];
        c += kb[i1];
      }
      float r0 = a, r1 = c;
      if (cs) {
        const float2 k = cs[(size_t)b * HALF + i];
        r0 = a * k.x - c * k.y;
        r1 = a * k.y + c * k.x;
      }
      kc[i0] = from_f32<bf16_t>(r0);
      kc[i1] = from_f32<bf16_t>(r1);
    }
    for (int i = threadIdx.x; i < DH; i += 256) {
      float v = to_f32(vraw[i]);
      if (vb) v += vb[i];
      vc[(size_t)i * TA_PAGE] = from_f32<bf16_t>(v);
    }
    __syncthreads();     // the condition above is the same for every thread of the workgroup
  }

  const int my_end = row_ok ? kv_len : 0;
  const int vis_start = (window > 0 && kv_len > window) ? kv_len - window : 0;
  const int my_start = row_ok ? vis_start : 0;
  const int n_pages = (kv_len + TA_PAGE - 1) / TA_PAGE;
  int pg_lo = unit_first;
  int pg_hi = unit_first + unit_count;
  if (pg_hi > n_pages) pg_hi = n_pages;
  if (vis_start / TA_PAGE > pg_lo) pg_lo = vis_start / TA_PAGE;
  if (pg_lo >= pg_hi) {
    // a slice past this sequence's end or before its window (never the slice that stored the
    // new key): it says so in its (max, sum) and the merge passes over it
    if (splits > 1 && wave == 0 && h == 0 && row_ok) {
      float* pr = partial + ((size_t)blockIdx.y * nh + head) * (DH + 2);
      pr[DH] = -INFINITY;
      pr[DH + 1] = 0.f;
    }
    return;
  }

  // ---- this lane's row of q (the same in all four waves), rotated if asked for
  Frag qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (row_ok)
      qf[ks].q = *reinterpret_cast<const uint4*>(tokrow + (size_t)head * DH + ks * 16 + h * 8);
    else
      qf[ks].q = make_uint4(0, 0, 0, 0);
  }
  if ((cs != nullptr || bias != nullptr) && row_ok) {
    const float* qb = bias ? bias + (size_t)head * DH : nullptr;
    const float2* ct = cs ? cs + (size_t)b * HALF : nullptr;
    if (style == 0) {
#pragma unroll
      for (int ks = 0; ks < KS / 2; ++ks) {
        Frag lo = qf[ks], hi = qf[ks + KS / 2];
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          float a[2], c[2];
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const int d = ks * 16 + h * 8 + 2 * e2 + u;
            const uint32_t wl = lo.w[e2], wh = hi.w[e2];
            a[u] = __uint_as_float(u ? (wl & 0xffff0000u) : (wl << 16));
            c[u] = __uint_as_float(u ? (wh & 0xffff0000u) : (wh << 16));
            if (qb) {
              a[u] += qb[d];
              c[u] += qb[d + HALF];
            }
            if (ct) {
              const float2 k = ct[d];
              const float r0 = a[u] * k.x - c[u] * k.y, r1 = a[u] * k.y + c[u] * k.x;
              a[u] = r0;
              c[u] = r1;
            }
          }
          lo.w[e2] = pack2(a[0], a[1]);
          hi.w[e2] = pack2(c[0], c[1]);
        }
        qf[ks] = lo;
        qf[ks + KS / 2] = hi;
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        Frag f = qf[ks];
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          const int d = ks * 16 + h * 8 + 2 * e2;
          float a = __uint_as_float(f.w[e2] << 16), c = __uint_as_float(f.w[e2] & 0xffff0000u);
          if (qb) {
            a += qb[d];
            c += qb[d + 1];
          }
          if (ct) {
            const float2 k = ct[d / 2];
            const float r0 = a * k.x - c * k.y, r1 = a * k.y + c * k.x;
            a = r0;
            c = r1;
          }
          f.w[e2] = pack2(a, c);
        }
        qf[ks] = f;
      }
    }
  }

  floatx16 o[MYT];
#pragma unroll
  for (int i = 0; i < MYT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
  float m = -INFINITY, l = 0.f;

  const int* table = block_table + (size_t)b * max_blocks;

  u32x4 kreg[PER], vreg[PER];
#define FETCH_PAGE(pg_)                                                              \
  do {                                                                               \
    const size_t page_ = (size_t)table[pg_];                                         \
    const bf16_t* kp_ = kcache + (page_ * nkv + kvh) * (size_t)(TA_PAGE * DH);       \
    const bf16_t* vp_ = vcache + (page_ * nkv + kvh) * (size_t)(TA_PAGE * DH);       \
    _Pragma("unroll") for (int i = 0; i < PER; ++i) {                                \
      const int piece = threadIdx.x + i * 256;                                       \
      kreg[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kp_ + (size_t)piece * 8)); \
      vreg[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vp_ + (size_t)piece * 8)); \
    }                                                                                \
  } while (0)

  if (pg_lo < pg_hi) FETCH_PAGE(pg_lo);
  for (int pg = pg_lo; pg < pg_hi; ++pg) {
    const int key0 = pg * TA_PAGE;
    __syncthreads();                               // everyone is done with the previous page
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int piece = threadIdx.x + i * 256;
      const int krow = piece / (DH / 8), kcol = (piece % (DH / 8)) * 8;
      *reinterpret_cast<u32x4*>(Ks + krow * KSTR + kcol) = kreg[i];
      const int vrow = piece / (TA_PAGE / 8), vcol = (piece % (TA_PAGE / 8)) * 8;
      uint4 v = make_uint4(vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w);
      if (key0 + vcol + 8 > kv_len) {              // keys that no step has written read as zero
        uint2 lo = make_uint2(v.x, v.y), hi = make_uint2(v.z, v.w);
        lo = zero_from(lo, key0 + vcol, kv_len);
        hi = zero_from(hi, key0 + vcol + 4, kv_len);
        v = make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
      *reinterpret_cast<uint2*>(Vs + vrow * VSTR + vcol) = make_uint2(v.x, v.y);
      *reinterpret_cast<uint2*>(Vs + vrow * VSTR + vcol + 4) = make_uint2(v.z, v.w);
    }
    __syncthreads();
    if (pg + 1 < pg_hi) FETCH_PAGE(pg + 1);        // in flight while this page is multiplied

    // ---- scores of the whole page (every wave computes the same ones)
    floatx16 s[2];
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      floatx16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      const bf16_t* krow = Ks + (sub * 32 + j) * KSTR + h * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        Frag a;
        a.q = *reinterpret_cast<const uint4*>(krow + ks * 16);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, qf[ks].v, acc, 0, 0, 0);
      }
      s[sub] = acc;
    }
    float mx = -INFINITY;
    const bool all_visible = key0 + TA_PAGE <= kv_len && key0 >= vis_start;
    if (all_visible) {
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[sub][r]);
    } else {
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + sub * 32 + 8 * (r / 4) + 4 * h + (r % 4);
          const float t = (key >= my_start && key < my_end) ? s[sub][r] : -INFINITY;
          s[sub][r] = t;
          mx = fmaxf(mx, t);
        }
    }
    mx = max_xor32(mx);
    const float m_new = fmaxf(m, mx * scale_log2);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m - m_use);
    float rs = 0.f;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[sub][r], scale_log2, -m_use));
        s[sub][r] = p;
        rs += p;
      }
    rs = sum_xor32(rs);
    l = l * alpha + rs;
    m = m_new;
#pragma unroll
    for (int i = 0; i < MYT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[i][r] *= alpha;
    Frag pb[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        pb[t].w[e] = pack2(s[t / 2][8 * (t % 2) + 2 * e], s[t / 2][8 * (t % 2) + 2 * e + 1]);
    // ---- values: this wave's tiles of the head dimension
#pragma unroll
    for (int i = 0; i < MYT; ++i) {
      const int mt = wave + 4 * i;
      if (mt < MT) {
        const bf16_t* vrow = Vs + (mt * 32 + j) * VSTR + 4 * h;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int kb = 32 * (t / 2) + 16 * (t % 2);
          Frag a;
          a.h[0] = *reinterpret_cast<const uint2*>(vrow + kb);
          a.h[1] = *reinterpret_cast<const uint2*>(vrow + kb + 8);
          o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, pb[t].v, o[i], 0, 0, 0);
        }
      }
    }
  }
#undef FETCH_PAGE

  // ---- every wave writes its part of the head dimension; wave 0 the (max, sum)
  if (row_ok) {
    const int hd = head;
    if (splits == 1) {
      const float inv = l > 0.f ? 1.0f / l : 0.f;
      bf16_t* orow = out + (size_t)b * out_stride + (size_t)hd * DH;
#pragma unroll
      for (int i = 0; i < MYT; ++i) {
        const int mt = wave + 4 * i;
        if (mt < MT) {
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {
            uint2 v;
            v.x = pack2(o[i][4 * g4 + 0] * inv, o[i][4 * g4 + 1] * inv);
            v.y = pack2(o[i][4 * g4 + 2] * inv, o[i][4 * g4 + 3] * inv);
            *reinterpret_cast<uint2*>(orow + 32 * mt + 8 * g4 + 4 * h) = v;
          }
        }
      }
    } else {
      float* pr = partial + ((size_t)blockIdx.y * nh + hd) * (DH + 2);
#pragma unroll
      for (int i = 0; i < MYT; ++i) {
        const int mt = wave + 4 * i;
        if (mt < MT) {
#pragma unroll
          for (int r = 0; r < 16; ++r) pr[32 * mt + 8 * (r / 4) + 4 * h + (r % 4)] = o[i][r];
        }
      }
      if (wave == 0 && h == 0) {
        pr[DH] = m;
        pr[DH + 1] = l;
      }
    }
  }
}

// ------------------------------------------------------------------ keys in quarters
// Single tokens again, for the common case of few query heads per kv head. In
// attn_keys_lds_kernel every wave forms all 64 x 32 scores of a page, of which a group of
// 4 heads uses an eighth, and a page costs about 1.5 us of matrix and vector work however
// fast it arrives. Here a page still comes in with whole-line loads through LDS, but each
// of the four waves takes 16 of its 64 keys, for 16 query heads, on the 16x16 matrix
// instructions: S^T (16 keys x 16 heads) = K (16 x dh) . Q^T, then O^T (dh x 16 heads) +=
// V^T (dh x 16 keys) . P^T, where the accumulator layout of S^T is already the operand
// layout of P^T. Every wave keeps its own running maximum, sum and O^T over its keys; the
// four are merged through LDS at the end. A lane's part of q is 4 elements of the low
// half of the head and their 4 partners of the high half, so that either pairing of the
// rotation stays inside the lane.

template <int DH>
__global__ __launch_bounds__(256, 3) void attn_keys_q16_kernel(
    const bf16_t* __restrict__ qkv, int q_stride, const float* __restrict__ bias,
    const float2* __restrict__ cs, int style, const int* __restrict__ dest,
    bf16_t* __restrict__ out, int out_stride, bf16_t* __restrict__ kcache,
    bf16_t* __restrict__ vcache, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ pos0, int nh, int nkv, float scale_log2, int window,
    const int* __restrict__ units, const int* __restrict__ seq_units, float* __restrict__ partial) {
  constexpr int KT = DH / 32;                          // 32-slot steps of the first product
  constexpr int DT = DH / 16;                          // 16-row tiles of O^T
  constexpr int HALF = DH / 2;
  constexpr int KSTR = DH + 8, VSTR = TA_PAGE + 4;
  constexpr int PER = TA_PAGE * DH / 8 / 256;
  constexpr int KS_BYTES = TA_PAGE * KSTR * 2, VS_BYTES = DH * VSTR * 2;
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[KS_BYTES + VS_BYTES];
  bf16_t* Ks = reinterpret_cast<bf16_t*>(lds_raw);
  bf16_t* Vs = reinterpret_cast<bf16_t*>(lds_raw + KS_BYTES);
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int n = lane % 16, kb = lane / 16;             // query head (column), k-block
  // blockIdx.y names a unit of work: pages [unit_first, unit_first + unit_count) of sequence b
  const int* unit = units + TA_UNIT_INTS * blockIdx.y;
  const int b = unit[0], unit_first = unit[1], unit_count = unit[2];
  if (unit_count == 0) return;                   // a spare unit (every thread leaves here)
  const int splits = unit[6];                    // units that share this sequence
  const int group = nh / nkv;
  const int chunks = (group + 15) / 16;
  const int kvh = blockIdx.x / chunks, chunk = blockIdx.x % chunks;
  const int hg0 = chunk * 16;
  const int nrows = (group - hg0 < 16) ? group - hg0 : 16;
  // the record also holds the sequence's length and the unit's first two page numbers, so
  // that the first pages can be asked for without a walk through pos0 and the table first
  const int kv_len = unit[3];
  const int p0 = kv_len - 1;
  const bool row_ok = n < nrows;
  const int head = kvh * group + hg0 + (row_ok ? n : 0);
  const bf16_t* tokrow = qkv + (size_t)b * q_stride;

  if (dest != nullptr && p0 / TA_PAGE >= unit_first && p0 / TA_PAGE < unit_first + unit_count) {
    // every head chunk of the kv head stores the same bits: each workgroup must see the
    // write before its own reads, and only its own barrier gives it that
    const int slot = dest[b];
    const size_t page = (size_t)(slot / TA_PAGE);
    const int off = slot % TA_PAGE;
    const bf16_t* kraw = tokrow + (size_t)(nh + kvh) * DH;
    const bf16_t* vraw = tokrow + (size_t)(nh + nkv + kvh) * DH;
    const float* kbias = bias ? bias + (size_t)(nh + kvh) * DH : nullptr;
    const float* vbias = bias ? bias + (size_t)(nh + nkv + kvh) * DH : nullptr;
    bf16_t* kc = kcache + ((page * nkv + kvh) * TA_PAGE + off) * (size_t)DH;
    bf16_t* vc = vcache + (page * nkv + kvh) * (size_t)(DH * TA_PAGE) + off;
    for (int i = threadIdx.x; i < HALF; i += 256) {
      const int i0 = style == 0 ? i : 2 * i;
      const int i1 = style == 0 ? i + HALF : 2 * i + 1;
      float a = to_f32(kraw[i0]), c = to_f32(kraw[i1]);
      if (kbias) {
        a += kbias[i0];
        c += kbias[i1];
      }
      float r0 = a, r1 = c;
      if (cs) {
        const float2 k = cs[(size_t)b * HALF + i];
        r0 = a * k.x - c * k.y;
        r1 = a * k.y + c * k.x;
      }
      kc[i0] = from_f32<bf16_t>(r0);
      kc[i1] = from_f32<bf16_t>(r1);
    }
    for (int i = threadIdx.x; i < DH; i += 256) {
      float v = to_f32(vraw[i]);
      if (vbias) v += vbias[i];
      vc[(size_t)i * TA_PAGE] = from_f32<bf16_t>(v);
    }
    __syncthreads();     // the condition above is the same for every thread of the workgroup
  }

  const int vis_start = (window > 0 && kv_len > window) ? kv_len - window : 0;
  const int n_pages = (kv_len + TA_PAGE - 1) / TA_PAGE;
  int pg_lo = unit_first;
  int pg_hi = unit_first + unit_count;
  if (pg_hi > n_pages) pg_hi = n_pages;
  if (vis_start / TA_PAGE > pg_lo) pg_lo = vis_start / TA_PAGE;
  if (pg_lo >= pg_hi) {
    // a slice past this sequence's end or before its window (never the slice that stored the
    // new key): it says so in its (max, sum) and the merge passes over it
    if (splits > 1 && wave == 0 && kb == 0 && row_ok) {
      float* pr = partial + ((size_t)blockIdx.y * nh + head) * (DH + 2);
      pr[DH] = -INFINITY;
      pr[DH + 1] = 0.f;
    }
    return;
  }

  // Two pages are on their way while a third is multiplied: a workgroup's walk is a chain of
  // memory latencies otherwise. The loads are issued without conditions (a page past the
  // slice reads one harmless address in every lane), so that the waits can count them.
  const int* table = block_table + (size_t)b * max_blocks;
  u32x4 kreg[2][PER], vreg[2][PER];
  int next_page = pg_lo == unit_first ? unit[4] : table[pg_lo];      // a window may have moved pg_lo
  // the page number of a fetch was looked up a step earlier (`next_page`), so the fetch does
  // not wait for the table
#define LOOK_UP(pg_) table[(pg_) < pg_hi ? (pg_) : pg_lo]
#define FETCH_PAGE(set, pg_)                                                         \
  do {                                                                               \
    const bool live_ = (pg_) < pg_hi;                                                \
    const size_t page_ = (size_t)next_page;                                          \
    next_page = ((pg_) == unit_first && unit_count > 1) ? unit[5] : LOOK_UP((pg_) + 1); \
    const bf16_t* kp_ = kcache + (page_ * nkv + kvh) * (size_t)(TA_PAGE * DH);       \
    const bf16_t* vp_ = vcache + (page_ * nkv + kvh) * (size_t)(TA_PAGE * DH);       \
    _Pragma("unroll") for (int i = 0; i < PER; ++i) {                                \
      const size_t at_ = live_ ? (size_t)(threadIdx.x + i * 256) * 8 : 0;            \
      kreg[set][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kp_ + at_)); \
      vreg[set][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vp_ + at_)); \
    }                                                                                \
  } while (0)

  // ---- q of this lane's head: step t holds elements t*16 + kb*4 .. +3 of the low half in
  // h[0] and their partners DH/2 further on in h[1]; bias and rotation applied here. All
  // loads are issued first and without conditions (a lane without a head reads head 0 of its
  // group, absent angles or bias read the first bytes of the token's row and are not used):
  // one wait, not one per step.
  Frag16 qf[KT];
  {
    const bf16_t* qp = tokrow + (size_t)head * DH;
    const float* dummy = reinterpret_cast<const float*>(tokrow);
    const float* ctf = cs ? reinterpret_cast<const float*>(cs + (size_t)b * HALF) : dummy;
    const float* qb = bias ? bias + (size_t)head * DH : dummy;
    floatx4 ang0[KT], ang1[KT], bl[KT], bh[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) {
      const int d0 = t * 16 + kb * 4;
      qf[t].h[0] = *reinterpret_cast<const u32x2*>(qp + d0);
      qf[t].h[1] = *reinterpret_cast<const u32x2*>(qp + HALF + d0);
      // angles (cos, sin): pairs (d, d + DH/2) turn by angle d; pairs (2i, 2i + 1) by angle i
      const int i0 = style == 0 ? d0 : d0 / 2, i1 = style == 0 ? d0 + 2 : (HALF + d0) / 2;
      ang0[t] = *reinterpret_cast<const floatx4*>(ctf + (cs ? 2 * i0 : 0));
      ang1[t] = *reinterpret_cast<const floatx4*>(ctf + (cs ? 2 * i1 : 0));
      bl[t] = *reinterpret_cast<const floatx4*>(qb + (bias ? d0 : 0));
      bh[t] = *reinterpret_cast<const floatx4*>(qb + (bias ? HALF + d0 : 0));
    }
    // the first pages are asked for behind them: loads return in order, so the rotation
    // below waits for q alone and runs while the pages are on their way
    FETCH_PAGE(0, pg_lo);
    FETCH_PAGE(1, pg_lo + 1);
    if (cs != nullptr || bias != nullptr) {
#pragma unroll
      for (int t = 0; t < KT; ++t) {
        float lo[4], hi[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t wl = qf[t].w[e / 2], wh = qf[t].w[2 + e / 2];
          lo[e] = __uint_as_float((e & 1) ? (wl & 0xffff0000u) : (wl << 16));
          hi[e] = __uint_as_float((e & 1) ? (wh & 0xffff0000u) : (wh << 16));
          if (bias) {
            lo[e] += bl[t][e];
            hi[e] += bh[t][e];
          }
        }
        if (cs) {
          if (style == 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float c = e < 2 ? ang0[t][2 * e] : ang1[t][2 * e - 4];
              const float sn = e < 2 ? ang0[t][2 * e + 1] : ang1[t][2 * e - 3];
              const float r0 = lo[e] * c - hi[e] * sn, r1 = lo[e] * sn + hi[e] * c;
              lo[e] = r0;
              hi[e] = r1;
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; e += 2) {
              const float cl = ang0[t][e], sl = ang0[t][e + 1], ch = ang1[t][e], sh = ang1[t][e + 1];
              const float l0 = lo[e] * cl - lo[e + 1] * sl, l1 = lo[e] * sl + lo[e + 1] * cl;
              const float h0 = hi[e] * ch - hi[e + 1] * sh, h1 = hi[e] * sh + hi[e + 1] * ch;
              lo[e] = l0;
              lo[e + 1] = l1;
              hi[e] = h0;
              hi[e + 1] = h1;
            }
          }
        }
        qf[t].w[0] = pack2(lo[0], lo[1]);
        qf[t].w[1] = pack2(lo[2], lo[3]);
        qf[t].w[2] = pack2(hi[0], hi[1]);
        qf[t].w[3] = pack2(hi[2], hi[3]);
      }
    }
    if (!row_ok) {
#pragma unroll
      for (int t = 0; t < KT; ++t) qf[t].q = u32x4{0, 0, 0, 0};
    }
  }

  floatx4 o[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i) o[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // one page: `SET` names the registers that hold it. A step past the slice's last page keeps
  // the barriers and the loads and skips the rest.
  auto step = [&](auto set_tag, int pg) {
    constexpr int SET = decltype(set_tag)::value;
    const bool live = pg < pg_hi;
    const int key0 = pg * TA_PAGE;
    __syncthreads();                               // everyone is done with the previous page
    if (live) {
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int piece = threadIdx.x + i * 256;
        const int krow = piece / (DH / 8), kcol = (piece % (DH / 8)) * 8;
        *reinterpret_cast<u32x4*>(Ks + krow * KSTR + kcol) = kreg[SET][i];
        const int vrow = piece / (TA_PAGE / 8), vcol = (piece % (TA_PAGE / 8)) * 8;
        uint4 v = make_uint4(vreg[SET][i].x, vreg[SET][i].y, vreg[SET][i].z, vreg[SET][i].w);
        if (key0 + vcol + 8 > kv_len) {              // keys that no step has written read as zero
          uint2 lo = make_uint2(v.x, v.y), hi = make_uint2(v.z, v.w);
          lo = zero_from(lo, key0 + vcol, kv_len);
          hi = zero_from(hi, key0 + vcol + 4, kv_len);
          v = make_uint4(lo.x, lo.y, hi.x, hi.y);
        }
        *reinterpret_cast<uint2*>(Vs + vrow * VSTR + vcol) = make_uint2(v.x, v.y);
        *reinterpret_cast<uint2*>(Vs + vrow * VSTR + vcol + 4) = make_uint2(v.z, v.w);
      }
    }
    __syncthreads();
    FETCH_PAGE(SET, pg + 2);                       // in flight while this page and the next are multiplied
    if (live) {
      // ---- scores of this wave's 16 keys: register i is key 16*wave + 4*kb + i, head n
      floatx4 s = floatx4{0.f, 0.f, 0.f, 0.f};
      const bf16_t* krow = Ks + (16 * wave + n) * KSTR + kb * 4;   // as first operand, n is the key
#pragma unroll
      for (int t = 0; t < KT; ++t) {
        Frag16 a;
        a.h[0] = *reinterpret_cast<const u32x2*>(krow + t * 16);
        a.h[1] = *reinterpret_cast<const u32x2*>(krow + HALF + t * 16);
        s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, qf[t].v, s, 0, 0, 0);
      }
      const int kfirst = key0 + 16 * wave + 4 * kb;
      if (kfirst + 4 > kv_len || kfirst < vis_start) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (kfirst + i >= kv_len || kfirst + i < vis_start) s[i] = -INFINITY;
      }
      float mx = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
      mx = max_xor32(max_xor16(mx));
      const float m_new = fmaxf(m, mx * scale_log2);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m - m_use);
      float p[4], rs = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p[i] = __builtin_amdgcn_exp2f(fmaf(s[i], scale_log2, -m_use));
        rs += p[i];
      }
      rs = sum_xor32(sum_xor16(rs));
      l = l * alpha + rs;
      m = m_new;
      Frag8 pb;                                      // P^T as second operand: 4 keys of head n
      pb.w[0] = pack2(p[0], p[1]);
      pb.w[1] = pack2(p[2], p[3]);
      // ---- values: O^T tile dt holds head dims dt*16 + 4*kb + i of head n
      const bf16_t* vrow = Vs + n * VSTR + 16 * wave + 4 * kb;     // as first operand, n is the dim
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        Frag8 a;
        a.q = *reinterpret_cast<const u32x2*>(vrow + dt * 16 * VSTR);
#pragma unroll
        for (int i = 0; i < 4; ++i) o[dt][i] *= alpha;
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, pb.v, o[dt], 0, 0, 0);
      }
    }
  };
  for (int pg = pg_lo; pg < pg_hi; pg += 2) {
    step(std::integral_constant<int, 0>{}, pg);
    step(std::integral_constant<int, 1>{}, pg + 1);
  }
#undef FETCH_PAGE
#undef LOOK_UP

  // ---- merge the four waves: ml[4][16][2] then o[4][16][DH], in the pages' memory
  __syncthreads();
  float* ml = reinterpret_cast<float*>(lds_raw);
  float* os = ml + 4 * 16 * 2;
  if (kb == 0) {
    ml[(wave * 16 + n) * 2 + 0] = m;
    ml[(wave * 16 + n) * 2 + 1] = l;
  }
  {
    float* dst = os + ((size_t)wave * 16 + n) * DH + 4 * kb;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      *reinterpret_cast<floatx4*>(dst + dt * 16) = o[dt];
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < nrows * DH; idx += 256) {
    const int r = idx / DH, d = idx - r * DH;
    float mm = -INFINITY;
#pragma unroll
    for (int wv = 0; wv < 4; ++wv) mm = fmaxf(mm, ml[(wv * 16 + r) * 2]);
    const float m_use = (mm == -INFINITY) ? 0.f : mm;
    float acc = 0.f, ll = 0.f;
#pragma unroll
    for (int wv = 0; wv < 4; ++wv) {
      const float f = __builtin_amdgcn_exp2f(ml[(wv * 16 + r) * 2] - m_use);
      acc += f * os[((size_t)wv * 16 + r) * DH + d];
      ll += f * ml[(wv * 16 + r) * 2 + 1];
    }
    const int hd = kvh * group + hg0 + r;
    if (splits == 1) {
      const float inv = ll > 0.f ? 1.0f / ll : 0.f;
      out[(size_t)b * out_stride + (size_t)hd * DH + d] = from_f32<bf16_t>(acc * inv);
    } else {
      float* pr = partial + ((size_t)blockIdx.y * nh + hd) * (DH + 2);
      pr[d] = acc;
      if (d == 0) {
        pr[DH] = mm;
        pr[DH + 1] = ll;
      }
    }
  }
}

// grid (nh, batch), DH threads: merges the units of one (sequence, head); a sequence with
// one unit has its rows already. The partial rows of up to eight units are asked for at once
// (their maxima, sums and this thread's element), so that the kernel is two trips to memory
// behind its launch and not one per pass over the units.
template <int DH>
__global__ void attn_merge_kernel(const float* __restrict__ partial, bf16_t* __restrict__ out,
                                  int out_stride, int nh, const int* __restrict__ seq_units) {
  const int hd = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const int first = seq_units[2 * b], splits = seq_units[2 * b + 1];
  if (splits <= 1) return;
  const float* pr = partial + ((size_t)first * nh + hd) * (DH + 2);
  const size_t step = (size_t)nh * (DH + 2);
  constexpr int AHEAD = 8;
  float mm = -INFINITY, acc = 0.f, ll = 0.f;       // running maximum, and sums relative to it
  for (int s0 = 0; s0 < splits; s0 += AHEAD) {
    float ms[AHEAD], ls[AHEAD], os[AHEAD];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) {
      const int s = s0 + i < splits ? s0 + i : s0;   // past the end: the group's first unit again, not used
      ms[i] = pr[s * step + DH];
      ls[i] = pr[s * step + DH + 1];
      os[i] = pr[s * step + d];
    }
    float gm = mm;
#pragma unroll
    for (int i = 0; i < AHEAD; ++i)
      if (s0 + i < splits) gm = fmaxf(gm, ms[i]);
    const float m_use = (gm == -INFINITY) ? 0.f : gm;
    const float keep = (mm == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mm - m_use);
    acc *= keep;
    ll *= keep;
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) {
      if (s0 + i >= splits || ms[i] == -INFINITY) continue;   // an empty unit wrote nothing but its (max, sum)
      const float f = __builtin_amdgcn_exp2f(ms[i] - m_use);
      acc += f * os[i];
      ll += f * ls[i];
    }
    mm = gm;
  }
  const float inv = ll > 0.f ? 1.0f / ll : 0.f;
  out[(size_t)b * out_stride + (size_t)hd * DH + d] = from_f32<bf16_t>(acc * inv);
}

// ------------------------------------------------------------------ host side
static int check_common(const char* what, int batch, int nh, int nkv, int dh, int q_stride,
                        int out_stride, int max_blocks, const void* q, const void* out) {
  TA_REQUIRE(batch >= 0 && batch <= 65535, "%s: batch %d outside [0, 65535]", what, batch);
  TA_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "%s: %d heads do not divide into %d kv heads", what, nh, nkv);
  TA_REQUIRE(dh % 32 == 0 && dh >= 32 && dh <= 256,
             "%s: the matrix-core kernel takes head sizes 32, 64, ..., 256, not %d", what, dh);
  TA_REQUIRE(q_stride >= nh * dh && out_stride >= nh * dh, "%s: strides too small", what);
  TA_REQUIRE(q_stride % 8 == 0 && out_stride % 4 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 8) == 0,
             "%s: q rows must be 16-byte aligned and out rows 8-byte aligned", what);
  TA_REQUIRE(max_blocks > 0, "%s: empty block table", what);
  return 0;
}

#define DISPATCH_DH(dh, CALL)                   \
  switch (dh) {                                 \
    case 32: { constexpr int DH = 32; CALL; } break;   \
    case 64: { constexpr int DH = 64; CALL; } break;   \
    case 96: { constexpr int DH = 96; CALL; } break;   \
    case 128: { constexpr int DH = 128; CALL; } break; \
    case 160: { constexpr int DH = 160; CALL; } break; \
    case 192: { constexpr int DH = 192; CALL; } break; \
    case 224: { constexpr int DH = 224; CALL; } break; \
    case 256: { constexpr int DH = 256; CALL; } break; \
    default: return ta_fail("head size %d has no matrix-core kernel", dh); \
  }

static const float LOG2E = 1.4426950408889634f;

// Prompts (any mix of lengths, also single tokens). Same arguments as ta_attention_generic.
extern "C" int ta_attention_rows_bf16(hipStream_t stream, const void* q, int q_stride, void* out,
                                      int out_stride, const void* kcache, const void* vcache,
                                      const int* block_table, int max_blocks, const int* cu_q,
                                      const int* pos0, int batch, int max_qlen, int nh, int nkv,
                                      int dh, float scale, int window, int use_lds) {
  if (check_common("ta_attention_rows_bf16", batch, nh, nkv, dh, q_stride, out_stride, max_blocks, q, out)) return 1;
  TA_REQUIRE(max_qlen >= 0 && nkv <= 65535, "ta_attention_rows_bf16: bad max_qlen=%d or nkv=%d", max_qlen, nkv);
  if (batch == 0 || max_qlen == 0) return 0;
  const int group = nh / nkv;
  const long long rows = (long long)max_qlen * group;
  TA_REQUIRE(use_lds >= 0 && use_lds <= 2, "ta_attention_rows_bf16: unknown kernel %d", use_lds);
  dim3 g((unsigned)((rows + 127) / 128), nkv, batch), blk(256);
  if (use_lds == 2) {
    TA_REQUIRE(dh <= 128, "ta_attention_rows_bf16: the kernel that overlaps by half pages takes head sizes up to 128 (%d)", dh);
    // two blocks of rows per workgroup once that still fills every CU twice (two workgroups
    // share one); 2: one block each, all on the CUs at once, see the kernel
    const long long blocks = (long long)g.x * nkv * batch;
    int cus = 0, device = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)
      return ta_fail("ta_attention_rows_bf16: the device does not tell its number of CUs");
    int pair = blocks >= 4LL * cus;
    if (pair) g.x = (g.x + 1) / 2;
    else if (blocks <= 2LL * cus) pair = 2;
    TA_REQUIRE(g.x <= 65535, "ta_attention_rows_bf16: prompt too long for one launch");
    g = dim3(nkv, g.x, batch);          // kv heads vary fastest: see below
#define HALVES_CALL(DHV)                                                                              \
  attn_rows_halves_kernel<DHV><<<g, blk, 0, stream>>>((const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, \
                                                      (const bf16_t*)kcache, (const bf16_t*)vcache, block_table, \
                                                      max_blocks, cu_q, pos0, nh, nkv, scale * LOG2E, window, pair)
    switch (dh) {
      case 32: HALVES_CALL(32); break;
      case 64: HALVES_CALL(64); break;
      case 96: HALVES_CALL(96); break;
      default: HALVES_CALL(128); break;
    }
#undef HALVES_CALL
    return ta_check_launch("ta_attention_rows_bf16");
  }
  // long prompts share pages through LDS; short ones (little reuse, few rows) read them directly
  if (use_lds && dh <= 192) {        // beyond that a page and its padding outgrow 64 KB of LDS
    // two blocks of rows per workgroup once that still leaves a workgroup for every CU
    // (measured: below that the lost parallelism costs more than the balance gains)
    const int pair = (long long)g.x * nkv * batch >= 512;
    if (pair) g.x = (g.x + 1) / 2;
    // Consecutive workgroups go to the eight XCDs in turn, each with an L2 of its own. With the
    // kv head as the fastest index an XCD sees the pages of nkv / 8 heads only, which fit its
    // L2; with the row blocks fastest every XCD read every head's pages and they did not.
    TA_REQUIRE(g.x <= 65535, "ta_attention_rows_bf16: prompt too long for one launch");
    g = dim3(nkv, g.x, batch);
    DISPATCH_DH(dh, (attn_rows_lds_kernel<DH><<<g, blk, 0, stream>>>(
                        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kcache,
                        (const bf16_t*)vcache, block_table, max_blocks, cu_q, pos0, nh, nkv,
                        scale * LOG2E, window, pair)));
  } else {
    DISPATCH_DH(dh, (attn_rows_kernel<DH><<<g, blk, 0, stream>>>(
                        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kcache,
                        (const bf16_t*)vcache, block_table, max_blocks, cu_q, pos0, nh, nkv,
                        scale * LOG2E, window)));
  }
  return ta_check_launch("ta_attention_rows_bf16");
}

// Floats of scratch the single-token kernels need for `n_units` units of work.
extern "C" long long ta_attention_keys_scratch(int n_units, int nh, int dh) {
  return (long long)n_units * nh * (dh + 2);
}

// Single tokens: sequence b brings row b of qkv. The work is cut into n_units units:
// units [n_units][8] int32 on the device = (sequence, first page, pages, the sequence's length
// with this token, page numbers of the unit's first two pages, units of the sequence, 0), a
// unit of 0 pages being a spare one; seq_units [batch][2] = (first unit, units) of each
// sequence, whose units follow one another and cover its pages in order. The caller sees to it that they fit the
// block table. A sequence with one unit gets its rows directly, the others through scratch
// (ta_attention_keys_scratch floats) and a merge.
// waves: 4 or 8 waves per workgroup take the pages of a unit in turn and are merged
// through LDS; 0 and 1: four waves bring the pages in together through LDS (head sizes
// <= 192), 0 with a quarter of a page's keys per wave and up to 16 heads per kv head in a
// workgroup, 1 with all keys in every wave and up to 32 heads.
// Plain use: qkv holds rotated q heads (q_stride elements between tokens) and the cache
// already holds the step's keys and values: bias, cs and dest are null.
// Fused use: qkv = [q | k | v] raw projections; bias (float32 per column) is added, q and k
// are rotated by cs ([batch][dh/2] (cos, sin); null: no rotation; style 0 pairs (j, j+dh/2),
// 1 pairs (2j, 2j+1)) and the new key and value are stored at dest[b] = page * 64 + offset.
extern "C" int ta_attention_keys_bf16(hipStream_t stream, const void* qkv, int q_stride,
                                      const float* bias, const float* cs, int style,
                                      const int* dest, void* out, int out_stride, void* kcache,
                                      void* vcache, const int* block_table, int max_blocks,
                                      const int* pos0, int batch, int nh, int nkv, int dh,
                                      float scale, int window, const int* units,
                                      const int* seq_units, int n_units, int waves, float* scratch) {
  if (check_common("ta_attention_keys_bf16", batch, nh, nkv, dh, q_stride, out_stride, max_blocks, qkv, out)) return 1;
  TA_REQUIRE(n_units >= batch && n_units <= 65535 && units != nullptr && seq_units != nullptr,
             "ta_attention_keys_bf16: %d units of work for %d sequences", n_units, batch);
  TA_REQUIRE(scratch != nullptr, "ta_attention_keys_bf16: units need scratch memory");
  TA_REQUIRE(waves == 0 || waves == 1 || waves == 4 || waves == 8,
             "ta_attention_keys_bf16: waves per workgroup must be 4 or 8, or 0 or 1 for the kernels that share pages through LDS (%d)", waves);
  TA_REQUIRE(waves > 1 || dh <= 192, "ta_attention_keys_bf16: the LDS kernels take head sizes up to 192");
  TA_REQUIRE(style == 0 || style == 1, "ta_attention_keys_bf16: unknown pairing style %d", style);
  TA_REQUIRE((uintptr_t)cs % 16 == 0 && (uintptr_t)bias % 16 == 0,
             "ta_attention_keys_bf16: angles and bias must be 16-byte aligned");
  TA_REQUIRE(dest == nullptr || q_stride >= (nh + 2 * nkv) * dh,
             "ta_attention_keys_bf16: the fused form needs q, k and v in one row");
  if (batch == 0) return 0;
  const int group = nh / nkv;
  const int chunks = waves == 0 ? (group + 15) / 16 : (group + 31) / 32;
  TA_REQUIRE((long long)nkv * chunks <= 0x7fffffff, "ta_attention_keys_bf16: too many heads for one launch");
  const int nrows = group < 32 ? group : 32;
  // slices are the slowest index: consecutive workgroups, which go to the eight XCDs in
  // turn, are heads and sequences of one slice, so late slices, which short sequences do
  // not have, leave no XCD idle; the full early slices also start first
  dim3 g(nkv * chunks, n_units), blk(waves > 1 ? waves * 64 : 256);
  const size_t lds = waves > 1 ? (size_t)(waves * 32 * 2 + waves * nrows * dh) * sizeof(float) : 0;
  TA_REQUIRE(lds <= 65536, "ta_attention_keys_bf16: %zu bytes of LDS needed, 65536 available", lds);
#define KEYS_ARGS                                                                                  \
  (const bf16_t*)qkv, q_stride, bias, (const float2*)cs, style, dest, (bf16_t*)out, out_stride,    \
      (bf16_t*)kcache, (bf16_t*)vcache, block_table, max_blocks, pos0, nh, nkv, scale * LOG2E,     \
      window, units, seq_units, scratch
  if (waves == 0) {
    DISPATCH_DH(dh, (attn_keys_q16_kernel<DH><<<g, blk, 0, stream>>>(KEYS_ARGS)));
  } else if (waves == 1) {
    DISPATCH_DH(dh, (attn_keys_lds_kernel<DH><<<g, blk, 0, stream>>>(KEYS_ARGS)));
  } else if (waves == 8) {
    DISPATCH_DH(dh, (attn_keys_kernel<DH, 8><<<g, blk, lds, stream>>>(KEYS_ARGS)));
  } else {
    DISPATCH_DH(dh, (attn_keys_kernel<DH, 4><<<g, blk, lds, stream>>>(KEYS_ARGS)));
  }
#undef KEYS_ARGS
  if (ta_check_launch("ta_attention_keys_bf16")) return 1;
  dim3 g2(nh, batch);
  DISPATCH_DH(dh, (attn_merge_kernel<DH><<<g2, DH, 0, stream>>>(scratch, (bf16_t*)out, out_stride, nh,
                                                               seq_units)));
  return ta_check_launch("ta_attention_keys_bf16 (merge)");
  return 0;
}

// ------------------------------------------------------------------ no allocation
// See no_alloc.h. The array's name is only a handle in host code: its address on the
// current GPU comes from hipGetSymbolAddress, once per GPU, and that pointer is what the
// kernels are given.
#include <mutex>
#include "no_alloc.h"

static __device__ __align__(256) float ta_noalloc_scratch[TA_NOALLOC_SCRATCH_FLOATS];

#define TA_NOALLOC_MAX_DEVICES 64
static float* g_noalloc_ptr[TA_NOALLOC_MAX_DEVICES] = {nullptr};
static std::mutex g_noalloc_lock;

static int noalloc_scratch(float** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return ta_fail("ta_attention_keys_bf16_noalloc: hipGetDevice: %s", hipGetErrorString(e));
  TA_REQUIRE(dev >= 0 && dev < TA_NOALLOC_MAX_DEVICES, "ta_attention_keys_bf16_noalloc: device %d", dev);
  std::lock_guard<std::mutex> hold(g_noalloc_lock);
  if (g_noalloc_ptr[dev] == nullptr) {
    float* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(ta_noalloc_scratch));
    if (e != hipSuccess || p == nullptr)
      return ta_fail("ta_attention_keys_bf16_noalloc: the static scratch buffer has no address on device %d: %s",
                     dev, hipGetErrorString(e));
    g_noalloc_ptr[dev] = p;
  }
  *ptr = g_noalloc_ptr[dev];
  return 0;
}

extern "C" long long ta_noalloc_scratch_floats() { return TA_NOALLOC_SCRATCH_FLOATS; }

extern "C" int ta_attention_keys_bf16_noalloc(hipStream_t stream, const void* qkv, int q_stride,
                                              const float* bias, const float* cs, int style,
                                              const int* dest, void* out, int out_stride,
                                              void* kcache, void* vcache, const int* block_table,
                                              int max_blocks, const int* pos0, int batch, int nh,
                                              int nkv, int dh, float scale, int window,
                                              const int* units, const int* seq_units, int n_units,
                                              int waves) {
  TA_REQUIRE(n_units >= 0 && nh > 0 && dh > 0, "ta_attention_keys_bf16_noalloc: bad sizes units=%d nh=%d dh=%d",
             n_units, nh, dh);
  const long long need = ta_attention_keys_scratch(n_units, nh, dh);
  TA_REQUIRE(need <= (long long)TA_NOALLOC_SCRATCH_FLOATS,
             "ta_attention_keys_bf16_noalloc: %d units of %d heads of %d need %lld floats of scratch, the "
             "static buffer holds %d; use fewer units or ta_attention_keys_bf16 with a buffer of the caller's",
             n_units, nh, dh, need, TA_NOALLOC_SCRATCH_FLOATS);
  float* scratch = nullptr;
  if (noalloc_scratch(&scratch)) return 1;
  return ta_attention_keys_bf16(stream, qkv, q_stride, bias, cs, style, dest, out, out_stride, kcache,
                                vcache, block_table, max_blocks, pos0, batch, nh, nkv, dh, scale, window,
                                units, seq_units, n_units, waves, scratch);
}
