// Next-token choice from float32 logits: argmax, and sampling from
// softmax(logits / temperature) restricted by top-k and top-p.
//
// Sampling works on fixed-point probabilities q_i = floor(2^40 * exp2((l_i - max) / T * log2 e)),
// so every sum is an integer sum: the kept set and the drawn token do not depend
// on the order in which threads add, and a row gives the same token in any batch.
// Order of preference: higher logit first, lower index first among equals. Kept
// are the first top_k tokens of that order, cut after the token with which the
// kept probability reaches top_p. The token drawn for a uniform u in [0,1) is the
// first kept token, in index order, whose running sum exceeds floor(u * kept sum).
#include "common.h"

#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / TA_WAVE)
typedef unsigned long long u64;

__device__ __forceinline__ uint32_t order_key(float l) {
  const uint32_t b = __float_as_uint(l);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
// floor(2^40 * exp((l - m) / T)) from the hardware's exp2 and two 32-bit conversions: the
// library's expf and a float-to-64-bit conversion are some fifty instructions, and a row of
// 128 K tokens on one CU is bound by exactly these
__device__ __forceinline__ u64 fixed_mass(float l, float m, float inv_t) {
  const float w = __builtin_amdgcn_exp2f((l - m) * inv_t * 1.44269504088896341f);   // in [0, 1]
  const float upper = w * 1048576.0f;                    // 2^20; exact, as is what follows
  const uint32_t hi = (uint32_t)upper;
  const uint32_t lo = (uint32_t)((upper - (float)hi) * 1048576.0f);
  return ((u64)hi << 20) + lo;
}
__device__ __forceinline__ u64 shfl_xor_u64(u64 v, int o) {
  uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
  lo = __shfl_xor(lo, o, TA_WAVE);
  hi = __shfl_xor(hi, o, TA_WAVE);
  return ((u64)hi << 32) | lo;
}
__device__ __forceinline__ u64 shfl_up_u64(u64 v, int o) {
  uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
  lo = __shfl_up(lo, o, TA_WAVE);
  hi = __shfl_up(hi, o, TA_WAVE);
  return ((u64)hi << 32) | lo;
}

// ------------------------------------------------------------------ argmax
// Highest logit; among equals the lowest index.
__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_kernel(const float* __restrict__ logits,
                                                                 size_t ld, int vocab,
                                                                 int* __restrict__ out) {
  const float* row = logits + (size_t)blockIdx.x * ld;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  // a thread meets its indices in ascending order, so among equals the first one stays
#define CONSIDER(v_, i_)                                          \
  do {                                                            \
    const float cv_ = (v_);                                       \
    if (cv_ > best || bi == 0x7fffffff) {                         \
      if (!(cv_ < best)) { /* NaN never wins over a number already held */ \
        best = cv_;                                               \
        bi = (i_);                                                \
      }                                                           \
    }                                                             \
  } while (0)
  int done = 0;
  if (((uintptr_t)row % 16) == 0) {
    // sixteen bytes per lane; a single workgroup per row is bound by what one CU can load
    const float4* row4 = reinterpret_cast<const float4*>(row);
    const int n4 = vocab / 4;
    // eight loads on their way per thread: with one, a row of 128 K logits took 22 us
    constexpr int AHEAD = 8;
    int j = threadIdx.x;
    for (; j + (AHEAD - 1) * SAMPLE_THREADS < n4; j += AHEAD * SAMPLE_THREADS) {
      float4 v[AHEAD];
#pragma unroll
      for (int u = 0; u < AHEAD; ++u) v[u] = row4[j + u * SAMPLE_THREADS];
#pragma unroll
      for (int u = 0; u < AHEAD; ++u) {
        const int jj = j + u * SAMPLE_THREADS;
        CONSIDER(v[u].x, 4 * jj);
        CONSIDER(v[u].y, 4 * jj + 1);
        CONSIDER(v[u].z, 4 * jj + 2);
        CONSIDER(v[u].w, 4 * jj + 3);
      }
    }
    for (; j < n4; j += SAMPLE_THREADS) {
      const float4 v = row4[j];
      CONSIDER(v.x, 4 * j);
      CONSIDER(v.y, 4 * j + 1);
      CONSIDER(v.z, 4 * j + 2);
      CONSIDER(v.w, 4 * j + 3);
    }
    done = n4 * 4;
  }
  for (int i = done + threadIdx.x; i < vocab; i += SAMPLE_THREADS) CONSIDER(row[i], i);
#undef CONSIDER
#pragma unroll
  for (int o = TA_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, TA_WAVE);
    const int oi = __shfl_xor(bi, o, TA_WAVE);
    if (ov > best || (ov == best && oi < bi)) {
      best = ov;
      bi = oi;
    }
  }
  __shared__ float sv[SAMPLE_WAVES];
  __shared__ int si[SAMPLE_WAVES];
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  if (lane == 0) {
    sv[wave] = best;
    si[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SAMPLE_WAVES; ++w)
      if (sv[w] > best || (sv[w] == best && si[w] < bi)) {
        best = sv[w];
        bi = si[w];
      }
    out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
  }
}

extern "C" int ta_argmax(hipStream_t stream, const float* logits, long long ld, int n, int vocab,
                         int* out) {
  TA_REQUIRE(n >= 0 && vocab > 0 && ld >= vocab, "ta_argmax: bad sizes n=%d vocab=%d ld=%lld", n, vocab, ld);
  if (n == 0) return 0;
  argmax_kernel<<<n, SAMPLE_THREADS, 0, stream>>>(logits, (size_t)ld, vocab, out);
  return ta_check_launch("ta_argmax");
}

// ------------------------------------------------------------------ sampling
struct SelectState {
  uint32_t prefix, mask;
  uint32_t count_above;
  u64 mass_above;
  uint32_t tie_count;
  u64 tie_mass;
};

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, size_t ld, int vocab, float inv_t, int top_k, float top_p,
    const float* __restrict__ uniform, int* __restrict__ out) {
  const float* row = logits + (size_t)blockIdx.x * ld;
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  __shared__ float s_f[SAMPLE_WAVES];
  __shared__ u64 s_q[SAMPLE_WAVES];
  __shared__ uint32_t s_c[SAMPLE_WAVES];
  __shared__ uint32_t h_cnt[256];
  __shared__ u64 h_mass[256];
  __shared__ SelectState st;
  __shared__ float s_max;
  __shared__ u64 s_total;
  __shared__ int s_pick;

  // ---- max
  float m = -INFINITY;
  {
    int done = 0;
    if (((uintptr_t)row % 16) == 0) {
      const float4* row4 = reinterpret_cast<const float4*>(row);
      const int n4 = vocab / 4;
      for (int j = threadIdx.x; j < n4; j += SAMPLE_THREADS) {
        const float4 v = row4[j];
        m = fmaxf(fmaxf(m, v.x), fmaxf(fmaxf(v.y, v.z), v.w));
      }
      done = n4 * 4;
    }
    for (int i = done + threadIdx.x; i < vocab; i += SAMPLE_THREADS) m = fmaxf(m, row[i]);
  }
  m = wave_max(m);
  if (lane == 0) s_f[wave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    float mm = s_f[0];
    for (int w = 1; w < SAMPLE_WAVES; ++w) mm = fmaxf(mm, s_f[w]);
    s_max = mm;
  }
  __syncthreads();
  m = s_max;

  // ---- total mass (only the cuts need it; without them the sweeps below sum what is kept)
  const bool cut = top_k < vocab || top_p < 1.0f;
  u64 tot = 0;
  if (cut)
    for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) tot += fixed_mass(row[i], m, inv_t);
#pragma unroll
  for (int o = TA_WAVE / 2; o > 0; o >>= 1) tot += shfl_xor_u64(tot, o);
  if (lane == 0) s_q[wave] = tot;
  __syncthreads();
  if (threadIdx.x == 0) {
    u64 t = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) t += s_q[w];
    s_total = t;
    st.prefix = 0;
    st.mask = 0;
    st.count_above = 0;
    st.mass_above = 0;
    st.tie_count = 0xffffffffu;   // "every token of the threshold value is kept"
    st.tie_mass = 0;
    s_pick = 0;
  }
  __syncthreads();
  const u64 total = s_total;

  // ---- threshold of the kept set (only when top-k or top-p cut anything)
  if (cut) {
    const uint32_t k_lim = (uint32_t)(top_k < vocab ? top_k : vocab);
    u64 p_lim = (u64)ceil((double)top_p * (double)total);
    if (p_lim < 1) p_lim = 1;
    if (p_lim > total) p_lim = total;
    for (int pass = 0; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      for (int i = threadIdx.x; i < 256; i += SAMPLE_THREADS) {
        h_cnt[i] = 0;
        h_mass[i] = 0;
      }
      __syncthreads();
      const uint32_t prefix = st.prefix, mask = st.mask;
      for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
        const float l = row[i];
        const uint32_t key = order_key(l);
        if ((key & mask) == prefix) {
          const int bin = (key >> shift) & 255;
          atomicAdd(&h_cnt[bin], 1u);
          atomicAdd(&h_mass[bin], fixed_mass(l, m, inv_t));
        }
      }
      __syncthreads();
      if (threadIdx.x == 0) {
        uint32_t ca = st.count_above;
        u64 ma = st.mass_above;
        int chosen = -1;
        for (int bin = 255; bin >= 0; --bin) {
          if (h_cnt[bin] == 0) continue;
          if (ca + h_cnt[bin] >= k_lim || ma + h_mass[bin] >= p_lim) {
            chosen = bin;
            break;
          }
          ca += h_cnt[bin];
          ma += h_mass[bin];
        }
        // p_lim <= total, so the lowest non-empty bin reaches it at the latest
        if (chosen < 0) chosen = 0;
        st.count_above = ca;
        st.mass_above = ma;
        st.prefix = prefix | ((uint32_t)chosen << shift);
        st.mask = mask | (255u << shift);
        if (pass == 3) {
          const uint32_t c_t = h_cnt[chosen];
          const u64 q_t = c_t ? h_mass[chosen] / c_t : 0;
          uint32_t n = k_lim - ca;                       // >= 1
          if (q_t > 0) {
            const u64 need = (p_lim - ma + q_t - 1) / q_t;  // >= 1
            if (need < n) n = (uint32_t)need;
          }
          if (n > c_t) n = c_t;
          st.tie_count = n;
          st.tie_mass = q_t;
        }
      }
      __syncthreads();
    }
  }
  const uint32_t thr = st.prefix;          // 0 when nothing is cut: every key is > 0
  const uint32_t n_tie = st.tie_count;

  // ---- ordered sweeps: wave w owns the contiguous indices [w*span, (w+1)*span)
  const int span = ((vocab + SAMPLE_WAVES - 1) / SAMPLE_WAVES + TA_WAVE - 1) / TA_WAVE * TA_WAVE;
  const int lo = wave * span;
  const int hi = (lo + span < vocab) ? lo + span : vocab;
  const u64 lanes_below = ((u64)1 << lane) - 1;

  // sweep 1: threshold-valued tokens per wave -> rank base of each wave
  uint32_t ties = 0;
  for (int i0 = lo; i0 < hi; i0 += TA_WAVE) {
    const int i = i0 + lane;
    const bool tie = cut && i < hi && order_key(row[i]) == thr;
    ties += __popcll(__ballot(tie));
  }
  if (lane == 0) s_c[wave] = ties;
  __syncthreads();
  uint32_t tie_base = 0;
  for (int w = 0; w < wave; ++w) tie_base += s_c[w];
  __syncthreads();

  // sweep 2: kept mass per wave -> mass base of each wave
  u64 kept = 0;
  {
    uint32_t rank = tie_base;
    for (int i0 = lo; i0 < hi; i0 += TA_WAVE) {
      const int i = i0 + lane;
      bool keep = false, tie = false;
      float l = 0.f;
      if (i < hi) {
        l = row[i];
        const uint32_t key = order_key(l);
        tie = cut && key == thr;
        keep = !cut || key > thr;
      }
      const u64 b = __ballot(tie);
      if (tie && rank + __popcll(b & lanes_below) < n_tie) keep = true;
      rank += __popcll(b);
      if (keep) kept += fixed_mass(l, m, inv_t);
    }
  }
#pragma unroll
  for (int o = TA_WAVE / 2; o > 0; o >>= 1) kept += shfl_xor_u64(kept, o);
  if (lane == 0) s_q[wave] = kept;
  __syncthreads();
  u64 mass_base = 0, kept_total = 0;
  for (int w = 0; w < SAMPLE_WAVES; ++w) {
    if (w < wave) mass_base += s_q[w];
    kept_total += s_q[w];
  }
  u64 target = (u64)((double)uniform[blockIdx.x] * (double)kept_total);
  if (kept_total > 0 && target >= kept_total) target = kept_total - 1;

  // sweep 3: the wave whose range holds the target finds the token
  if (kept_total > 0 && target >= mass_base && target < mass_base + s_q[wave]) {
    uint32_t rank = tie_base;
    u64 run = mass_base;
    for (int i0 = lo; i0 < hi; i0 += TA_WAVE) {
      const int i = i0 + lane;
      bool keep = false, tie = false;
      float l = 0.f;
      if (i < hi) {
        l = row[i];
        const uint32_t key = order_key(l);
        tie = cut && key == thr;
        keep = !cut || key > thr;
      }
      const u64 b = __ballot(tie);
      if (tie && rank + __popcll(b & lanes_below) < n_tie) keep = true;
      rank += __popcll(b);
      const u64 q = keep ? fixed_mass(l, m, inv_t) : 0;
      u64 inc = q;                                   // inclusive scan over the wave
#pragma unroll
      for (int o = 1; o < TA_WAVE; o <<= 1) {
        const u64 up = shfl_up_u64(inc, o);
        if (lane >= o) inc += up;
      }
      const bool hit = q > 0 && run + inc > target && run + inc - q <= target;
      const u64 hb = __ballot(hit);
      if (hb) {
        if (hit) s_pick = i;
        break;
      }
      {  // the last lane holds the sum of this group of 64
        uint32_t lo32 = (uint32_t)inc, hi32 = (uint32_t)(inc >> 32);
        lo32 = __shfl(lo32, TA_WAVE - 1, TA_WAVE);
        hi32 = __shfl(hi32, TA_WAVE - 1, TA_WAVE);
        run += ((u64)hi32 << 32) | lo32;
      }
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = s_pick;
}

// Sum over the 64 lanes, the same in every lane, without going through the LDS crossbar:
// DPP moves inside a row of 16 lanes (1 apart, 2 apart, mirrored within 8, mirrored within 16),
// then the lane swaps of gfx950 across rows. A shuffle costs over a hundred cycles in a chain
// of its own; this is a dozen vector operations.
template <int CTRL>
__device__ __forceinline__ u64 dpp_move_u64(u64 v) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)v, CTRL, 0xf, 0xf, true);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_mov_dpp((int)(uint32_t)(v >> 32), CTRL, 0xf, 0xf, true);
  return ((u64)hi << 32) | lo;
}
__device__ __forceinline__ u64 wave_sum_u64(u64 v) {
  v += dpp_move_u64<0xB1>(v);
  v += dpp_move_u64<0x4E>(v);
  v += dpp_move_u64<0x141>(v);
  v += dpp_move_u64<0x140>(v);
  {
    const auto lo = __builtin_amdgcn_permlane16_swap((uint32_t)v, (uint32_t)v, false, false);
    const auto hi = __builtin_amdgcn_permlane16_swap((uint32_t)(v >> 32), (uint32_t)(v >> 32), false, false);
    v = (((u64)hi[0] << 32) | lo[0]) + (((u64)hi[1] << 32) | lo[1]);
  }
  {
    const auto lo = __builtin_amdgcn_permlane32_swap((uint32_t)v, (uint32_t)v, false, false);
    const auto hi = __builtin_amdgcn_permlane32_swap((uint32_t)(v >> 32), (uint32_t)(v >> 32), false, false);
    v = (((u64)hi[0] << 32) | lo[0]) + (((u64)hi[1] << 32) | lo[1]);
  }
  return v;
}

// a mass no row reaches (2^17 tokens of 2^40 each are 2^57), with room to add to it
#define NO_MASS_LIMIT ((u64)1 << 62)
#define CAND_PER_WAVE 256  // tokens near the maximum that a wave's share of the row may hold
#define NEAR_BINS 96       // steps of 1/9 counted one by one: down to e^-10.7 of the largest probability

// distance from the maximum in steps of 1/9 of (max - logit) / T; 255 holds all that is further
__device__ __forceinline__ int near_bin(float l, float m, float inv_t) {
  const float d = (m - l) * inv_t * 9.0f;
  return d < 255.0f ? (int)d : 255;
}

// One digit of the threshold key: the highest bin with which the count reaches k_lim or
// the mass p_lim. The last digit also settles how many tokens of the threshold value are
// kept (the lower indices among equals).
__device__ void choose_digit(SelectState& st, const uint32_t* h_cnt, const u64* h_mass, int shift,
                             bool last, uint32_t k_lim, u64 p_lim) {
  uint32_t ca = st.count_above;
  u64 ma = st.mass_above;
  int chosen = -1;
  for (int bin = 255; bin >= 0; --bin) {
    if (h_cnt[bin] == 0) continue;
    if (ca + h_cnt[bin] >= k_lim || ma + h_mass[bin] >= p_lim) {
      chosen = bin;
      break;
    }
    ca += h_cnt[bin];
    ma += h_mass[bin];
  }
  // p_lim <= total, so the lowest non-empty bin reaches it at the latest
  if (chosen < 0) chosen = 0;
  st.count_above = ca;
  st.mass_above = ma;
  st.prefix |= (uint32_t)chosen << shift;
  st.mask |= 255u << shift;
  if (last) {
    const uint32_t c_t = h_cnt[chosen];
    const u64 q_t = c_t ? h_mass[chosen] / c_t : 0;
    uint32_t n = k_lim - ca;                       // >= 1
    if (q_t > 0) {
      const u64 need = (p_lim - ma + q_t - 1) / q_t;  // >= 1
      if (need < n) n = (uint32_t)need;
    }
    if (n > c_t) n = c_t;
    st.tie_count = n;
    st.tie_mass = q_t;
  }
}

// The same choice for rows that start on 16-byte boundaries: every pass over the row brings
// sixteen bytes per lane. A pass that one thread walks four bytes at a time is a chain of
// its own loads; with vectors a pass is bound by what one CU can pull out of the L2, where
// the row (half a megabyte at 128 K tokens) stays after the first pass. All sums are integer
// sums and the sweeps keep the order of the indices, so this kernel and the one above choose
// the same token.
#define VEC_STEPS 64      // steps of 256 tokens whose sums a wave remembers (16 waves: 262,144 tokens)
struct Four {
  float v[4];
  bool ok[4];
};
// group j of the row: tokens 4j .. 4j+3. The row's stride is a multiple of four, so the last
// group may be read whole; what lies past the vocabulary is marked and reads as -inf. No
// branch: a loop can ask for several groups before it looks at the first.
__device__ __forceinline__ Four load_four(const float* __restrict__ row, int j, int vocab) {
  Four f;
  const float4 x = *reinterpret_cast<const float4*>(row + 4 * j);
  const float in[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    f.ok[e] = 4 * j + e < vocab;
    f.v[e] = f.ok[e] ? in[e] : -INFINITY;
  }
  return f;
}
// the same for a group that may lie past the row: then nothing of it is there
__device__ __forceinline__ Four load_four_if(const float* __restrict__ row, int j, int groups, int vocab) {
  return load_four(row, j < groups ? j : 0, j < groups ? vocab : 0);
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_vec_kernel(
    const float* __restrict__ logits, size_t ld, int vocab, float inv_t, int top_k, float top_p,
    const float* __restrict__ uniform, int* __restrict__ out) {
  const float* row = logits + (size_t)blockIdx.x * ld;
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  const int groups = (vocab + 3) / 4;                  // runs of four tokens
  __shared__ float s_f[SAMPLE_WAVES];
  __shared__ u64 s_q[SAMPLE_WAVES];
  __shared__ uint32_t s_c[SAMPLE_WAVES];
  __shared__ uint32_t h_cnt[256];
  __shared__ u64 h_mass[256];
  __shared__ SelectState st;
  __shared__ float s_max;
  __shared__ u64 s_total;
  __shared__ int s_pick;
  __shared__ u64 s_step[SAMPLE_WAVES][VEC_STEPS];      // kept mass of each step of a wave's range
  // tokens near the maximum, gathered in index order: wave w's share of the row in cand_*[w]
  __shared__ float cand_l[SAMPLE_WAVES][CAND_PER_WAVE];
  __shared__ int cand_i[SAMPLE_WAVES][CAND_PER_WAVE];
  __shared__ int s_ccnt[SAMPLE_WAVES];
  __shared__ int s_small;

  // ---- max
  float m = -INFINITY;
  // four groups are asked for before the first is looked at: one CU pulls what its loads in
  // flight allow, and a pass over the row is this kernel's unit of cost
  for (int j = threadIdx.x; j < groups; j += 4 * SAMPLE_THREADS) {
    Four f[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) f[u] = load_four_if(row, j + u * SAMPLE_THREADS, groups, vocab);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      m = fmaxf(fmaxf(m, f[u].v[0]), fmaxf(fmaxf(f[u].v[1], f[u].v[2]), f[u].v[3]));
  }
  m = wave_max(m);
  if (lane == 0) s_f[wave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    float mm = s_f[0];
    for (int w = 1; w < SAMPLE_WAVES; ++w) mm = fmaxf(mm, s_f[w]);
    s_max = mm;
  }
  __syncthreads();
  m = s_max;

  const bool cut = top_k < vocab || top_p < 1.0f;
  if (threadIdx.x == 0) {
    s_total = 0;
    st.prefix = 0;
    st.mask = 0;
    st.count_above = 0;
    st.mass_above = 0;
    st.tie_count = 0xffffffffu;   // "every token of the threshold value is kept"
    st.tie_mass = 0;
    s_pick = 0;
    s_small = 0;
  }
  for (int i = threadIdx.x; i < 256; i += SAMPLE_THREADS) {
    h_cnt[i] = 0;
    h_mass[i] = 0;
  }
  __syncthreads();

  // ---- with a cut: the tokens by their distance from the maximum, in steps of 1/9 of a
  // unit of (max - logit) / T. The sums give the total mass, and the step in which the count
  // reaches top_k or the mass reaches top_p bounds the kept set: usually a few hundred
  // tokens, which are then gathered into LDS and cut and drawn from there, so the row is
  // read three times in all instead of nine. When that step lies far from the maximum or
  // the tokens do not fit, the digits of the threshold are found over the whole row as in
  // the kernel above.
  if (cut) {
    // steps from NEAR_BINS on are lumped into the last one, summed in registers: most tokens
    // lie there, and the cut almost never does
    uint32_t far_cnt = 0;
    u64 far_mass = 0;
    const bool need_total = top_p < 1.0f;    // top-k alone never asks for the mass of the far tokens
    for (int j = threadIdx.x; j < groups; j += 4 * SAMPLE_THREADS) {
      Four f[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) f[u] = load_four_if(row, j + u * SAMPLE_THREADS, groups, vocab);
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (!f[u].ok[e]) continue;
          const int bin = near_bin(f[u].v[e], m, inv_t);
          if (bin < NEAR_BINS) {             // such a token has mass left by a wide margin
            atomicAdd(&h_cnt[bin], 1u);
            atomicAdd(&h_mass[bin], fixed_mass(f[u].v[e], m, inv_t));
          } else {
            ++far_cnt;
            if (need_total) far_mass += fixed_mass(f[u].v[e], m, inv_t);
          }
        }
    }
    far_cnt = (uint32_t)wave_sum_u64(far_cnt);
    far_mass = wave_sum_u64(far_mass);
    if (lane == 0 && far_cnt) {
      atomicAdd(&h_cnt[255], far_cnt);
      atomicAdd(&h_mass[255], far_mass);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      u64 t = 0;
      for (int bin = 0; bin < 256; ++bin) t += h_mass[bin];
      s_total = t;
      const uint32_t k_lim = (uint32_t)(top_k < vocab ? top_k : vocab);
      u64 p_lim = (u64)ceil((double)top_p * (double)t);
      if (p_lim < 1) p_lim = 1;
      if (p_lim > t) p_lim = t;
      if (top_p >= 1.0f) p_lim = NO_MASS_LIMIT;   // the far tokens' mass was not summed; nothing is cut by mass
      uint32_t ca = 0;
      u64 ma = 0;
      int last = 255;
      for (int bin = 0; bin < 256; ++bin) {
        ca += h_cnt[bin];
        ma += h_mass[bin];
        if (ca >= k_lim || ma >= p_lim) {
          last = bin;
          break;
        }
      }
      s_pick = last;                          // borrowed until the draw: the last step that matters
      s_small = t > 0 && last < NEAR_BINS && ca <= (uint32_t)(SAMPLE_WAVES * CAND_PER_WAVE);
    }
    __syncthreads();
  }
  const u64 total = s_total;
  const int near_last = s_pick;
  __syncthreads();
  if (threadIdx.x == 0) s_pick = 0;

  // ---- gather the tokens of the steps up to that one, wave by wave in index order
  const int span = ((groups + SAMPLE_WAVES - 1) / SAMPLE_WAVES + TA_WAVE - 1) / TA_WAVE * TA_WAVE;
  const int lo = wave * span;
  const int hi = (lo + span < groups) ? lo + span : groups;
  const u64 lanes_below = ((u64)1 << lane) - 1;
  if (cut && s_small) {
    int have = 0;
    for (int j0 = lo; j0 < hi; j0 += TA_WAVE) {
      const int j = j0 + lane;
      Four f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        f.v[e] = -INFINITY;
        f.ok[e] = false;
      }
      if (j < hi) f = load_four(row, j, vocab);
      bool take[4];
      int before = 0, all = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        take[e] = f.ok[e] && near_bin(f.v[e], m, inv_t) <= near_last;
        const u64 b = __ballot(take[e]);
        before += __popcll(b & lanes_below);
        all += __popcll(b);
      }
      int at = have + before;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (take[e]) {
          if (at < CAND_PER_WAVE) {
            cand_l[wave][at] = f.v[e];
            cand_i[wave][at] = 4 * j + e;
          }
          ++at;
        }
      have += all;
    }
    if (lane == 0) s_ccnt[wave] = have;
    __syncthreads();
    if (threadIdx.x == 0) {
      int ok = 1;
      for (int w = 0; w < SAMPLE_WAVES; ++w)
        if (s_ccnt[w] > CAND_PER_WAVE) ok = 0;         // a wave's share did not fit: the long way
      s_small = ok;
    }
    __syncthreads();
  }

  if (cut && s_small) {
    // ---- the cut among the gathered tokens (they hold every token at or above the threshold)
    const uint32_t k_lim = (uint32_t)(top_k < vocab ? top_k : vocab);
    u64 p_lim = (u64)ceil((double)top_p * (double)total);
    if (p_lim < 1) p_lim = 1;
    if (p_lim > total) p_lim = total;
    if (top_p >= 1.0f) p_lim = NO_MASS_LIMIT;      // see above: only top_k cuts
    const int mine = s_ccnt[wave];
    for (int pass = 0; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      for (int i = threadIdx.x; i < 256; i += SAMPLE_THREADS) {
        h_cnt[i] = 0;
        h_mass[i] = 0;
      }
      __syncthreads();
      const uint32_t prefix = st.prefix, mask = st.mask;
      for (int c = lane; c < mine; c += TA_WAVE) {
        const float l = cand_l[wave][c];
        const uint32_t key = order_key(l);
        if ((key & mask) == prefix) {
          const int bin = (key >> shift) & 255;
          atomicAdd(&h_cnt[bin], 1u);
          atomicAdd(&h_mass[bin], fixed_mass(l, m, inv_t));
        }
      }
      __syncthreads();
      if (threadIdx.x == 0) choose_digit(st, h_cnt, h_mass, shift, pass == 3, k_lim, p_lim);
      __syncthreads();
    }
    const uint32_t thr = st.prefix;
    const uint32_t n_tie = st.tie_count;
    // ---- the draw, in index order: wave by wave, and inside a wave as gathered
    uint32_t ties = 0;
    for (int c0 = 0; c0 < mine; c0 += TA_WAVE) {
      const int c = c0 + lane;
      ties += __popcll(__ballot(c < mine && order_key(cand_l[wave][c]) == thr));
    }
    if (lane == 0) s_c[wave] = ties;
    __syncthreads();
    uint32_t tie_base = 0;
    for (int w = 0; w < wave; ++w) tie_base += s_c[w];
    u64 kept = 0;
    {
      uint32_t rank = tie_base;
      for (int c0 = 0; c0 < mine; c0 += TA_WAVE) {
        const int c = c0 + lane;
        bool keep = false, tie = false;
        float l = 0.f;
        if (c < mine) {
          l = cand_l[wave][c];
          const uint32_t key = order_key(l);
          tie = key == thr;
          keep = key > thr;
        }
        const u64 b = __ballot(tie);
        if (tie && rank + __popcll(b & lanes_below) < n_tie) keep = true;
        rank += __popcll(b);
        if (keep) kept += fixed_mass(l, m, inv_t);
      }
    }
    kept = wave_sum_u64(kept);
    if (lane == 0) s_q[wave] = kept;
    __syncthreads();
    u64 mass_base = 0, kept_total = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) {
      if (w < wave) mass_base += s_q[w];
      kept_total += s_q[w];
    }
    u64 target = (u64)((double)uniform[blockIdx.x] * (double)kept_total);
    if (kept_total > 0 && target >= kept_total) target = kept_total - 1;
    if (kept_total > 0 && target >= mass_base && target < mass_base + s_q[wave]) {
      uint32_t rank = tie_base;
      u64 run = mass_base;
      for (int c0 = 0; c0 < mine; c0 += TA_WAVE) {
        const int c = c0 + lane;
        bool keep = false, tie = false;
        float l = 0.f;
        if (c < mine) {
          l = cand_l[wave][c];
          const uint32_t key = order_key(l);
          tie = key == thr;
          keep = key > thr;
        }
        const u64 b = __ballot(tie);
        if (tie && rank + __popcll(b & lanes_below) < n_tie) keep = true;
        rank += __popcll(b);
        const u64 q = keep ? fixed_mass(l, m, inv_t) : 0;
        u64 inc = q;
#pragma unroll
        for (int o = 1; o < TA_WAVE; o <<= 1) {
          const u64 up = shfl_up_u64(inc, o);
          if (lane >= o) inc += up;
        }
        const bool hit = q > 0 && run + inc > target && run + inc - q <= target;
        if (__ballot(hit)) {
          if (hit) s_pick = cand_i[wave][c];
          break;
        }
        uint32_t lo32 = (uint32_t)inc, hi32 = (uint32_t)(inc >> 32);
        lo32 = __shfl(lo32, TA_WAVE - 1, TA_WAVE);
        hi32 = __shfl(hi32, TA_WAVE - 1, TA_WAVE);
        run += ((u64)hi32 << 32) | lo32;
      }
    }
    __syncthreads();
    if (threadIdx.x == 0) out[blockIdx.x] = s_pick;
    return;
  }

  // ---- threshold of the kept set (only when top-k or top-p cut anything)
  if (cut) {
    const uint32_t k_lim = (uint32_t)(top_k < vocab ? top_k : vocab);
    u64 p_lim = (u64)ceil((double)top_p * (double)total);
    if (p_lim < 1) p_lim = 1;
    if (p_lim > total) p_lim = total;
    if (top_p >= 1.0f) p_lim = NO_MASS_LIMIT;      // see above: only top_k cuts
    for (int pass = 0; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      for (int i = threadIdx.x; i < 256; i += SAMPLE_THREADS) {
        h_cnt[i] = 0;
        h_mass[i] = 0;
      }
      __syncthreads();
      const uint32_t prefix = st.prefix, mask = st.mask;
      for (int j = threadIdx.x; j < groups; j += SAMPLE_THREADS) {
        const Four f = load_four(row, j, vocab);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t key = order_key(f.v[e]);
          if (f.ok[e] && (key & mask) == prefix) {
            const int bin = (key >> shift) & 255;
            atomicAdd(&h_cnt[bin], 1u);
            atomicAdd(&h_mass[bin], fixed_mass(f.v[e], m, inv_t));
          }
        }
      }
      __syncthreads();
      if (threadIdx.x == 0) choose_digit(st, h_cnt, h_mass, shift, pass == 3, k_lim, p_lim);
      __syncthreads();
    }
  }
  const uint32_t thr = st.prefix;          // 0 when nothing is cut: every key is > 0
  const uint32_t n_tie = st.tie_count;

  // ---- ordered sweeps: wave w owns the contiguous groups [lo, hi); inside a step of 64
  // groups the order of the indices is lane by lane, and inside a lane element by element

  // which of a lane's four tokens are kept, given the ties counted before this step
#define KEEP_FOUR(f_, rank_, keep_, q_)                                                   \
  do {                                                                                    \
    bool tie_[4];                                                                         \
    uint32_t before_ = 0, all_ = 0;                                                       \
    _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                       \
      const uint32_t key_ = order_key(f_.v[e]);                                           \
      tie_[e] = cut && f_.ok[e] && key_ == thr;                                           \
      keep_[e] = f_.ok[e] && (!cut || key_ > thr);                                        \
      const u64 b_ = __ballot(tie_[e]);                                                   \
      before_ += __popcll(b_ & lanes_below);                                              \
      all_ += __popcll(b_);                                                               \
    }                                                                                     \
    uint32_t mine_ = rank_ + before_;            /* ties in the lanes before this one */  \
    _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                       \
      if (tie_[e]) {                                                                      \
        if (mine_ < n_tie) keep_[e] = true;                                               \
        ++mine_;                                                                          \
      }                                                                                   \
      q_[e] = keep_[e] ? fixed_mass(f_.v[e], m, inv_t) : 0;                               \
    }                                                                                     \
    rank_ += all_;                                                                        \
  } while (0)

  // sweep 1: threshold-valued tokens per wave -> rank base of each wave
  uint32_t ties = 0;
  if (cut)
    for (int j0 = lo; j0 < hi; j0 += TA_WAVE) {
      const int j = j0 + lane;
      Four f;
      if (j < hi) f = load_four(row, j, vocab);
#pragma unroll
      for (int e = 0; e < 4; ++e) ties += __popcll(__ballot(j < hi && f.ok[e] && order_key(f.v[e]) == thr));
    }
  if (lane == 0) s_c[wave] = ties;
  __syncthreads();
  uint32_t tie_base = 0;
  for (int w = 0; w < wave; ++w) tie_base += s_c[w];
  __syncthreads();

  // sweep 2: kept mass per wave -> mass base of each wave
  u64 kept = 0;
  {
    uint32_t rank = tie_base;
    for (int j0 = lo; j0 < hi; j0 += TA_WAVE) {
      const int j = j0 + lane;
      Four f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        f.v[e] = -INFINITY;
        f.ok[e] = false;
      }
      if (j < hi) f = load_four(row, j, vocab);
      bool keep[4];
      u64 q[4];
      if (cut) {
        KEEP_FOUR(f, rank, keep, q);
      } else {                                   // temperature alone: every token is kept
#pragma unroll
        for (int e = 0; e < 4; ++e) q[e] = f.ok[e] ? fixed_mass(f.v[e], m, inv_t) : 0;
      }
      const u64 here = wave_sum_u64(q[0] + q[1] + q[2] + q[3]);
      const int step = (j0 - lo) / TA_WAVE;
      if (lane == 0 && step < VEC_STEPS) s_step[wave][step] = here;
      kept += here;
    }
  }
  if (lane == 0) s_q[wave] = kept;
  __syncthreads();
  u64 mass_base = 0, kept_total = 0;
  for (int w = 0; w < SAMPLE_WAVES; ++w) {
    if (w < wave) mass_base += s_q[w];
    kept_total += s_q[w];
  }
  u64 target = (u64)((double)uniform[blockIdx.x] * (double)kept_total);
  if (kept_total > 0 && target >= kept_total) target = kept_total - 1;

  // sweep 3: the wave whose range holds the target finds the token
  if (kept_total > 0 && target >= mass_base && target < mass_base + s_q[wave]) {
    uint32_t rank = tie_base;
    u64 run = mass_base;
    for (int j0 = lo; j0 < hi; j0 += TA_WAVE) {
      const int j = j0 + lane;
      Four f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        f.v[e] = -INFINITY;
        f.ok[e] = false;
      }
      if (j < hi) f = load_four(row, j, vocab);
      const int step = (j0 - lo) / TA_WAVE;
      if (step < VEC_STEPS && run + s_step[wave][step] <= target) {
        // the target lies behind this step: only its ties have to be counted
        run += s_step[wave][step];
        if (cut) {
#pragma unroll
          for (int e = 0; e < 4; ++e) rank += __popcll(__ballot(f.ok[e] && order_key(f.v[e]) == thr));
        }
        continue;
      }
      bool keep[4];
      u64 q[4];
      if (cut) {
        KEEP_FOUR(f, rank, keep, q);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) q[e] = f.ok[e] ? fixed_mass(f.v[e], m, inv_t) : 0;
      }
      const u64 mine = q[0] + q[1] + q[2] + q[3];
      u64 inc = mine;                                // inclusive scan over the wave
#pragma unroll
      for (int o = 1; o < TA_WAVE; o <<= 1) {
        const u64 up = shfl_up_u64(inc, o);
        if (lane >= o) inc += up;
      }
      const bool hit = mine > 0 && run + inc > target && run + inc - mine <= target;
      if (__ballot(hit)) {
        if (hit) {
          u64 at = run + inc - mine;                 // mass before this lane's four tokens
          int pick = 4 * j;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (q[e] > 0 && at + q[e] > target && at <= target) pick = 4 * j + e;
            at += q[e];
          }
          s_pick = pick;
        }
        break;
      }
      {  // the last lane holds the sum of this step
        uint32_t lo32 = (uint32_t)inc, hi32 = (uint32_t)(inc >> 32);
        lo32 = __shfl(lo32, TA_WAVE - 1, TA_WAVE);
        hi32 = __shfl(hi32, TA_WAVE - 1, TA_WAVE);
        run += ((u64)hi32 << 32) | lo32;
      }
    }
  }
#undef KEEP_FOUR
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = s_pick;
}

extern "C" int ta_sample(hipStream_t stream, const float* logits, long long ld, int n, int vocab,
                         float temperature, int top_k, float top_p, const float* uniform,
                         int* out) {
  TA_REQUIRE(n >= 0 && vocab > 0 && ld >= vocab, "ta_sample: bad sizes n=%d vocab=%d ld=%lld", n, vocab, ld);
  TA_REQUIRE(temperature > 0.f, "ta_sample: temperature %g must be > 0 (0 means argmax)", (double)temperature);
  TA_REQUIRE(top_k >= 1, "ta_sample: top_k %d < 1", top_k);
  TA_REQUIRE(top_p >= 0.f && top_p <= 1.f, "ta_sample: top_p %g outside [0, 1]", (double)top_p);
  if (n == 0) return 0;
  if (((uintptr_t)logits % 16) == 0 && ld % 4 == 0)
    sample_vec_kernel<<<n, SAMPLE_THREADS, 0, stream>>>(logits, (size_t)ld, vocab, 1.0f / temperature,
                                                        top_k, top_p, uniform, out);
  else
    sample_kernel<<<n, SAMPLE_THREADS, 0, stream>>>(logits, (size_t)ld, vocab, 1.0f / temperature,
                                                    top_k, top_p, uniform, out);
  return ta_check_launch("ta_sample");
}
