// Memory-bound parts of the step: embedding rows, residual-add + RMS norm,
// rotary position encoding fused with the cache write, SwiGLU.
//
// The residual stream is float32 in both engine dtypes; every sum of squares,
// rotation angle and activation is computed in float32.
#include "common.h"

// ------------------------------------------------------------------ errors
static thread_local char g_err[512] = "";

int ta_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return 1;
}

int ta_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return ta_fail("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

extern "C" const char* ta_last_error() { return g_err; }
extern "C" int ta_page_size() { return TA_PAGE; }

// ------------------------------------------------------------------ embedding
// x[t, :] = table[token[t], :] widened to float32 (no scaling). Token ids that the host has
// checked never fall outside the table; ids that were chosen on the GPU reach this kernel
// unseen, so an id outside [0, vocab) reads nothing and its row becomes NaN, which every
// logit of that sequence then shows.
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ tokens,
                             float* __restrict__ x, int d, int vocab) {
  const int t = blockIdx.x;
  const int id = tokens[t];
  float* out = x + (size_t)t * d;
  if (id < 0 || id >= vocab) {
    for (int i = threadIdx.x; i < d; i += blockDim.x) out[i] = __builtin_nanf("");
    return;
  }
  const T* row = table + (size_t)id * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) out[i] = to_f32(row[i]);
}

// The same for bfloat16 rows of a multiple of 8 elements: sixteen bytes per load, so that a
// row of 4,096 is two loads per thread on their way together and not sixteen (a step of 8
// tokens: 10.6 -> 5 us, all of it the two trips to memory behind the launch).
__global__ void embed_bf16x8_kernel(const bf16_t* __restrict__ table, const int* __restrict__ tokens,
                                    float* __restrict__ x, int d, int vocab) {
  const int t = blockIdx.x;
  const int id = tokens[t];
  float* out = x + (size_t)t * d;
  const bool ok = id >= 0 && id < vocab;
  const bf16_t* row = table + (size_t)(ok ? id : 0) * d;
  for (int i = threadIdx.x * 8; i < d; i += blockDim.x * 8) {
    const uint4 v = *reinterpret_cast<const uint4*>(row + i);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    float f[8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      f[2 * k] = ok ? __uint_as_float(w[k] << 16) : __builtin_nanf("");
      f[2 * k + 1] = ok ? __uint_as_float(w[k] & 0xffff0000u) : __builtin_nanf("");
    }
    *reinterpret_cast<float4*>(out + i) = make_float4(f[0], f[1], f[2], f[3]);
    *reinterpret_cast<float4*>(out + i + 4) = make_float4(f[4], f[5], f[6], f[7]);
  }
}

extern "C" int ta_embed(hipStream_t stream, int dtype, const void* table, int vocab, int d,
                        const int* tokens, int nt, float* x) {
  TA_REQUIRE(dtype == TA_F32 || dtype == TA_BF16, "ta_embed: unknown dtype %d", dtype);
  TA_REQUIRE(vocab > 0 && d > 0 && nt >= 0, "ta_embed: bad sizes vocab=%d d=%d nt=%d", vocab, d, nt);
  if (nt == 0) return 0;
  if (dtype == TA_F32)
    embed_kernel<float><<<nt, 256, 0, stream>>>((const float*)table, tokens, x, d, vocab);
  else if (d % 8 == 0 && ((uintptr_t)table % 16) == 0 && ((uintptr_t)x % 16) == 0)
    embed_bf16x8_kernel<<<nt, 256, 0, stream>>>((const bf16_t*)table, tokens, x, d, vocab);
  else
    embed_kernel<bf16_t><<<nt, 256, 0, stream>>>((const bf16_t*)table, tokens, x, d, vocab);
  return ta_check_launch("ta_embed");
}

// ------------------------------------------------------------------ add + RMS norm
// For output row i (source row r = rows ? rows[i] : i):
//   v = x[r] + delta[r] + delta_bias        (terms that are null are left out)
//   if store_x: x[r] = v
//   out[i] = v / sqrt(mean(v^2) + eps) * w
// One workgroup per row; the reduction order depends on d and the block size only,
// and the block size is chosen from d, so a row gives the same bits in any batch.
template <typename T> struct Vec4;
template <> struct Vec4<float> {
  float4 v;
  __device__ __forceinline__ void load(const float* p) { v = *reinterpret_cast<const float4*>(p); }
  __device__ __forceinline__ void store(float* p) const { *reinterpret_cast<float4*>(p) = v; }
  __device__ __forceinline__ float get(int i) const { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
  __device__ __forceinline__ void set(float a, float b, float c, float d) { v = make_float4(a, b, c, d); }
};
template <> struct Vec4<bf16_t> {
  uint2 v;
  __device__ __forceinline__ void load(const bf16_t* p) { v = *reinterpret_cast<const uint2*>(p); }
  __device__ __forceinline__ void store(bf16_t* p) const { *reinterpret_cast<uint2*>(p) = v; }
  __device__ __forceinline__ float get(int i) const {
    const uint32_t w = i < 2 ? v.x : v.y;
    return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
  }
  __device__ __forceinline__ void set(float a, float b, float c, float d) {
    v.x = (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(b) << 16);
    v.y = (uint32_t)f32_to_bf16_bits(c) | ((uint32_t)f32_to_bf16_bits(d) << 16);
  }
};

__device__ __forceinline__ float block_sum(float v, float* part, int nwaves) {
  v = wave_sum(v);
  const int wave = threadIdx.x / TA_WAVE, lane = threadIdx.x % TA_WAVE;
  if (lane == 0) part[wave] = v;
  __syncthreads();
  float tot = 0.f;
  for (int i = 0; i < nwaves; ++i) tot += part[i];     // same order in every thread
  return tot;
}

// d % 4 == 0 and d <= 4 * U * blockDim.x: a thread keeps its 4 * U values in registers, so
// every load of the row is in flight at once and the row is read a single time. U = 4 for
// steps of many rows; the few rows of a single-token step take U = 1 and four times the
// threads (a row's chain of load, sum, barrier and store is what such a launch waits for,
// and it is shorter with one vector per thread). MAXPL: planes of a delta that a thread asks
// for (a plane that is not there reads plane 0 again and is not added).
template <typename TD, typename TO, int U, int MAXPL>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ x, const TD* __restrict__ delta,
                                       const float* __restrict__ delta_bias,
                                       const float* __restrict__ w, const int* __restrict__ rows,
                                       TO* __restrict__ out, int d, float eps, int store_x,
                                       int planes, size_t plane) {
  __shared__ float part[16];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* xr = x + (size_t)r * d;
  const TD* dr = delta ? delta + (size_t)r * d : nullptr;
  const int nv = d / 4;
  float v[U][4];
  Vec4<float> xv[U];
  Vec4<TD> dv[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int c = threadIdx.x + u * blockDim.x;
    if (c < nv) {
      xv[u].load(xr + 4 * c);
      if (dr) dv[u].load(dr + 4 * c);
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int c = threadIdx.x + u * blockDim.x;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float t = 0.f;
      if (c < nv) {
        t = xv[u].get(e);
        if (dr) t += dv[u].get(e);
      }
      v[u][e] = t;
    }
    // further planes of a delta that came in parts, added in order; all are asked for
    // before the first is added
    if (MAXPL > 1 && dr && c < nv && planes > 1) {
      Vec4<TD> more[MAXPL > 1 ? MAXPL - 1 : 1];
#pragma unroll
      for (int pl = 1; pl < MAXPL; ++pl) more[pl - 1].load(dr + (pl < planes ? (size_t)pl * plane : 0) + 4 * c);
#pragma unroll
      for (int pl = 1; pl < MAXPL; ++pl)
#pragma unroll
        for (int e = 0; e < 4; ++e) v[u][e] += pl < planes ? more[pl - 1].get(e) : 0.f;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (c < nv && delta_bias) v[u][e] += delta_bias[4 * c + e];
      ss += v[u][e] * v[u][e];
    }
  }
  const float tot = block_sum(ss, part, blockDim.x / TA_WAVE);
  const float rstd = 1.0f / sqrtf(tot / (float)d + eps);
  TO* orow = out + (size_t)i * d;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int c = threadIdx.x + u * blockDim.x;
    if (c < nv) {
      if (store_x) {
        Vec4<float> sv;
        sv.set(v[u][0], v[u][1], v[u][2], v[u][3]);
        sv.store(xr + 4 * c);
      }
      Vec4<float> wv;
      wv.load(w + 4 * c);
      Vec4<TO> ov;
      ov.set(v[u][0] * rstd * wv.get(0), v[u][1] * rstd * wv.get(1), v[u][2] * rstd * wv.get(2),
             v[u][3] * rstd * wv.get(3));
      ov.store(orow + 4 * c);
    }
  }
}

template <typename TD, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const TD* __restrict__ delta,
                                   const float* __restrict__ delta_bias,
                                   const float* __restrict__ w, const int* __restrict__ rows,
                                   TO* __restrict__ out, int d, float eps, int store_x,
                                   int planes, size_t plane) {
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* xr = x + (size_t)r * d;
  const TD* dr = delta ? delta + (size_t)r * d : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    float v = xr[c];
    if (dr)
      for (int pl = 0; pl < planes; ++pl) v += to_f32(dr[(size_t)pl * plane + c]);
    if (delta_bias) v += delta_bias[c];
    ss += v * v;
  }
  __shared__ float part[16];
  const float tot = block_sum(ss, part, blockDim.x / TA_WAVE);
  const float rstd = 1.0f / sqrtf(tot / (float)d + eps);
  TO* orow = out + (size_t)i * d;
  for (int c = threadIdx.x; c < d; c += blockDim.x) {
    float v = xr[c];
    if (dr)
      for (int pl = 0; pl < planes; ++pl) v += to_f32(dr[(size_t)pl * plane + c]);
    if (delta_bias) v += delta_bias[c];
    // the element is read again before it is overwritten, by this same thread only
    if (store_x) xr[c] = v;
    orow[c] = from_f32<TO>(v * rstd * w[c]);
  }
}

extern "C" int ta_add_rmsnorm(hipStream_t stream, int delta_dtype, int out_dtype, float* x,
                              const void* delta, const float* delta_bias, const float* w,
                              const int* rows, void* out, int n_out, int d, float eps,
                              int store_x, int planes, long long plane) {
  // planes > 1: delta came in parts, `plane` elements apart, that are added in order
  TA_REQUIRE(d > 0 && n_out >= 0, "ta_add_rmsnorm: bad sizes n_out=%d d=%d", n_out, d);
  TA_REQUIRE(planes >= 1 && planes <= TA_MAX_PLANES && (planes == 1 || (delta && plane > 0)),
             "ta_add_rmsnorm: %d planes of a delta (at most %d)", planes, TA_MAX_PLANES);
  TA_REQUIRE(eps >= 0.f, "ta_add_rmsnorm: eps %g < 0", (double)eps);
  TA_REQUIRE(!(rows && store_x), "ta_add_rmsnorm: store_x with gathered rows is not defined");
  if (n_out == 0) return 0;
  const bool aligned = ((uintptr_t)x % 16 == 0) && ((uintptr_t)delta % 16 == 0) &&
                       ((uintptr_t)w % 16 == 0) && ((uintptr_t)out % 16 == 0) && plane % 4 == 0;
  const bool vec = d % 4 == 0 && d <= 16384 && aligned;
  // few rows (a single-token step): one vector per thread while a workgroup can hold the row.
  // Only where the output is bfloat16: the order of a row's sum of squares follows the number
  // of threads, and the float32 engine keeps a row's bits whatever the step it comes in
  const bool few = vec && n_out <= 64 && d <= 4096 && out_dtype == TA_BF16;
  int threads = 256;
  if (vec) {
    threads = 64;
    while (threads * (few ? 4 : 16) < d) threads *= 2;       // 64 .. 1024, a function of d (and of few)
  }
  dim3 g(n_out), b(threads);
#define LAUNCH_V(TD, TO, U, MAXPL)                                                                \
  add_rmsnorm_vec_kernel<TD, TO, U, MAXPL><<<g, b, 0, stream>>>(x, (const TD*)delta, delta_bias, w, rows, \
                                                                (TO*)out, d, eps, store_x, planes, (size_t)plane)
#define LAUNCH(TD, TO)                                                                            \
  do {                                                                                            \
    if (vec && few) {                                                                             \
      if (planes <= 1) LAUNCH_V(TD, TO, 1, 1);                                                    \
      else if (planes <= 4) LAUNCH_V(TD, TO, 1, 4);                                               \
      else LAUNCH_V(TD, TO, 1, TA_MAX_PLANES);                                                    \
    } else if (vec) {                                                                             \
      if (planes <= 1) LAUNCH_V(TD, TO, 4, 1); else LAUNCH_V(TD, TO, 4, TA_MAX_PLANES);           \
    } else                                                                                        \
      add_rmsnorm_kernel<TD, TO><<<g, b, 0, stream>>>(x, (const TD*)delta, delta_bias, w, rows,   \
                                                      (TO*)out, d, eps, store_x, planes,          \
                                                      (size_t)plane);                             \
  } while (0)
  if (delta_dtype == TA_F32 && out_dtype == TA_F32) LAUNCH(float, float);
  else if (delta_dtype == TA_F32 && out_dtype == TA_BF16) LAUNCH(float, bf16_t);
  else if (delta_dtype == TA_BF16 && out_dtype == TA_BF16) LAUNCH(bf16_t, bf16_t);
  else if (delta_dtype == TA_BF16 && out_dtype == TA_F32) LAUNCH(bf16_t, float);
  else return ta_fail("ta_add_rmsnorm: unknown dtypes %d %d", delta_dtype, out_dtype);
#undef LAUNCH
#undef LAUNCH_V
  return ta_check_launch("ta_add_rmsnorm");
}

// ------------------------------------------------------------------ rotary + cache write
// Angles of a step: cs[t][j] = (cos a, sin a), a = (float)pos[t] * inv_freq[j] formed
// in float32. Every layer with the same frequencies shares the table of the step.
__global__ void rope_table_kernel(const int* __restrict__ pos, const float* __restrict__ inv_freq,
                                  float2* __restrict__ cs, int half) {
  const int t = blockIdx.x;
  const float p = (float)pos[t];
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    float sn, c;
    sincosf(p * inv_freq[j], &sn, &c);
    cs[(size_t)t * half + j] = make_float2(c, sn);
  }
}

extern "C" int ta_rope_table(hipStream_t stream, const int* pos, const float* inv_freq, float* cs,
                             int nt, int half) {
  TA_REQUIRE(nt >= 0 && half > 0, "ta_rope_table: bad sizes nt=%d half=%d", nt, half);
  if (nt == 0) return 0;
  rope_table_kernel<<<nt, 64, 0, stream>>>(pos, inv_freq, (float2*)cs, half);
  return ta_check_launch("ta_rope_table");
}

// qkv: [nt, nq + 2*nkv, dh]. Per token t:
//   q heads: (+bias) rotated in place
//   k heads: (+bias) rotated, written to the K cache at dest[t] (and back in place)
//   v heads: (+bias) copied to the V cache at dest[t]
// dest[t] = page * TA_PAGE + offset inside the page. A key page is laid out
// [page][kv head][TA_PAGE][dh]; a value page is transposed, [page][kv head][dh][TA_PAGE],
// so that the matrix cores read 8-byte runs of consecutive keys for one output column.
// dest[t] < 0 or kcache == null: nothing is cached.
// cs == null: no rotation. style 0: pairs (j, j+dh/2); 1: pairs (2j, 2j+1).
template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, const float* __restrict__ bias,
                                     const int* __restrict__ dest, const float2* __restrict__ cs,
                                     int style, T* __restrict__ kcache, T* __restrict__ vcache,
                                     int nq, int nkv, int dh) {
  const int t = blockIdx.x;
  const int h = blockIdx.y;
  T* v = qkv + ((size_t)t * (nq + 2 * nkv) + h) * dh;
  const float* b = bias ? bias + (size_t)h * dh : nullptr;
  const int half = dh / 2;
  const int slot = dest ? dest[t] : -1;
  const bool cache = kcache != nullptr && slot >= 0;
  const size_t page = cache ? (size_t)(slot / TA_PAGE) : 0;
  const int off = cache ? slot % TA_PAGE : 0;
  if (h < nq + nkv) {
    T* kc = nullptr;
    if (h >= nq && cache) kc = kcache + ((page * nkv + (h - nq)) * TA_PAGE + off) * dh;
    const float2* ct = cs ? cs + (size_t)t * half : nullptr;
    for (int j = threadIdx.x; j < half; j += blockDim.x) {
      const int i0 = style == 0 ? j : 2 * j;
      const int i1 = style == 0 ? j + half : 2 * j + 1;
      float a = to_f32(v[i0]), c = to_f32(v[i1]);
      if (b) {
        a += b[i0];
        c += b[i1];
      }
      float r0 = a, r1 = c;
      if (ct) {
        const float2 k = ct[j];
        r0 = a * k.x - c * k.y;
        r1 = a * k.y + c * k.x;
      }
      const T o0 = from_f32<T>(r0), o1 = from_f32<T>(r1);
      v[i0] = o0;
      v[i1] = o1;
      if (kc) {
        kc[i0] = o0;
        kc[i1] = o1;
      }
    }
  } else {
    T* vc = cache ? vcache + (page * nkv + (h - nq - nkv)) * (size_t)dh * TA_PAGE + off : nullptr;
    if (!b && !vc) return;
    for (int i = threadIdx.x; i < dh; i += blockDim.x) {
      T o = v[i];
      if (b) {
        o = from_f32<T>(to_f32(o) + b[i]);
        v[i] = o;
      }
      if (vc) vc[(size_t)i * TA_PAGE] = o;
    }
  }
}

// The same for prompts, four tokens per workgroup, four elements per access. Needs dh % 8
// == 0 and rows that start on 16-byte boundaries. q and k: an item is two runs of four
// elements whose pairs lie inside it (style 0: elements j..j+3 and their partners dh/2
// further on; style 1: eight consecutive elements). v: a thread takes one head dimension of
// one kv head for the four tokens, and when the four land side by side in a page (the usual
// case inside a prompt) it stores them with one access instead of four 128 bytes apart.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_vec_kernel(
    T* __restrict__ qkv, const float* __restrict__ bias, const int* __restrict__ dest,
    const float2* __restrict__ cs, int style, T* __restrict__ kcache, T* __restrict__ vcache,
    int nt, int nq, int nkv, int dh) {
  const int t0 = blockIdx.x * 4;
  const int ntok = nt - t0 < 4 ? nt - t0 : 4;
  const int half = dh / 2, per_head = dh / 8;
  const size_t width = (size_t)(nq + 2 * nkv) * dh;
  const bool cache = kcache != nullptr && dest != nullptr;
  int slot[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) slot[i] = (cache && i < ntok) ? dest[t0 + i] : -1;

  // ---- q and k heads
  // blockIdx.y: the items of a group of four tokens are dealt out to several workgroups, so
  // that a prompt of a few thousand tokens still fills the CUs
  const int stride = 256 * gridDim.y, lane0 = threadIdx.x + 256 * blockIdx.y;
  const int items = ntok * (nq + nkv) * per_head;
  for (int it = lane0; it < items; it += stride) {
    const int u = it % per_head;
    const int h = (it / per_head) % (nq + nkv);
    const int ti = it / (per_head * (nq + nkv));
    const int t = t0 + ti;
    const int o0 = style == 0 ? 4 * u : 8 * u;
    const int o1 = style == 0 ? 4 * u + half : 8 * u + 4;
    T* v = qkv + (size_t)t * width + (size_t)h * dh;
    Vec4<T> x0, x1;
    x0.load(v + o0);
    x1.load(v + o1);
    float a[4], c[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      a[e] = x0.get(e);
      c[e] = x1.get(e);
      if (bias) {
        a[e] += bias[(size_t)h * dh + o0 + e];
        c[e] += bias[(size_t)h * dh + o1 + e];
      }
    }
    if (cs) {
      const float2* ct = cs + (size_t)t * half;
      if (style == 0) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float2 k = ct[4 * u + e];
          const float r0 = a[e] * k.x - c[e] * k.y, r1 = a[e] * k.y + c[e] * k.x;
          a[e] = r0;
          c[e] = r1;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
          const float2 ka = ct[4 * u + e / 2], kc2 = ct[4 * u + 2 + e / 2];
          const float a0 = a[e] * ka.x - a[e + 1] * ka.y, a1 = a[e] * ka.y + a[e + 1] * ka.x;
          const float c0 = c[e] * kc2.x - c[e + 1] * kc2.y, c1 = c[e] * kc2.y + c[e + 1] * kc2.x;
          a[e] = a0;
          a[e + 1] = a1;
          c[e] = c0;
          c[e + 1] = c1;
        }
      }
    }
    x0.set(a[0], a[1], a[2], a[3]);
    x1.set(c[0], c[1], c[2], c[3]);
    x0.store(v + o0);
    x1.store(v + o1);
    const int sl = ti == 0 ? slot[0] : ti == 1 ? slot[1] : ti == 2 ? slot[2] : slot[3];
    if (h >= nq && sl >= 0) {
      T* kc = kcache + (((size_t)(sl / TA_PAGE) * nkv + (h - nq)) * TA_PAGE + sl % TA_PAGE) * dh;
      x0.store(kc + o0);
      x1.store(kc + o1);
    }
  }

  // ---- v heads
  const bool together = ntok == 4 && slot[0] >= 0 && slot[0] % 4 == 0 && slot[1] == slot[0] + 1 &&
                        slot[2] == slot[0] + 2 && slot[3] == slot[0] + 3;
  const float* vb = bias ? bias + (size_t)(nq + nkv) * dh : nullptr;
  if (!vb && !cache) return;
  for (int it = lane0; it < nkv * dh; it += stride) {
    const int d = it % dh, g = it / dh;
    float val[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      val[i] = 0.f;
      if (i < ntok) {
        T* p = qkv + (size_t)(t0 + i) * width + (size_t)(nq + nkv + g) * dh + d;
        val[i] = to_f32(*p);
        if (vb) {
          val[i] = to_f32(from_f32<T>(val[i] + vb[it]));
          *p = from_f32<T>(val[i]);
        }
      }
    }
    if (together) {
      Vec4<T> o;
      o.set(val[0], val[1], val[2], val[3]);
      o.store(vcache + ((size_t)(slot[0] / TA_PAGE) * nkv + g) * (size_t)dh * TA_PAGE +
              (size_t)d * TA_PAGE + slot[0] % TA_PAGE);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (slot[i] >= 0)
          vcache[((size_t)(slot[i] / TA_PAGE) * nkv + g) * (size_t)dh * TA_PAGE + (size_t)d * TA_PAGE +
                 slot[i] % TA_PAGE] = from_f32<T>(val[i]);
    }
  }
}

extern "C" int ta_rope_kv_write(hipStream_t stream, int dtype, void* qkv, const float* bias,
                                const int* dest, const float* cs, int style, void* kcache,
                                void* vcache, int nt, int nq, int nkv, int dh) {
  TA_REQUIRE(nq > 0 && nkv >= 0 && nt >= 0, "ta_rope_kv_write: bad sizes nt=%d nq=%d nkv=%d", nt, nq, nkv);
  TA_REQUIRE(dh > 0 && dh % 2 == 0, "ta_rope_kv_write: head size %d must be even", dh);
  TA_REQUIRE(style == 0 || style == 1, "ta_rope_kv_write: unknown pairing style %d", style);
  TA_REQUIRE((kcache == nullptr) == (vcache == nullptr), "ta_rope_kv_write: K and V cache must come together");
  if (nt == 0) return 0;
  const bool aligned = ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)kcache % 16) == 0 && ((uintptr_t)vcache % 16) == 0;
  if (nt >= 8 && dh % 8 == 0 && aligned && (dtype == TA_F32 || dtype == TA_BF16)) {
    const int groups = (nt + 3) / 4;
    int parts = 1;
    while (parts < 8 && groups * parts < 2048) parts *= 2;
    dim3 gv(groups, parts), bv(256);
    if (dtype == TA_F32)
      rope_kv_write_vec_kernel<float><<<gv, bv, 0, stream>>>((float*)qkv, bias, dest, (const float2*)cs, style,
                                                             (float*)kcache, (float*)vcache, nt, nq, nkv, dh);
    else
      rope_kv_write_vec_kernel<bf16_t><<<gv, bv, 0, stream>>>((bf16_t*)qkv, bias, dest, (const float2*)cs, style,
                                                              (bf16_t*)kcache, (bf16_t*)vcache, nt, nq, nkv, dh);
    return ta_check_launch("ta_rope_kv_write");
  }
  dim3 g(nt, nq + 2 * nkv), b(dh / 2 < 64 ? 64 : (dh / 2 <= 128 ? dh / 2 : 128));
  if (dtype == TA_F32)
    rope_kv_write_kernel<float><<<g, b, 0, stream>>>((float*)qkv, bias, dest, (const float2*)cs, style,
                                                     (float*)kcache, (float*)vcache, nq, nkv, dh);
  else if (dtype == TA_BF16)
    rope_kv_write_kernel<bf16_t><<<g, b, 0, stream>>>((bf16_t*)qkv, bias, dest, (const float2*)cs, style,
                                                      (bf16_t*)kcache, (bf16_t*)vcache, nq, nkv, dh);
  else
    return ta_fail("ta_rope_kv_write: unknown dtype %d", dtype);
  return ta_check_launch("ta_rope_kv_write");
}

// ------------------------------------------------------------------ SwiGLU
// out[t, i] = silu(g) * u, g = gu[t, i] (+bias[i]), u = gu[t, di + i] (+bias[di + i]),
// silu(z) = z / (1 + exp(-z)), all in float32, rounded once. grid (chunks of a row, rows).
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, const float* __restrict__ bias,
                              T* __restrict__ out, int di) {
  const size_t t = blockIdx.y;
  const T* g = gu + t * 2 * (size_t)di;
  T* o = out + t * (size_t)di;
  const bool vec = di % 4 == 0 && ((uintptr_t)gu % 16 == 0) && ((uintptr_t)out % 16 == 0);
  if (vec) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (4 * c >= di) return;
    Vec4<T> gv, uv, ov;
    gv.load(g + 4 * c);
    uv.load(g + di + 4 * c);
    float r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float a = gv.get(e), u = uv.get(e);
      if (bias) {
        a += bias[4 * c + e];
        u += bias[di + 4 * c + e];
      }
      r[e] = a / (1.0f + expf(-a)) * u;
    }
    ov.set(r[0], r[1], r[2], r[3]);
    ov.store(o + 4 * c);
  } else {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < di; i += gridDim.x * blockDim.x) {
      float a = to_f32(g[i]), u = to_f32(g[di + i]);
      if (bias) {
        a += bias[i];
        u += bias[di + i];
      }
      o[i] = from_f32<T>(a / (1.0f + expf(-a)) * u);
    }
  }
}

extern "C" int ta_swiglu(hipStream_t stream, int dtype, const void* gate_up, const float* bias,
                         void* out, int nt, int di) {
  TA_REQUIRE(nt >= 0 && di > 0, "ta_swiglu: bad sizes nt=%d di=%d", nt, di);
  TA_REQUIRE(nt <= 65535 * 64, "ta_swiglu: too many rows for one launch");
  if (nt == 0) return 0;
  const int per_block = 256 * 4;
  for (int t0 = 0; t0 < nt; t0 += 65535) {
    const int rows = nt - t0 < 65535 ? nt - t0 : 65535;
    dim3 g((di + per_block - 1) / per_block, rows), b(256);
    const size_t in_off = (size_t)t0 * 2 * di, out_off = (size_t)t0 * di;
    if (dtype == TA_F32)
      swiglu_kernel<float><<<g, b, 0, stream>>>((const float*)gate_up + in_off, bias, (float*)out + out_off, di);
    else if (dtype == TA_BF16)
      swiglu_kernel<bf16_t><<<g, b, 0, stream>>>((const bf16_t*)gate_up + in_off, bias, (bf16_t*)out + out_off, di);
    else
      return ta_fail("ta_swiglu: unknown dtype %d", dtype);
  }
  return ta_check_launch("ta_swiglu");
}

// ------------------------------------------------------------------ random fill
// out[i] = mean + std * z_i with z_i standard normal from a counter-based generator:
// two 32-bit hashes of (seed, stream, i) feed one Box-Muller draw, so a tensor's
// values depend on (seed, stream) and the element index only.
__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

template <typename T>
__global__ void fill_normal_kernel(T* __restrict__ out, size_t n, uint64_t seed, uint64_t stream_id,
                                   float mean, float std) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const uint64_t key = mix64(seed * 0x9E3779B97F4A7C15ull + stream_id);
  for (; i < n; i += stride) {
    const uint64_t r = mix64(key + (uint64_t)i * 0xD1342543DE82EF95ull);
    const float u1 = ((float)(uint32_t)(r >> 40) + 1.0f) * (1.0f / 16777216.0f);   // (0, 1]
    const float u2 = (float)(uint32_t)((r >> 8) & 0xffffffu) * (1.0f / 16777216.0f);
    const float z = sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
    out[i] = from_f32<T>(mean + std * z);
  }
}

extern "C" int ta_fill_normal(hipStream_t stream, int dtype, void* out, long long n,
                              unsigned long long seed, unsigned long long stream_id, float mean,
                              float std) {
  TA_REQUIRE(n >= 0, "ta_fill_normal: negative size");
  if (n == 0) return 0;
  size_t blocks = ((size_t)n + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  if (dtype == TA_F32)
    fill_normal_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>((float*)out, (size_t)n, seed, stream_id, mean, std);
  else if (dtype == TA_BF16)
    fill_normal_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>((bf16_t*)out, (size_t)n, seed, stream_id, mean, std);
  else
    return ta_fail("ta_fill_normal: unknown dtype %d", dtype);
  return ta_check_launch("ta_fill_normal");
}

// ------------------------------------------------------------------ conversion at load
// dst[i] = src[i] in another floating type: what the loader runs on the device after the raw
// bytes of a file tensor have arrived, when the file stores another type than the engine
// keeps (float16 matrices of the reference's own files, bfloat16 norm weights that are
// kept in 32 bits). Every widening is exact; narrowing to bfloat16 rounds to nearest even.
// Source types: 0 float32, 1 bfloat16, 2 float16. Destination types: 0 float32, 1 bfloat16.
__device__ __forceinline__ float to_f32(_Float16 x) { return (float)x; }

template <typename S, typename D>
__global__ void convert_kernel(const S* __restrict__ src, D* __restrict__ dst, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = from_f32<D>(to_f32(src[i]));
}

template <typename S>
static int convert_to(hipStream_t stream, int dst_dtype, const void* src, void* dst, size_t n) {
  size_t blocks = (n + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  if (dst_dtype == TA_F32)
    convert_kernel<S, float><<<(unsigned)blocks, 256, 0, stream>>>((const S*)src, (float*)dst, n);
  else if (dst_dtype == TA_BF16)
    convert_kernel<S, bf16_t><<<(unsigned)blocks, 256, 0, stream>>>((const S*)src, (bf16_t*)dst, n);
  else
    return ta_fail("ta_convert: unknown destination dtype %d", dst_dtype);
  return ta_check_launch("ta_convert");
}

extern "C" int ta_convert(hipStream_t stream, int src_dtype, int dst_dtype, const void* src,
                          void* dst, long long n) {
  TA_REQUIRE(n >= 0, "ta_convert: negative size");
  if (n == 0) return 0;
  if (src_dtype == TA_F32) return convert_to<float>(stream, dst_dtype, src, dst, (size_t)n);
  if (src_dtype == TA_BF16) return convert_to<bf16_t>(stream, dst_dtype, src, dst, (size_t)n);
  if (src_dtype == 2) return convert_to<_Float16>(stream, dst_dtype, src, dst, (size_t)n);
  return ta_fail("ta_convert: unknown source dtype %d", src_dtype);
}

// ------------------------------------------------------------------ read probe
// What this machine's memory gives a kernel that only reads: every workgroup streams its
// share of the buffer with eight non-temporal 16-byte loads per thread in flight, the access
// pattern of the weight streams of a decode step without any of their work. The measurements
// state their own numbers against the published peak; this is the other yardstick.
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) read_probe_kernel(const probe_u32x4* __restrict__ src, size_t n16,
                                                         uint32_t* __restrict__ sink) {
  const size_t per = n16 / gridDim.x;               // 16-byte pieces per workgroup
  const probe_u32x4* mine = src + (size_t)blockIdx.x * per;
  probe_u32x4 acc = {0, 0, 0, 0};
  for (size_t i = threadIdx.x; i + 7 * 256 < per; i += 8 * 256) {
    probe_u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(&mine[i + u * 256]);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  // never true for a buffer of small numbers; keeps the loads alive
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[threadIdx.x] = acc.x;
}

// Reads `bytes` (a multiple of 16) at src with `workgroups` workgroups of 256 threads.
extern "C" int ta_read_probe(hipStream_t stream, const void* src, long long bytes, int workgroups, void* sink) {
  TA_REQUIRE(bytes > 0 && bytes % 16 == 0 && ((uintptr_t)src % 16) == 0, "ta_read_probe: %lld bytes at an unaligned place", bytes);
  TA_REQUIRE(workgroups > 0 && workgroups <= 65535 && sink != nullptr, "ta_read_probe: %d workgroups", workgroups);
  read_probe_kernel<<<workgroups, 256, 0, stream>>>((const probe_u32x4*)src, (size_t)bytes / 16, (uint32_t*)sink);
  return ta_check_launch("ta_read_probe");
}
