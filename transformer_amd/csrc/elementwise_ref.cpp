// Plain twins of elementwise.hip: embedding rows, residual add + RMS norm, rotation angles,
// rotation with the cache write, SiLU-and-multiply, the counter-based normal fill.
#include "ref_common.h"

#include <cmath>
#include <cstring>
#include <limits>
#include <vector>

static char g_error[512] = "";

int ta_ref_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

extern "C" const char* ta_ref_last_error() { return g_error; }
extern "C" int ta_ref_page_size() { return TA_REF_PAGE; }

// out[t, :] = table[tokens[t], :]; no scaling (test-utils/src/llama.rs:18-23 copies the
// rows as they are). An id outside the table gives a row of NaN, as the kernel does.
extern "C" int ta_ref_embed(const float* table, int vocab, int d, const int* tokens, int nt, float* out) {
  TA_REF_REQUIRE(vocab > 0 && d > 0 && nt >= 0, "ta_ref_embed: bad sizes");
  for (int t = 0; t < nt; ++t) {
    const int id = tokens[t];
    for (int i = 0; i < d; ++i)
      out[(size_t)t * d + i] = (id < 0 || id >= vocab) ? std::numeric_limits<float>::quiet_NaN()
                                                       : table[(size_t)id * d + i];
  }
  return 0;
}

// For output row i (source row r = rows ? rows[i] : i):
//   v = x[r] + delta[0][r] + ... + delta[planes-1][r] + delta_bias   (what is null is left out)
//   if store_x: x[r] = v
//   out[i] = v * rsqrt(mean(v^2) + eps) * w
// The norm itself: models/llama/common/src/compute.rs:206-207, :273-274, :358-359; the
// adds are the residual sums of :267-270 and :290-292 carried to the norm that follows.
extern "C" int ta_ref_add_rmsnorm(float* x, const float* delta, int planes, long long plane,
                                  const float* delta_bias, const float* w, const int* rows,
                                  int n_out, int d, float eps, int store_x, float* out) {
  TA_REF_REQUIRE(n_out >= 0 && d > 0 && planes >= 1, "ta_ref_add_rmsnorm: bad sizes");
  std::vector<double> v(d);
  for (int i = 0; i < n_out; ++i) {
    const size_t r = rows ? (size_t)rows[i] : (size_t)i;
    double sq = 0.0;
    for (int c = 0; c < d; ++c) {
      // the kernel adds in float32, in this order; the twin keeps the order and widens
      double s = x[r * d + c];
      if (delta)
        for (int p = 0; p < planes; ++p) s += delta[(size_t)p * plane + r * d + c];
      if (delta_bias) s += delta_bias[c];
      v[c] = s;
      sq += s * s;
    }
    const double f = 1.0 / std::sqrt(sq / d + (double)eps);
    for (int c = 0; c < d; ++c) {
      if (store_x) x[r * d + c] = (float)v[c];
      out[(size_t)i * d + c] = (float)(v[c] * f * w[c]);
    }
  }
  return 0;
}

// cs[t][j] = (cos a, sin a), a = float32(pos[t]) * inv_freq[j] formed in float32 (the angle
// is the kernel's; only its cosine and sine are taken in double here).
extern "C" int ta_ref_rope_table(const int* pos, const float* inv_freq, int nt, int half, float* cs) {
  TA_REF_REQUIRE(nt >= 0 && half > 0, "ta_ref_rope_table: bad sizes");
  for (int t = 0; t < nt; ++t)
    for (int j = 0; j < half; ++j) {
      const float a = (float)pos[t] * inv_freq[j];
      cs[((size_t)t * half + j) * 2 + 0] = (float)std::cos((double)a);
      cs[((size_t)t * half + j) * 2 + 1] = (float)std::sin((double)a);
    }
  return 0;
}

// qkv [nt][nq + 2 nkv][dh], per token: the bias is added to every head; q and k heads are
// rotated pair by pair, (u, v) -> (u cos - v sin, u sin + v cos) with the pair (j, j + dh/2)
// (style 0) or (2j, 2j + 1) (style 1) turning by angle j (compute.rs:232-233 rotates q and
// k before the cache is written); everything is written back to qkv, and k and v also go to
// the cache at dest[t] = page * 64 + offset (compute.rs:243-264 writes rows pos..pos+seq).
extern "C" int ta_ref_rope_kv_write(float* qkv, const float* bias, const int* dest, const float* cs,
                                    int style, float* kcache, float* vcache, int nt, int nq, int nkv,
                                    int dh) {
  TA_REF_REQUIRE(nt >= 0 && nq > 0 && nkv > 0 && dh > 0 && dh % 2 == 0, "ta_ref_rope_kv_write: bad sizes");
  TA_REF_REQUIRE(style == 0 || style == 1, "ta_ref_rope_kv_write: unknown pairing %d", style);
  const int half = dh / 2, heads = nq + 2 * nkv;
  for (int t = 0; t < nt; ++t) {
    const bool cache = kcache != nullptr && dest != nullptr;
    const size_t page = cache ? (size_t)(dest[t] / TA_REF_PAGE) : 0;
    const int off = cache ? dest[t] % TA_REF_PAGE : 0;
    for (int h = 0; h < heads; ++h) {
      float* v = qkv + ((size_t)t * heads + h) * dh;
      const float* b = bias ? bias + (size_t)h * dh : nullptr;
      if (h < nq + nkv) {
        for (int j = 0; j < half; ++j) {
          const int i0 = style == 0 ? j : 2 * j, i1 = style == 0 ? j + half : 2 * j + 1;
          double a = v[i0], c = v[i1];
          if (b) {
            a += b[i0];
            c += b[i1];
          }
          double r0 = a, r1 = c;
          if (cs) {
            const double co = cs[((size_t)t * half + j) * 2], si = cs[((size_t)t * half + j) * 2 + 1];
            r0 = a * co - c * si;
            r1 = a * si + c * co;
          }
          v[i0] = (float)r0;
          v[i1] = (float)r1;
        }
        if (h >= nq && cache)
          for (int i = 0; i < dh; ++i)
            kcache[((page * nkv + (h - nq)) * TA_REF_PAGE + off) * dh + i] = v[i];
      } else {
        for (int i = 0; i < dh; ++i) {
          if (b) v[i] = (float)((double)v[i] + b[i]);
          if (cache) vcache[((page * nkv + (h - nq - nkv)) * dh + i) * TA_REF_PAGE + off] = v[i];
        }
      }
    }
  }
  return 0;
}

// out[t][i] = silu(g) * u with g = gu[t][i] (+ bias[i]), u = gu[t][di + i] (+ bias[di + i]),
// silu(z) = z / (1 + exp(-z)) (compute.rs:286-288: gate and up are the two halves of a row).
extern "C" int ta_ref_swiglu(const float* gu, const float* bias, float* out, int nt, int di) {
  TA_REF_REQUIRE(nt >= 0 && di > 0, "ta_ref_swiglu: bad sizes");
  for (int t = 0; t < nt; ++t)
    for (int i = 0; i < di; ++i) {
      double g = gu[(size_t)t * 2 * di + i], u = gu[(size_t)t * 2 * di + di + i];
      if (bias) {
        g += bias[i];
        u += bias[di + i];
      }
      out[(size_t)t * di + i] = (float)(g / (1.0 + std::exp(-g)) * u);
    }
  return 0;
}

// out[i] = mean + std * z_i, z_i from the kernel's generator: the same integer hashes of
// (seed, stream, i) and the same two uniforms (exactly), then one Box-Muller draw, here in
// double (the kernel's float32 logarithm and cosine differ from it by rounding).
static uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

extern "C" int ta_ref_fill_normal(float* out, long long n, unsigned long long seed,
                                  unsigned long long stream_id, float mean, float std_) {
  TA_REF_REQUIRE(n >= 0, "ta_ref_fill_normal: negative size");
  const uint64_t key = mix64(seed * 0x9E3779B97F4A7C15ull + stream_id);
  for (long long i = 0; i < n; ++i) {
    const uint64_t r = mix64(key + (uint64_t)i * 0xD1342543DE82EF95ull);
    const double u1 = ((double)(uint32_t)(r >> 40) + 1.0) / 16777216.0;      // (0, 1]
    const double u2 = (double)(uint32_t)((r >> 8) & 0xffffffu) / 16777216.0;
    const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.28318530717958647692 * u2);
    out[i] = (float)((double)mean + (double)std_ * z);
  }
  return 0;
}

// dst[i] = src[i] in another floating type, as the loader's conversion kernel does it: src is
// float32, bfloat16 (src_type 1) or float16 (src_type 2) given as raw 16-bit patterns; the
// result is returned as float32 holding exactly what dst_type stores (0: float32, widening is
// exact; 1: bfloat16, rounded to nearest, ties to even).
static float half_bits_to_float(uint16_t h) {
  const int sign = h >> 15, exp = (h >> 10) & 31, man = h & 1023;
  double v;
  if (exp == 0) v = std::ldexp((double)man, -24);
  else if (exp == 31) v = man ? std::numeric_limits<double>::quiet_NaN() : std::numeric_limits<double>::infinity();
  else v = std::ldexp(1.0 + man / 1024.0, exp - 15);
  return (float)(sign ? -v : v);
}

static float round_to_bf16(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7f800000u) == 0x7f800000u) return f;              // infinities and NaN keep their class
  u = (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
  std::memcpy(&f, &u, 4);
  return f;
}

extern "C" int ta_ref_convert(int src_type, int dst_type, const void* src, float* dst, long long n) {
  TA_REF_REQUIRE(src_type >= 0 && src_type <= 2 && (dst_type == 0 || dst_type == 1) && n >= 0,
                 "ta_ref_convert: unknown types %d -> %d", src_type, dst_type);
  for (long long i = 0; i < n; ++i) {
    float v;
    if (src_type == 0) {
      v = ((const float*)src)[i];
    } else if (src_type == 1) {
      const uint32_t u = (uint32_t)((const uint16_t*)src)[i] << 16;
      std::memcpy(&v, &u, 4);
    } else {
      v = half_bits_to_float(((const uint16_t*)src)[i]);
    }
    dst[i] = dst_type == 1 ? round_to_bf16(v) : v;
  }
  return 0;
}
