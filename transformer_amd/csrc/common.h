// Shared device helpers and the host-side error convention of the kernel library.
//
// Every exported function returns 0 on success. On failure it returns non-zero
// and leaves a message that ta_last_error() returns; arguments are checked on
// the host before any kernel is launched, so a refused call has launched nothing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#define TA_WAVE 64
#define TA_PAGE 64   // tokens per cache page; the Python side asserts the same number
#define TA_UNIT_INTS 8    // int32 values in the record of a unit of work of the single-token attention
#define TA_MAX_PLANES 8   // parts in which a product may leave a float32 result for the next norm to add

enum ta_dtype { TA_F32 = 0, TA_BF16 = 1 };

struct bf16_t {
  uint16_t v;
};

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return __uint_as_float(((uint32_t)x.v) << 16); }

// round to nearest even with the hardware's conversion (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  const __bf16 b = (__bf16)f;
  return __builtin_bit_cast(uint16_t, b);
}
// two values in one instruction: a in the low half, b in the high half
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float a, float b) {
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
  bf16x2_t v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

template <typename T> __device__ __forceinline__ T from_f32(float f);
template <> __device__ __forceinline__ float from_f32<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float f) {
  bf16_t r;
  r.v = f32_to_bf16_bits(f);
  return r;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = TA_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, TA_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = TA_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, TA_WAVE));
  return v;
}

// ---------------------------------------------------------------- host side
int ta_fail(const char* fmt, ...);            // records the message, returns 1
int ta_check_launch(const char* what);        // hipGetLastError -> message

#define TA_REQUIRE(cond, ...)            \
  do {                                   \
    if (!(cond)) return ta_fail(__VA_ARGS__); \
  } while (0)
