// Plain C++ twins of the HIP kernels: what each kernel computes, written as loops over whole
// arrays with double-precision sums, on the host, with no tiling, no reordering and no
// device. They are what the kernel tests compare against from C++ (the NumPy functions under
// tests/ are the other, independent statement of the same formulas); nothing on the product
// path calls them. Arrays are float32 whatever the engine stores (a caller widens bfloat16,
// which is exact, and rounds a result where the kernel stores bfloat16); integer tables are
// int32; the paged cache has the kernels' layout: keys [pages][kv heads][64][head size],
// values [pages][kv heads][head size][64].
//
// Every function returns 0, or 1 after leaving a message for ta_ref_last_error().
#pragma once
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#define TA_REF_PAGE 64

int ta_ref_fail(const char* fmt, ...);

#define TA_REF_REQUIRE(cond, ...)                 \
  do {                                            \
    if (!(cond)) return ta_ref_fail(__VA_ARGS__); \
  } while (0)
