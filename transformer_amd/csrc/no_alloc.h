// An entry point for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in
// the reference, whose attention operator takes its workspace from the caller's stream pool
// (models/llama/common/src/compute.rs:168-183).
//
// ta_attention_keys_bf16_noalloc is ta_attention_keys_bf16 (the single-token attention over
// the paged cache: same arguments, same kernels, same results) without the `scratch`
// argument. The partial rows that its units of work leave for the merge kernel go into a
// buffer that is part of the library's image on every GPU: TA_NOALLOC_SCRATCH_FLOATS float32
// values (4 MiB), which each GPU the library runs on holds until the process ends. The call
// allocates nothing and frees nothing, on the device or through any library.
//
// Limits and rules:
//   * n_units * nh * (dh + 2) must not exceed TA_NOALLOC_SCRATCH_FLOATS (the 8B shape at a
//     batch of 64, cut into 128 units, needs 0.53 M of the 1 M floats); a larger call is refused with an error
//     before anything is launched.
//   * Every call on a GPU shares that GPU's buffer, whatever its stream: calls that overlap on
//     one GPU race. Calls on one stream follow one another and are safe.
//   * The buffer keeps the last call's contents. Nothing in it has to start at zero: a
//     sequence's units all write their partial rows before the merge reads them.
//   * The buffer's address is looked up once per GPU, at the first call made with that GPU
//     current.
#pragma once
#include <hip/hip_runtime.h>

#define TA_NOALLOC_SCRATCH_FLOATS (1 << 20)

extern "C" int ta_attention_keys_bf16_noalloc(hipStream_t stream, const void* qkv, int q_stride,
                                              const float* bias, const float* cs, int style,
                                              const int* dest, void* out, int out_stride,
                                              void* kcache, void* vcache, const int* block_table,
                                              int max_blocks, const int* pos0, int batch, int nh,
                                              int nkv, int dh, float scale, int window,
                                              const int* units, const int* seq_units, int n_units,
                                              int waves);

// Floats of the static buffer (TA_NOALLOC_SCRATCH_FLOATS), for callers that size their batches.
extern "C" long long ta_noalloc_scratch_floats();
