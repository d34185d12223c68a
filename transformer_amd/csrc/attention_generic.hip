// Causal grouped-query attention over the paged cache, float32 arithmetic on the
// vector ALU, for any head size that is a multiple of 16 up to 256 and both
// storage types. It serves prompts and single tokens alike.
//
// A workgroup owns 16 "rows" of one (sequence, kv head): row = (query token,
// query head inside the kv head's group), so the heads of a group share every
// key/value load. Keys are walked in chunks of 32 aligned to absolute positions
// and every row's running maximum, sum and output are updated in that order, so
// a row's result depends only on its own query and keys: not on the batch, not
// on how the tokens were cut into steps, not on which pages hold the keys.
#include "common.h"

#define ROWS 16
#define CHUNK 32

__device__ __forceinline__ float group16_max(float v) {
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 16));
  return v;
}
__device__ __forceinline__ float group16_sum(float v) {
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, 16);
  return v;
}

template <typename T>
__global__ __launch_bounds__(256) void attn_generic_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
    const T* __restrict__ kcache, const T* __restrict__ vcache,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ pos0, int nh, int nkv, int dh, float scale, int window) {
  extern __shared__ float smem[];
  const int group = nh / nkv;
  const int b = blockIdx.z, kvh = blockIdx.y;
  const int q0 = cu_q[b], qlen = cu_q[b + 1] - q0;
  const int nrows = qlen * group;
  const int row0 = blockIdx.x * ROWS;
  if (row0 >= nrows) return;
  const int p0 = pos0[b];
  const int rloc = threadIdx.x / 16, lane = threadIdx.x % 16;
  const int row = row0 + rloc;
  const bool row_ok = row < nrows;
  const int qi = row_ok ? row / group : 0;
  const int head = kvh * group + (row_ok ? row % group : 0);
  const int DHP = dh + 1;
  float* Qs = smem;                 // [ROWS][dh]
  float* KVs = Qs + ROWS * dh;      // [CHUNK][dh + 1]
  float* Ps = KVs + CHUNK * DHP;    // [ROWS][CHUNK]

  for (int i = threadIdx.x; i < ROWS * dh; i += 256) {
    const int r = i / dh, d = i - r * dh, rr = row0 + r;
    float v = 0.f;
    if (rr < nrows)
      v = to_f32(q[(size_t)(q0 + rr / group) * q_stride + (size_t)(kvh * group + rr % group) * dh + d]);
    Qs[i] = v;
  }

  // key range of this tile of rows
  const int qi_min = row0 / group;
  const int last_row = (row0 + ROWS - 1 < nrows - 1) ? row0 + ROWS - 1 : nrows - 1;
  const int tile_end = p0 + last_row / group + 1;                       // exclusive
  int tile_start = 0;
  if (window > 0) {
    tile_start = p0 + qi_min + 1 - window;
    if (tile_start < 0) tile_start = 0;
  }
  const int my_end = p0 + qi + 1;
  int my_start = 0;
  if (window > 0) {
    my_start = my_end - window;
    if (my_start < 0) my_start = 0;
  }

  const int nd = dh / 16;
  float acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;

  const int* table = block_table + (size_t)b * max_blocks;
  for (int c = tile_start / CHUNK; c * CHUNK < tile_end; ++c) {
    const int key0 = c * CHUNK;
    const size_t page = (size_t)table[key0 / TA_PAGE];
    const size_t base = ((page * nkv + kvh) * TA_PAGE + key0 % TA_PAGE) * (size_t)dh;
    const size_t vbase = (page * nkv + kvh) * (size_t)dh * TA_PAGE + key0 % TA_PAGE;
    // ---- K chunk -> LDS (keys that are not written yet read as zero)
    for (int i = threadIdx.x; i < CHUNK * dh; i += 256) {
      const int k = i / dh, d = i - k * dh;
      KVs[k * DHP + d] = (key0 + k < tile_end) ? to_f32(kcache[base + i]) : 0.f;
    }
    __syncthreads();
    float s0 = 0.f, s1 = 0.f;
    {
      const float* qr = Qs + rloc * dh;
      const float* k0 = KVs + lane * DHP;
      const float* k1 = KVs + (lane + 16) * DHP;
      for (int d = 0; d < dh; ++d) {
        const float qv = qr[d];
        s0 = fmaf(qv, k0[d], s0);
        s1 = fmaf(qv, k1[d], s1);
      }
    }
    const int kk0 = key0 + lane, kk1 = kk0 + 16;
    const bool v0 = row_ok && kk0 >= my_start && kk0 < my_end;
    const bool v1 = row_ok && kk1 >= my_start && kk1 < my_end;
    s0 = v0 ? s0 * scale : -INFINITY;
    s1 = v1 ? s1 * scale : -INFINITY;
    const float m_new = fmaxf(m, group16_max(fmaxf(s0, s1)));
    float alpha = 1.f, e0 = 0.f, e1 = 0.f;
    if (m_new != -INFINITY) {
      alpha = expf(m - m_new);          // m = -inf gives 0
      e0 = v0 ? expf(s0 - m_new) : 0.f;
      e1 = v1 ? expf(s1 - m_new) : 0.f;
    }
    l = l * alpha + group16_sum(e0 + e1);
    m = m_new;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] *= alpha;
    Ps[rloc * CHUNK + lane] = e0;
    Ps[rloc * CHUNK + lane + 16] = e1;
    __syncthreads();
    // ---- V chunk -> LDS
    for (int i = threadIdx.x; i < CHUNK * dh; i += 256) {     // value pages are [dh][TA_PAGE]
      const int d = i / CHUNK, k = i - d * CHUNK;
      KVs[k * DHP + d] = (key0 + k < tile_end) ? to_f32(vcache[vbase + (size_t)d * TA_PAGE + k]) : 0.f;
    }
    __syncthreads();
    {
      const float* pr = Ps + rloc * CHUNK;
      for (int k = 0; k < CHUNK; ++k) {
        const float p = pr[k];
        const float* vr = KVs + k * DHP + lane;
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (i < nd) acc[i] = fmaf(p, vr[16 * i], acc[i]);
      }
    }
    __syncthreads();
  }
  if (row_ok) {
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    T* o = out + (size_t)(q0 + qi) * out_stride + (size_t)head * dh + lane;
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (i < nd) o[16 * i] = from_f32<T>(acc[i] * inv);
  }
}

// q: [nt, ...] with q_stride elements between tokens, head h at offset h*dh.
// out: [nt, nh*dh] with out_stride elements between tokens.
// kcache: one layer, [pages][nkv][TA_PAGE][dh]; vcache: [pages][nkv][dh][TA_PAGE].
// block_table: [B][max_blocks].
// cu_q: [B+1] first token of each sequence in q. pos0: [B] tokens cached before this
// step (the step's own keys are already in the cache). window <= 0: all keys.
extern "C" int ta_attention_generic(hipStream_t stream, int dtype, const void* q, int q_stride,
                                    void* out, int out_stride, const void* kcache,
                                    const void* vcache, const int* block_table, int max_blocks,
                                    const int* cu_q, const int* pos0, int batch, int max_qlen,
                                    int nh, int nkv, int dh, float scale, int window) {
  TA_REQUIRE(batch >= 0 && max_qlen >= 0, "ta_attention_generic: bad batch=%d max_qlen=%d", batch, max_qlen);
  TA_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "ta_attention_generic: %d heads do not divide into %d kv heads", nh, nkv);
  TA_REQUIRE(dh >= 16 && dh <= 256 && dh % 16 == 0,
             "ta_attention_generic: head size %d is not a multiple of 16 in [16, 256]", dh);
  TA_REQUIRE(q_stride >= nh * dh && out_stride >= nh * dh, "ta_attention_generic: strides too small");
  TA_REQUIRE(max_blocks > 0, "ta_attention_generic: empty block table");
  TA_REQUIRE(batch <= 65535 && nkv <= 65535, "ta_attention_generic: grid too large");
  if (batch == 0 || max_qlen == 0) return 0;
  const int group = nh / nkv;
  dim3 g((max_qlen * group + ROWS - 1) / ROWS, nkv, batch), blk(256);
  const size_t lds = (size_t)(ROWS * dh + CHUNK * (dh + 1) + ROWS * CHUNK) * sizeof(float);
  if (dtype == TA_F32)
    attn_generic_kernel<float><<<g, blk, lds, stream>>>(
        (const float*)q, q_stride, (float*)out, out_stride, (const float*)kcache,
        (const float*)vcache, block_table, max_blocks, cu_q, pos0, nh, nkv, dh, scale, window);
  else if (dtype == TA_BF16)
    attn_generic_kernel<bf16_t><<<g, blk, lds, stream>>>(
        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kcache,
        (const bf16_t*)vcache, block_table, max_blocks, cu_q, pos0, nh, nkv, dh, scale, window);
  else
    return ta_fail("ta_attention_generic: unknown dtype %d", dtype);
  return ta_check_launch("ta_attention_generic");
}
