// Plain twin of the attention kernels (attention_generic.hip, attention_mfma.hip): causal
// grouped-query attention of each sequence's new tokens over its keys in the paged cache.
#include "ref_common.h"

#include <cmath>
#include <vector>

// Sequence b brings rows cu_q[b] .. cu_q[b+1] of q; its new tokens sit at positions
// pos0[b], pos0[b] + 1, ..., and its cache (which already holds these tokens' keys and
// values) is reached through row b of block_table: position p lies in page
// block_table[b][p / 64] at offset p % 64. Query head h reads kv head h / (nh / nkv). A query
// at position p sees keys 0..p, or keys p - window + 1 .. p with a window
// (models/llama/common/src/compute.rs:243-264: keys 0..pos+seq of the request's cache; no
// scale and no mask are arguments of the reference's operator, :511-526).
//   s_j = scale * q . k_j;  p_j = exp(s_j - max s) / sum;  out = sum p_j v_j
extern "C" int ta_ref_attention(const float* q, int q_stride, float* out, int out_stride,
                                const float* kcache, const float* vcache, const int* block_table,
                                int max_blocks, const int* cu_q, const int* pos0, int batch, int nh,
                                int nkv, int dh, float scale, int window) {
  TA_REF_REQUIRE(batch >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0 && dh > 0, "ta_ref_attention: bad sizes");
  TA_REF_REQUIRE(q_stride >= nh * dh && out_stride >= nh * dh && max_blocks > 0, "ta_ref_attention: bad strides");
  const int group = nh / nkv;
  std::vector<double> s, o(dh);
  for (int b = 0; b < batch; ++b) {
    const int* table = block_table + (size_t)b * max_blocks;
    for (int row = cu_q[b]; row < cu_q[b + 1]; ++row) {
      const int p = pos0[b] + (row - cu_q[b]);
      const int first = (window > 0 && p + 1 > window) ? p + 1 - window : 0;
      TA_REF_REQUIRE(p / TA_REF_PAGE < max_blocks, "ta_ref_attention: position %d is past the block table", p);
      for (int h = 0; h < nh; ++h) {
        const int g = h / group;
        const float* qv = q + (size_t)row * q_stride + (size_t)h * dh;
        s.assign(p + 1, 0.0);
        double top = -INFINITY;
        for (int j = first; j <= p; ++j) {
          const float* kv = kcache + (((size_t)table[j / TA_REF_PAGE] * nkv + g) * TA_REF_PAGE + j % TA_REF_PAGE) * dh;
          double dot = 0.0;
          for (int i = 0; i < dh; ++i) dot += (double)qv[i] * kv[i];
          s[j] = dot * scale;
          if (s[j] > top) top = s[j];
        }
        double sum = 0.0;
        for (int i = 0; i < dh; ++i) o[i] = 0.0;
        for (int j = first; j <= p; ++j) {
          const double w = std::exp(s[j] - top);
          sum += w;
          const float* vv = vcache + ((size_t)table[j / TA_REF_PAGE] * nkv + g) * (size_t)dh * TA_REF_PAGE + j % TA_REF_PAGE;
          for (int i = 0; i < dh; ++i) o[i] += w * vv[(size_t)i * TA_REF_PAGE];
        }
        for (int i = 0; i < dh; ++i) out[(size_t)row * out_stride + (size_t)h * dh + i] = (float)(o[i] / sum);
      }
    }
  }
  return 0;
}
