// Plain twins of sampling.hip: argmax, and the draw from softmax(logits / temperature) cut
// by top-k and top-p.
#include "ref_common.h"

#include <algorithm>
#include <cmath>
#include <numeric>
#include <vector>

// out[r] = index of the highest logit of row r, the lowest index among equals; NaN never wins
// over a number.
extern "C" int ta_ref_argmax(const float* logits, long long ld, int n, int vocab, int* out) {
  TA_REF_REQUIRE(n >= 0 && vocab > 0 && ld >= vocab, "ta_ref_argmax: bad sizes");
  for (int r = 0; r < n; ++r) {
    const float* row = logits + (size_t)r * ld;
    int best = -1;
    for (int i = 0; i < vocab; ++i) {
      if (row[i] != row[i]) continue;
      if (best < 0 || row[i] > row[best]) best = i;
    }
    out[r] = best < 0 ? 0 : best;
  }
  return 0;
}

// The kernel's rule on the same fixed-point masses q_i = floor(2^40 exp((l_i - max) / T)):
// tokens are preferred by higher logit, then lower index; kept are the first top_k of that
// order, cut after the token with which the kept mass reaches ceil(top_p * total mass); the
// token drawn for u in [0, 1) is the first kept token, in index order, whose running sum of
// kept masses exceeds floor(u * kept mass). (The reference hands temperature, top_p, top_k
// and one random number per row to an external operator:
// tensor/src/operators/random_sample.rs:64-75.) The masses come from the double
// exponential here and from the hardware's exp2 in the kernel, so a mass may differ in its
// last bits and a draw that falls within them of a boundary may go to the neighbour.
// `kept` (optional, [n][vocab]) receives the kept masses as doubles, 0 for tokens cut off.
extern "C" int ta_ref_sample(const float* logits, long long ld, int n, int vocab, float temperature,
                             int top_k, float top_p, const float* uniform, int* out, double* kept) {
  TA_REF_REQUIRE(n >= 0 && vocab > 0 && ld >= vocab, "ta_ref_sample: bad sizes");
  TA_REF_REQUIRE(temperature > 0.f && top_k >= 1 && top_p >= 0.f && top_p <= 1.f, "ta_ref_sample: bad arguments");
  std::vector<uint64_t> q(vocab);
  std::vector<int> order(vocab);
  std::vector<char> keep(vocab);
  for (int r = 0; r < n; ++r) {
    const float* row = logits + (size_t)r * ld;
    float top = row[0];
    for (int i = 1; i < vocab; ++i) top = std::max(top, row[i]);
    unsigned __int128 total = 0;
    for (int i = 0; i < vocab; ++i) {
      q[i] = (uint64_t)std::floor(1099511627776.0 * std::exp(((double)row[i] - (double)top) / (double)temperature));
      total += q[i];
    }
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return row[x] > row[y]; });
    const long double limit = std::ceil((long double)top_p * (long double)total);
    std::fill(keep.begin(), keep.end(), 0);
    unsigned __int128 mass = 0;
    const int k = std::min(top_k, vocab);
    for (int j = 0; j < k; ++j) {
      keep[order[j]] = 1;
      mass += q[order[j]];
      if (top_p < 1.0f && (long double)mass >= limit) break;
    }
    if (kept)
      for (int i = 0; i < vocab; ++i) kept[(size_t)r * vocab + i] = keep[i] ? (double)q[i] : 0.0;
    const unsigned __int128 target = (unsigned __int128)std::floor((long double)uniform[r] * (long double)mass);
    unsigned __int128 run = 0;
    int chosen = order[0];
    for (int i = 0; i < vocab; ++i) {
      if (!keep[i]) continue;
      run += q[i];
      if (run > target) {
        chosen = i;
        break;
      }
    }
    out[r] = chosen;
  }
  return 0;
}
