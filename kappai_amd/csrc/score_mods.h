// What an attention kernel may do to a score between the scaled dot product and the softmax, and a
// sink: one more term of the softmax's denominator that has no key and no value.
//   softcap     0: nothing; else score <- softcap * tanh(score / softcap)
//   dist_bias   [heads, dist_cols] float32, added after the cap: column min(i - j, dist_cols - 1)
//               for query position i and key position j; null: nothing
//   sink        [heads] float32: exp(sink[h]) joins the denominator once; null: nothing
#pragma once
#include <hip/hip_runtime.h>

struct kappai_score_mods {
  float softcap;
  const float* dist_bias;
  int dist_cols;
  const float* sink;
};

__host__ __device__ __forceinline__ bool kappai_mods_on(const kappai_score_mods* m) {
  return m != nullptr && (m->softcap > 0.f || m->dist_bias != nullptr || m->sink != nullptr);
}

// `s` is the scaled dot product; the result is what the softmax sees (natural-logarithm units).
__device__ __forceinline__ float kappai_modified_score(const kappai_score_mods& m, float s, int h,
                                                       int dist) {
  if (m.softcap > 0.f) s = m.softcap * tanhf(s / m.softcap);
  if (m.dist_bias != nullptr)
    s += m.dist_bias[(size_t)h * m.dist_cols + max(0, min(dist, m.dist_cols - 1))];
  return s;
}
