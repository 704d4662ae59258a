// What an attention kernel may do to a score between the scaled dot product and the softmax, and a
// sink: one more term of the softmax's denominator that has no key and no value.
//   softcap     0: nothing; else score <- softcap * tanh(score / softcap)
//   dist_bias   [heads, dist_cols] float32, added after the cap: column min(i - j, dist_cols - 1)
//               for query position i and key position j; null: nothing
//   sink        [heads] float32: exp(sink[h]) joins the denominator once; null: nothing
#pragma once
#include <hip/hip_runtime.h>

// Which keys a position sees, as one number that every attention kernel takes in its `window`
// place: 0: all keys up to its own; n > 0: the last n (a sliding window); n < 0: those of its
// own chunk of -n positions, chunks counted from position 0 of the sequence.  The first key seen
// never moves back as the position grows, which is all the kernels' tile bounds rely on.
__host__ __device__ __forceinline__ int kappai_first_key(int pos, int window) {
  if (window > 0) return pos + 1 > window ? pos + 1 - window : 0;
  if (window < 0) return pos < 0 ? 0 : pos - pos % (-window);
  return 0;
}

struct kappai_score_mods {
  float softcap;
  const float* dist_bias;
  int dist_cols;
  const float* sink;
};

__host__ __device__ __forceinline__ bool kappai_mods_on(const kappai_score_mods* m) {
  return m != nullptr && (m->softcap > 0.f || m->dist_bias != nullptr || m->sink != nullptr);
}

// (a cap or a bias: the scores themselves change; a sink alone leaves them as they are)
__host__ __device__ __forceinline__ bool kappai_mods_change_scores(const kappai_score_mods* m) {
  return m != nullptr && (m->softcap > 0.f || m->dist_bias != nullptr);
}

// cap * tanh(s / cap) for the kernels that work in bfloat16: tanh(x) = 1 - 2 / (1 + e^(2x)) by the
// hardware's exponential and reciprocal (absolute error of a few 1e-7 of the cap).
__device__ __forceinline__ float kappai_fast_cap(float s, float cap) {
  const float e = __builtin_amdgcn_exp2f(s * (2.885390081777927f / cap));    // 2 log2(e) / cap
  return cap * (1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + e));
}

// `s` is the scaled dot product; the result is what the softmax sees (natural-logarithm units).
__device__ __forceinline__ float kappai_modified_score(const kappai_score_mods& m, float s, int h,
                                                       int dist) {
  if (m.softcap > 0.f) s = m.softcap * tanhf(s / m.softcap);
  if (m.dist_bias != nullptr)
    s += m.dist_bias[(size_t)h * m.dist_cols + max(0, min(dist, m.dist_cols - 1))];
  return s;
}
