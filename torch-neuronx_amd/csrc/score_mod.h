// Score functors and index-computed masks shared by the forward and backward kernels: the
// stand-ins for the score_mod / mask_mod functions (and joint_mod, the derivative of score_mod)
// that the reference renders into its templated kernels
// (torch_neuronx/neuron_dynamo_backend/flex_attention/flex_attention.py.jinja:74-92, applied
// :2495-2660; flex_attention_bwd.py.jinja:958-988, applied :1261-1271).  Order, on s = scale * q.k:
//   s *= key_weight[h][j];  s += key_bias[h][j];  s += alibi[h] * (j - i);  s = cap * tanh(s / cap)
// then the masks (causal, window, document ids).
#pragma once

#include <stdint.h>

#include "../../include/mi355_sdpa.h"

namespace mi355 {

struct ScoreMod {
  const float* alibi = nullptr;       // (Hq,)
  const float* key_bias = nullptr;    // (Hq, S)
  const float* key_weight = nullptr;  // (Hq, S)
  const int32_t* doc_q = nullptr;     // (B, L)
  const int32_t* doc_k = nullptr;     // (B, S)
  float softcap = 0.f;
  int doc_sorted = 0;
  int any = 0;  // one of the above is set
};

static inline ScoreMod score_mod_of(const mi355_sdpa_mask_spec& m) {
  ScoreMod s;
  s.alibi = m.alibi_slopes, s.key_bias = m.key_bias, s.key_weight = m.key_weight;
  s.doc_q = m.doc_ids_q, s.doc_k = m.doc_ids_k;
  s.softcap = m.softcap > 0.f ? m.softcap : 0.f;
  s.doc_sorted = m.doc_ids_sorted != 0 && m.doc_ids_q && m.doc_ids_k;
  s.any = s.alibi || s.key_bias || s.key_weight || (s.doc_q && s.doc_k) || s.softcap > 0.f;
  return s;
}

#if defined(__HIPCC__)
// tanh through one exponential and one reciprocal: 1 - 2 / (1 + e^(2x)); saturates cleanly (e = inf
// gives 1, e = 0 gives -1) and is good to about 1e-7 absolute, which is what a score needs
__device__ __forceinline__ float tanh_fast(float x) {
  const float e = __builtin_amdgcn_exp2f(x * 2.885390081777927f);  // 2 log2(e)
  return 1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f);
}

// First index of the sorted array a[0 .. n) whose value is >= x (n if none), found by a whole
// wavefront: every round samples 64 evenly spaced positions and keeps the interval between the last
// sample below x and the first one at or above it, so 4096 elements take two rounds of one load each.
__device__ __forceinline__ int wave_lower_bound(const int32_t* a, int n, int x, int lane) {
  int lo = 0, len = n;
  while (len > 0) {
    const int step = (len + 63) >> 6;
    const int idx = lo + (lane + 1) * step - 1;
    const bool below = idx < lo + len && a[idx] < x;
    const int cnt = __builtin_popcountll(__builtin_amdgcn_ballot_w64(below));
    const int end = lo + len;
    lo += cnt * step;
    len = min(step - 1, end - lo);
  }
  return __builtin_amdgcn_readfirstlane(lo);
}
#endif

}  // namespace mi355
