// Score functors and index-computed masks shared by the forward and backward kernels: the
// stand-ins for the score_mod / mask_mod functions (and joint_mod, the derivative of score_mod)
// that the reference renders into its templated kernels
// (torch_neuronx/neuron_dynamo_backend/flex_attention/flex_attention.py.jinja:74-92, applied
// :2495-2660; flex_attention_bwd.py.jinja:958-988, applied :1261-1271).  Order, on s = scale * q.k:
//   s *= key_weight[h][j];  s += key_bias[h][j];  s += alibi[h] * (j - i);  s = cap * tanh(s / cap)
// then the masks (causal, window, document ids).
#pragma once

#include <limits.h>
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

// One score through the functors, element by element (the generic and the float32 kernels):
// x = scale * q.k of (batch b, head h, query i, key j); L and S are the row lengths of the id and
// per-key vectors.  `dfac` receives d mod / d x, which multiplies the gradient of the score; a score
// that the document ids drop comes back as -inf.
__device__ __forceinline__ float score_mod_at(const ScoreMod& sm, float x, int b, int h, int i, int j, int L, int S, float& dfac) {
  dfac = 1.f;
  if (!sm.any) return x;
  if (sm.key_weight) {
    const float w = sm.key_weight[(int64_t)h * S + j];
    x *= w, dfac = w;
  }
  if (sm.key_bias) x += sm.key_bias[(int64_t)h * S + j];
  if (sm.alibi) x = fmaf(sm.alibi[h], (float)(j - i), x);
  if (sm.softcap > 0.f) {
    const float th = tanhf(x / sm.softcap);
    x = sm.softcap * th, dfac *= 1.f - th * th;
  }
  if (sm.doc_q && sm.doc_k && sm.doc_q[(int64_t)b * L + i] != sm.doc_k[(int64_t)b * S + j]) x = -INFINITY;
  return x;
}

// First index of the sorted array a[0 .. n) whose value is >= x (n if none), found by a whole
// wavefront, for N values of x at once: every round samples 64 evenly spaced positions per search
// (all the loads of a round go out together) and keeps the interval between the last sample below x
// and the first one at or above it, so 4096 elements take two trips to memory whatever N is.
// The first round's samples do not depend on x: a caller fetches them (doc_first_samples) together
// with whatever tells it x, which saves one of the trips.
__device__ __forceinline__ int doc_first_samples(const int32_t* a, int n, int lane) {
  const int idx = (lane + 1) * ((n + 63) >> 6) - 1;
  return (n > 0 && idx < n) ? a[idx] : INT_MAX;
}
template <int N>
__device__ __forceinline__ void wave_lower_bounds(const int32_t* a, int n, const int (&x)[N], int (&out)[N], int lane, int first) {
  int lo[N], len[N];
  {  // round one, on the samples the caller brought
    const int step = (n + 63) >> 6;
    const int idx = (lane + 1) * step - 1;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const bool below = n > 0 && idx < n && first < x[i];
      const int cnt = __builtin_popcountll(__builtin_amdgcn_ballot_w64(below));
      lo[i] = cnt * step;
      len[i] = max(min(step - 1, n - lo[i]), 0);
    }
  }
  for (;;) {
    int left = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) left |= len[i];
    if (left <= 0) break;  // (uniform: every lane holds the same intervals)
    int v[N], step[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
      step[i] = (len[i] + 63) >> 6;
      const int idx = lo[i] + (lane + 1) * step[i] - 1;
      v[i] = (len[i] > 0 && idx < lo[i] + len[i]) ? a[idx] : INT_MAX;
    }
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = lo[i] + (lane + 1) * step[i] - 1;
      const bool below = len[i] > 0 && idx < lo[i] + len[i] && v[i] < x[i];
      const int cnt = __builtin_popcountll(__builtin_amdgcn_ballot_w64(below));
      const int end = lo[i] + len[i];
      lo[i] += cnt * step[i];
      len[i] = max(min(step[i] - 1, end - lo[i]), 0);
    }
  }
#pragma unroll
  for (int i = 0; i < N; ++i) out[i] = __builtin_amdgcn_readfirstlane(lo[i]);
}
// The run [first, past) of the sorted ids a[0 .. n) whose value lies in [id_lo, id_hi], for two such
// id ranges at once (a workgroup's rows and a wavefront's rows, say).
__device__ __forceinline__ void doc_runs(const int32_t* a, int n, int lo0, int hi0, int lo1, int hi1, int (&run0)[2], int (&run1)[2],
                                         int lane, int first) {
  const int x[4] = {lo0, hi0 == INT_MAX ? INT_MAX : hi0 + 1, lo1, hi1 == INT_MAX ? INT_MAX : hi1 + 1};
  int r[4];
  wave_lower_bounds<4>(a, n, x, r, lane, first);
  run0[0] = r[0], run0[1] = hi0 == INT_MAX ? n : r[1];
  run1[0] = r[2], run1[1] = hi1 == INT_MAX ? n : r[3];
}
#endif

}  // namespace mi355
