// Generic fused SDPA forward for gfx950: float32 accumulation, any head dim up to 512,
// arbitrary strides, GQA, causal, additive bias or boolean keep-mask, per-batch key
// lengths and a dropout keep-mask.  One 64-lane wavefront owns one query row: lanes span
// 64 keys for the logits and 64 value columns for the output, the running max / sum of the
// online softmax are wave reductions, and nothing is shared between wavefronts.
//
// It is the numerical twin of the math path (torch_neuronx/_sdpa_math.py:51-95): logits are
// (Q K^T) * scale in float32, causal fill comes first and the bias is added after, a row
// with no live key gives a zero output row and lse = -inf, and for half-precision inputs
// the probabilities are rounded to the input dtype before they multiply V.
#include "common.h"
#include "score_mod.h"

namespace mi355 {
namespace {

constexpr int kMaxHeadDim = 512;
constexpr int kWaves = 4;

struct FwdG {
  T4 q, k, v, out, bias;
  float* lse;
  const int32_t* kv_lens;
  const uint8_t* keep;
  int64_t keep_ld;  // bytes from one row of keep bytes to the next
  float keep_scale;  // 1/(1-p), or 1 when p == 1 (the mask alone zeroes everything)
  int B, Hq, Hkv, L, S, E, Dv;
  int causal, bias_kind;  // 0 none, 1 additive, 2 bool
  float scale;
  int window, sink_keys;    // sliding window over the causal pattern: keys i-window+1 .. i and the first sink_keys
  const float* sink_logit;  // (B,Hq,n_sinks): logits without a value that join every row's softmax
  int n_sinks;
  ScoreMod sm;  // score functors and document ids
};

template <typename T, typename TB>
__global__ __launch_bounds__(64 * kWaves) void fwd_generic_kernel(FwdG p) {
  __shared__ float qrow[kWaves][kMaxHeadDim];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kWaves + wave;
  const int64_t rows = (int64_t)p.B * p.Hq * p.L;
  if (row >= rows) return;  // whole wavefront leaves together; no block-level barrier below
  const int i = (int)(row % p.L);
  const int h = (int)((row / p.L) % p.Hq);
  const int b = (int)(row / ((int64_t)p.L * p.Hq));
  const int hk = h / (p.Hq / p.Hkv);

  const T* q = (const T*)p.q.data + b * p.q.st[0] + h * p.q.st[1] + i * p.q.st[2];
  const T* kbase = (const T*)p.k.data + b * p.k.st[0] + hk * p.k.st[1];
  const T* vbase = (const T*)p.v.data + b * p.v.st[0] + hk * p.v.st[1];
  for (int e = lane; e < p.E; e += 64) qrow[wave][e] = to_f32(q[e * p.q.st[3]]);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");  // the row is visible to every lane

  int s_eff = p.S;
  if (p.kv_lens) s_eff = min(s_eff, max(0, p.kv_lens[b]));
  const int s_end = p.causal ? min(s_eff, i + 1) : s_eff;

  constexpr int NV = kMaxHeadDim / 64;
  float acc[NV];
#pragma unroll
  for (int c = 0; c < NV; ++c) acc[c] = 0.f;
  float m = -INFINITY, l = 0.f;

  const TB* bias_row = nullptr;
  if (p.bias_kind)
    bias_row = (const TB*)p.bias.data + b * p.bias.st[0] + h * p.bias.st[1] + i * p.bias.st[2];
  const uint8_t* keep_row =
      p.keep ? p.keep + (((int64_t)b * p.Hq + h) * p.L + i) * p.keep_ld : nullptr;

  for (int j0 = 0; j0 < s_end; j0 += 64) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (j < s_end) {
      const T* kr = kbase + j * p.k.st[2];
      float dot = 0.f;
      for (int e = 0; e < p.E; ++e) dot = fmaf(qrow[wave][e], to_f32(kr[e * p.k.st[3]]), dot);
      s = dot * p.scale;
      if (p.sm.any) {
        if (p.sm.key_weight) s *= p.sm.key_weight[(int64_t)h * p.S + j];
        if (p.sm.key_bias) s += p.sm.key_bias[(int64_t)h * p.S + j];
        if (p.sm.alibi) s = fmaf(p.sm.alibi[h], (float)(j - i), s);
        if (p.sm.softcap > 0.f) s = p.sm.softcap * tanhf(s / p.sm.softcap);
        if (p.sm.doc_q && p.sm.doc_k && p.sm.doc_q[(int64_t)b * p.L + i] != p.sm.doc_k[(int64_t)b * p.S + j]) s = -INFINITY;
      }
      if (p.window > 0 && i - j >= p.window && j >= p.sink_keys) s = -INFINITY;
      if (p.bias_kind == 1) {
        s += to_f32(bias_row[j * p.bias.st[3]]);
      } else if (p.bias_kind == 2) {
        if (!((const uint8_t*)bias_row)[j * p.bias.st[3]]) s = -INFINITY;
      }
    }
    const float tmax = wave_max(s);
    const float m_new = fmaxf(m, tmax);
    if (m_new == -INFINITY) continue;  // uniform: nothing alive yet
    const float alpha = expf(m - m_new);
    float pr = expf(s - m_new);  // exp(-inf) = 0 for masked lanes
    l = l * alpha + wave_sum(pr);
    m = m_new;
    if (keep_row) pr = (j < s_end && keep_row[j]) ? pr * p.keep_scale : 0.f;
    pr = to_f32((T)pr);
#pragma unroll
    for (int c = 0; c < NV; ++c) acc[c] *= alpha;
    const int jn = min(64, s_end - j0);
    for (int jj = 0; jj < jn; ++jj) {
      const float pj = __shfl(pr, jj, 64);
      if (pj == 0.f) continue;
      const T* vr = vbase + (j0 + jj) * p.v.st[2];
#pragma unroll
      for (int c = 0; c < NV; ++c) {
        const int d = lane + 64 * c;
        if (d < p.Dv) acc[c] = fmaf(pj, to_f32(vr[d * p.v.st[3]]), acc[c]);
      }
    }
  }

  if (p.sink_logit) {
    // (several sink logits act as one: the logarithm of the sum of their exponentials)
    const float* zs = p.sink_logit + ((int64_t)b * p.Hq + h) * p.n_sinks;
    float zm = -INFINITY, zl = 0.f;
    for (int n = 0; n < p.n_sinks; ++n) zm = fmaxf(zm, zs[n]);
    for (int n = 0; n < p.n_sinks; ++n) zl += zm == -INFINITY ? 0.f : expf(zs[n] - zm);
    const float z = zm == -INFINITY ? -INFINITY : zm + logf(zl);
    if (z != -INFINITY) {
      const float m2 = fmaxf(m, z);
      const float a = m == -INFINITY ? 0.f : expf(m - m2);
      l = l * a + expf(z - m2);
      m = m2;
#pragma unroll
      for (int c = 0; c < NV; ++c) acc[c] *= a;
    }
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  T* o = (T*)p.out.data + b * p.out.st[0] + h * p.out.st[1] + i * p.out.st[2];
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int d = lane + 64 * c;
    if (d < p.Dv) o[d * p.out.st[3]] = (T)(acc[c] * inv);
  }
  if (p.lse && lane == 0) p.lse[row] = (l > 0.f) ? m + logf(l) : -INFINITY;
}

template <typename T>
int launch_t(const FwdG& g, int bias_dtype, hipStream_t s) {
  const int64_t rows = (int64_t)g.B * g.Hq * g.L;
  dim3 grid((unsigned)((rows + kWaves - 1) / kWaves)), block(64 * kWaves);
  if (g.bias_kind == 2 || g.bias_kind == 0)
    hipLaunchKernelGGL((fwd_generic_kernel<T, uint8_t>), grid, block, 0, s, g);
  else if (bias_dtype == MI355_SDPA_F32)
    hipLaunchKernelGGL((fwd_generic_kernel<T, float>), grid, block, 0, s, g);
  else if (bias_dtype == MI355_SDPA_F16)
    hipLaunchKernelGGL((fwd_generic_kernel<T, f16_t>), grid, block, 0, s, g);
  else if (bias_dtype == MI355_SDPA_BF16)
    hipLaunchKernelGGL((fwd_generic_kernel<T, bf16_t>), grid, block, 0, s, g);
  else {
    set_error("SDPA: unsupported attn_bias dtype %d", bias_dtype);
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  return check_launch("fwd_generic_kernel");
}

}  // namespace

int launch_fwd_generic(const mi355_sdpa_fwd_params& p, hipStream_t s) {
  FwdG g;
  g.q = view(p.q), g.k = view(p.k), g.v = view(p.v), g.out = view(p.out), g.bias = view(p.bias);
  g.lse = p.lse, g.kv_lens = p.kv_lens, g.keep = p.dropout_p > 0.f ? p.dropout_keep : nullptr;
  g.keep_ld = (p.dropout_keep_ld > 0 ? p.dropout_keep_ld : p.k.size[2]);
  g.keep_scale = p.dropout_p < 1.f ? 1.f / (1.f - p.dropout_p) : 1.f;
  g.B = (int)p.q.size[0], g.Hq = (int)p.q.size[1], g.L = (int)p.q.size[2], g.E = (int)p.q.size[3];
  g.Hkv = (int)p.k.size[1], g.S = (int)p.k.size[2], g.Dv = (int)p.v.size[3];
  g.causal = p.is_causal, g.scale = p.scale;
  g.bias_kind = !p.bias.data ? 0 : (p.bias_dtype == MI355_SDPA_BOOL ? 2 : 1);
  g.window = p.mask.window, g.sink_keys = p.mask.sink_keys, g.sink_logit = p.mask.sink_logit;
  g.n_sinks = p.mask.n_sink_logits > 0 ? p.mask.n_sink_logits : 1;
  g.sm = score_mod_of(p.mask);
  if (g.E > kMaxHeadDim || g.Dv > kMaxHeadDim) {
    set_error("SDPA: head dim %d/%d exceeds the supported maximum %d", g.E, g.Dv, kMaxHeadDim);
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  if ((int64_t)g.B * g.Hq * g.L == 0) return MI355_SDPA_OK;
  switch (p.dtype) {
    case MI355_SDPA_F32: return launch_t<float>(g, p.bias_dtype, s);
    case MI355_SDPA_F16: return launch_t<f16_t>(g, p.bias_dtype, s);
    case MI355_SDPA_BF16: return launch_t<bf16_t>(g, p.bias_dtype, s);
  }
  set_error("SDPA: query dtype must be float32, float16, or bfloat16, got dtype id %d", p.dtype);
  return MI355_SDPA_ERR_INVALID;
}

}  // namespace mi355
