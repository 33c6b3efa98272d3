// Generic fused SDPA backward for gfx950, the float32 twin of
// torch_neuronx/_sdpa_math.py:98-176 (compute_attention_backward) with the group sum of
// torch_neuronx/neuron_dynamo_backend/decompositions.py:2569-2599 folded in.
//
// Two passes, no atomics, deterministic:
//   row pass (one wavefront per query row i): delta_i = sum_d dO_id O_id, then over key tiles
//     P = exp(S - lse_i), dP = dO V^T, dLogits = P (dP - delta_i)  [-> grad_bias],  dQ_i += scale dLogits K
//   col pass (one wavefront per key row j of a kv head): over the query heads of the group and
//     their query tiles  dV_j += P^T dO,  dK_j += scale dLogits^T Q
// The row term of the reference, sum_j dP P + sum_d dO (O - P V), equals sum_d dO O for any
// `out` (the two P-dependent parts cancel), so delta is taken from the `out` that is passed.
// A query row with lse = -inf contributes nothing; keys at or past kv_lens[b] get zero grads.
#include "common.h"
#include "score_mod.h"

namespace mi355 {
namespace {

constexpr int kMaxHeadDim = 512;
constexpr int kWaves = 4;
constexpr int NV = kMaxHeadDim / 64;

struct BwdG {
  T4 go, q, k, v, out, gq, gk, gv, bias, gbias;
  const float* lse;
  float* delta;  // workspace (B,Hq,L)
  const int32_t* kv_lens;
  const uint8_t* keep;
  int64_t keep_ld;  // bytes from one row of keep bytes to the next
  float keep_scale;
  int B, Hq, Hkv, L, S, E, Dv;
  int causal, bias_kind;
  float scale;
  int window, sink_keys;  // sliding window over the causal pattern: keys i-window+1 .. i and the first sink_keys
  ScoreMod sm;            // score functors and document ids
};

__device__ __forceinline__ float score_mod_generic(const BwdG& p, float s, int b, int h, int i, int j, float& dfac) {
  return score_mod_at(p.sm, s, b, h, i, j, p.L, p.S, dfac);
}

template <typename TB>
__device__ __forceinline__ float apply_bias(float s, const TB* row, int64_t off, int kind) {
  if (kind == 1) return s + to_f32(row[off]);
  if (kind == 2) return ((const uint8_t*)row)[off] ? s : -INFINITY;
  return s;
}

__device__ __forceinline__ void wave_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <typename T, typename TB>
__global__ __launch_bounds__(64 * kWaves) void bwd_row_kernel(BwdG p) {
  __shared__ float qrow[kWaves][kMaxHeadDim];
  __shared__ float dorow[kWaves][kMaxHeadDim];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kWaves + wave;
  if (row >= (int64_t)p.B * p.Hq * p.L) return;
  const int i = (int)(row % p.L);
  const int h = (int)((row / p.L) % p.Hq);
  const int b = (int)(row / ((int64_t)p.L * p.Hq));
  const int hk = h / (p.Hq / p.Hkv);

  const T* q = (const T*)p.q.data + b * p.q.st[0] + h * p.q.st[1] + i * p.q.st[2];
  const T* go = (const T*)p.go.data + b * p.go.st[0] + h * p.go.st[1] + i * p.go.st[2];
  const T* o = (const T*)p.out.data + b * p.out.st[0] + h * p.out.st[1] + i * p.out.st[2];
  const T* kbase = (const T*)p.k.data + b * p.k.st[0] + hk * p.k.st[1];
  const T* vbase = (const T*)p.v.data + b * p.v.st[0] + hk * p.v.st[1];
  float dpart = 0.f;
  for (int e = lane; e < p.E; e += 64) qrow[wave][e] = to_f32(q[e * p.q.st[3]]);
  for (int d = lane; d < p.Dv; d += 64) {
    const float g = to_f32(go[d * p.go.st[3]]);
    dorow[wave][d] = g;
    dpart = fmaf(g, to_f32(o[d * p.out.st[3]]), dpart);
  }
  const float delta = wave_sum(dpart);
  if (lane == 0) p.delta[row] = delta;
  wave_sync_lds();

  const float lse = p.lse[row];
  const bool dead = lse == -INFINITY;
  int s_eff = p.S;
  if (p.kv_lens) s_eff = min(s_eff, max(0, p.kv_lens[b]));
  const int s_end = dead ? 0 : (p.causal ? min(s_eff, i + 1) : s_eff);

  const TB* bias_row = nullptr;
  if (p.bias_kind)
    bias_row = (const TB*)p.bias.data + b * p.bias.st[0] + h * p.bias.st[1] + i * p.bias.st[2];
  T* gb_row = nullptr;
  if (p.gbias.data)
    gb_row = (T*)p.gbias.data + b * p.gbias.st[0] + h * p.gbias.st[1] + i * p.gbias.st[2];
  const uint8_t* keep_row =
      p.keep ? p.keep + (((int64_t)b * p.Hq + h) * p.L + i) * p.keep_ld : nullptr;

  float acc[NV];
#pragma unroll
  for (int c = 0; c < NV; ++c) acc[c] = 0.f;

  for (int j0 = 0; j0 < p.S; j0 += 64) {
    const int j = j0 + lane;
    float dlog = 0.f, dmod = 1.f;  // gradient of the modified score; derivative of the score functors
    if (j < s_end) {
      const T* kr = kbase + j * p.k.st[2];
      const T* vr = vbase + j * p.v.st[2];
      float dot = 0.f, dp = 0.f;
      for (int e = 0; e < p.E; ++e) dot = fmaf(qrow[wave][e], to_f32(kr[e * p.k.st[3]]), dot);
      for (int d = 0; d < p.Dv; ++d) dp = fmaf(dorow[wave][d], to_f32(vr[d * p.v.st[3]]), dp);
      float dfac;
      const float sm = score_mod_generic(p, dot * p.scale, b, h, i, j, dfac);
      const float s = apply_bias<TB>(sm, bias_row, j * p.bias.st[3], p.bias_kind);
      float pr = expf(s - lse);
      if (p.window > 0 && i - j >= p.window && j >= p.sink_keys) pr = 0.f;
      if (keep_row) dp = keep_row[j] ? dp * p.keep_scale : 0.f;
      dlog = pr * (dp - delta);
      dmod = dfac;
    }
    if (gb_row && j < p.S) gb_row[j * p.gbias.st[3]] = (T)dlog;
    if (j0 >= s_end) {
      if (!gb_row) break;
      continue;
    }
    const float ds = dlog * dmod * p.scale;
    const int jn = min(64, s_end - j0);
    for (int jj = 0; jj < jn; ++jj) {
      const float dj = __shfl(ds, jj, 64);
      if (dj == 0.f) continue;
      const T* kr = kbase + (j0 + jj) * p.k.st[2];
#pragma unroll
      for (int c = 0; c < NV; ++c) {
        const int e = lane + 64 * c;
        if (e < p.E) acc[c] = fmaf(dj, to_f32(kr[e * p.k.st[3]]), acc[c]);
      }
    }
  }
  T* gq = (T*)p.gq.data + b * p.gq.st[0] + h * p.gq.st[1] + i * p.gq.st[2];
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int e = lane + 64 * c;
    if (e < p.E) gq[e * p.gq.st[3]] = (T)acc[c];
  }
}

template <typename T, typename TB>
__global__ __launch_bounds__(64 * kWaves) void bwd_col_kernel(BwdG p) {
  __shared__ float krow[kWaves][kMaxHeadDim];
  __shared__ float vrow[kWaves][kMaxHeadDim];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kWaves + wave;
  if (row >= (int64_t)p.B * p.Hkv * p.S) return;
  const int j = (int)(row % p.S);
  const int hk = (int)((row / p.S) % p.Hkv);
  const int b = (int)(row / ((int64_t)p.S * p.Hkv));
  const int rep = p.Hq / p.Hkv;

  const T* k = (const T*)p.k.data + b * p.k.st[0] + hk * p.k.st[1] + j * p.k.st[2];
  const T* v = (const T*)p.v.data + b * p.v.st[0] + hk * p.v.st[1] + j * p.v.st[2];
  for (int e = lane; e < p.E; e += 64) krow[wave][e] = to_f32(k[e * p.k.st[3]]);
  for (int d = lane; d < p.Dv; d += 64) vrow[wave][d] = to_f32(v[d * p.v.st[3]]);
  wave_sync_lds();

  int s_eff = p.S;
  if (p.kv_lens) s_eff = min(s_eff, max(0, p.kv_lens[b]));
  const bool live_key = j < s_eff;

  float dk[NV], dv[NV];
#pragma unroll
  for (int c = 0; c < NV; ++c) dk[c] = 0.f, dv[c] = 0.f;

  if (live_key) {
    for (int hg = 0; hg < rep; ++hg) {
      const int h = hk * rep + hg;
      const T* qbase = (const T*)p.q.data + b * p.q.st[0] + h * p.q.st[1];
      const T* gobase = (const T*)p.go.data + b * p.go.st[0] + h * p.go.st[1];
      const float* lse = p.lse + ((int64_t)b * p.Hq + h) * p.L;
      const float* delta = p.delta + ((int64_t)b * p.Hq + h) * p.L;
      const int i_begin = p.causal ? (j / 64) * 64 : 0;
      for (int i0 = i_begin; i0 < p.L; i0 += 64) {
        const int i = i0 + lane;
        float pr = 0.f, ds = 0.f;
        if (i < p.L && (!p.causal || j <= i) && (p.window <= 0 || i - j < p.window || j < p.sink_keys)) {
          const float l = lse[i];
          if (l != -INFINITY) {
            const T* qr = qbase + i * p.q.st[2];
            const T* gr = gobase + i * p.go.st[2];
            float dot = 0.f, dp = 0.f;
            for (int e = 0; e < p.E; ++e) dot = fmaf(krow[wave][e], to_f32(qr[e * p.q.st[3]]), dot);
            for (int d = 0; d < p.Dv; ++d) dp = fmaf(vrow[wave][d], to_f32(gr[d * p.go.st[3]]), dp);
            float dfac;
            float s = score_mod_generic(p, dot * p.scale, b, h, i, j, dfac);
            if (p.bias_kind) {
              const TB* brow = (const TB*)p.bias.data + b * p.bias.st[0] + h * p.bias.st[1] + i * p.bias.st[2];
              s = apply_bias<TB>(s, brow, j * p.bias.st[3], p.bias_kind);
            }
            pr = expf(s - l);
            float keepf = 1.f;
            if (p.keep)
              keepf = p.keep[(((int64_t)b * p.Hq + h) * p.L + i) * p.keep_ld + j] ? p.keep_scale : 0.f;
            ds = pr * (dp * keepf - delta[i]) * dfac * p.scale;
            pr *= keepf;
          }
        }
        const int in = min(64, p.L - i0);
        for (int ii = 0; ii < in; ++ii) {
          const float pi = __shfl(pr, ii, 64);
          const float di = __shfl(ds, ii, 64);
          if (pi == 0.f && di == 0.f) continue;
          const T* qr = qbase + (i0 + ii) * p.q.st[2];
          const T* gr = gobase + (i0 + ii) * p.go.st[2];
#pragma unroll
          for (int c = 0; c < NV; ++c) {
            const int x = lane + 64 * c;
            if (x < p.Dv) dv[c] = fmaf(pi, to_f32(gr[x * p.go.st[3]]), dv[c]);
            if (x < p.E) dk[c] = fmaf(di, to_f32(qr[x * p.q.st[3]]), dk[c]);
          }
        }
      }
    }
  }
  T* gk = (T*)p.gk.data + b * p.gk.st[0] + hk * p.gk.st[1] + j * p.gk.st[2];
  T* gv = (T*)p.gv.data + b * p.gv.st[0] + hk * p.gv.st[1] + j * p.gv.st[2];
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int x = lane + 64 * c;
    if (x < p.E) gk[x * p.gk.st[3]] = (T)dk[c];
    if (x < p.Dv) gv[x * p.gv.st[3]] = (T)dv[c];
  }
}

// Gradient of the sink logit z of one (batch, head): the sink's probability in row i is
// exp(z - lse_i) and its dP is 0 (it carries no value), so d z = - sum_i exp(z - lse_i) delta_i.
// One workgroup per (batch, head), summed in a fixed order.
__global__ __launch_bounds__(256) void sink_grad_kernel(const float* lse, const float* delta, const float* z, float* out, int L, int n_sinks) {
  __shared__ float part[256];
  const int bh = blockIdx.x / n_sinks;  // (one workgroup per sink logit: each has its own probability exp(z_n - lse_i))
  const float zz = z[blockIdx.x];
  float s = 0.f;
  for (int i = threadIdx.x; i < L; i += 256) {
    const float l = lse[(int64_t)bh * L + i];
    if (l != -INFINITY && zz != -INFINITY) s -= expf(zz - l) * delta[(int64_t)bh * L + i];
  }
  part[threadIdx.x] = s;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) part[threadIdx.x] += part[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[blockIdx.x] = part[0];
}

template <typename T, typename TB>
int launch_tb(const BwdG& g, hipStream_t s) {
  const int64_t qrows = (int64_t)g.B * g.Hq * g.L, krows = (int64_t)g.B * g.Hkv * g.S;
  dim3 block(64 * kWaves);
  if (qrows) {
    hipLaunchKernelGGL((bwd_row_kernel<T, TB>), dim3((unsigned)((qrows + kWaves - 1) / kWaves)), block, 0, s, g);
    int rc = check_launch("bwd_row_kernel");
    if (rc) return rc;
  }
  if (krows) {
    hipLaunchKernelGGL((bwd_col_kernel<T, TB>), dim3((unsigned)((krows + kWaves - 1) / kWaves)), block, 0, s, g);
    return check_launch("bwd_col_kernel");
  }
  return MI355_SDPA_OK;
}

template <typename T>
int launch_t(const BwdG& g, int bias_dtype, hipStream_t s) {
  if (g.bias_kind != 1) return launch_tb<T, uint8_t>(g, s);
  if (bias_dtype == MI355_SDPA_F32) return launch_tb<T, float>(g, s);
  if (bias_dtype == MI355_SDPA_F16) return launch_tb<T, f16_t>(g, s);
  if (bias_dtype == MI355_SDPA_BF16) return launch_tb<T, bf16_t>(g, s);
  set_error("SDPA: unsupported attn_bias dtype %d", bias_dtype);
  return MI355_SDPA_ERR_UNSUPPORTED;
}

}  // namespace

int launch_sink_grad(const float* lse, const float* delta, const float* sink_logit, float* grad, int64_t heads, int L,
                     int n_sinks, hipStream_t s) {
  if (heads == 0) return MI355_SDPA_OK;
  n_sinks = n_sinks > 0 ? n_sinks : 1;
  hipLaunchKernelGGL(sink_grad_kernel, dim3((unsigned)(heads * n_sinks)), dim3(256), 0, s, lse, delta, sink_logit, grad, L, n_sinks);
  return check_launch("sink_grad_kernel");
}

size_t bwd_generic_workspace(const mi355_sdpa_bwd_params& p) {
  return (size_t)(p.q.size[0] * p.q.size[1] * p.q.size[2]) * sizeof(float);
}

int launch_bwd_generic(const mi355_sdpa_bwd_params& p, hipStream_t s) {
  BwdG g;
  g.go = view(p.grad_out), g.q = view(p.q), g.k = view(p.k), g.v = view(p.v), g.out = view(p.out);
  g.gq = view(p.grad_q), g.gk = view(p.grad_k), g.gv = view(p.grad_v);
  g.bias = view(p.bias), g.gbias = view(p.grad_bias);
  g.lse = p.lse, g.delta = (float*)p.workspace, g.kv_lens = p.kv_lens;
  g.keep = p.dropout_p > 0.f ? p.dropout_keep : nullptr;
  g.keep_ld = (p.dropout_keep_ld > 0 ? p.dropout_keep_ld : p.k.size[2]);
  g.keep_scale = p.dropout_p < 1.f ? 1.f / (1.f - p.dropout_p) : 1.f;
  g.B = (int)p.q.size[0], g.Hq = (int)p.q.size[1], g.L = (int)p.q.size[2], g.E = (int)p.q.size[3];
  g.Hkv = (int)p.k.size[1], g.S = (int)p.k.size[2], g.Dv = (int)p.v.size[3];
  g.causal = p.is_causal, g.scale = p.scale;
  g.bias_kind = !p.bias.data ? 0 : (p.bias_dtype == MI355_SDPA_BOOL ? 2 : 1);
  g.window = p.mask.window, g.sink_keys = p.mask.sink_keys;
  g.sm = score_mod_of(p.mask);
  if (g.E > kMaxHeadDim || g.Dv > kMaxHeadDim) {
    set_error("SDPA: head dim %d/%d exceeds the supported maximum %d", g.E, g.Dv, kMaxHeadDim);
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  int rc;
  switch (p.dtype) {
    case MI355_SDPA_F32: rc = launch_t<float>(g, p.bias_dtype, s); break;
    case MI355_SDPA_F16: rc = launch_t<f16_t>(g, p.bias_dtype, s); break;
    case MI355_SDPA_BF16: rc = launch_t<bf16_t>(g, p.bias_dtype, s); break;
    default:
      set_error("SDPA: query dtype must be float32, float16, or bfloat16, got dtype id %d", p.dtype);
      return MI355_SDPA_ERR_INVALID;
  }
  if (rc == MI355_SDPA_OK && p.grad_sink_logit && p.mask.sink_logit)
    rc = launch_sink_grad(p.lse, g.delta, p.mask.sink_logit, p.grad_sink_logit, (int64_t)g.B * g.Hq, g.L, p.mask.n_sink_logits, s);
  return rc;
}

}  // namespace mi355
