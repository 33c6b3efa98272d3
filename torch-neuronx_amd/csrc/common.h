// Shared device/host helpers for the gfx950 SDPA kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/mi355_sdpa.h"

namespace mi355 {

// host side -------------------------------------------------------------------------------
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
int check_launch(const char* what);
// The dynamic-LDS limit of a kernel, raised once per device and call site: the attribute belongs to a
// device's copy of the kernel, so a process that drives several GPUs sets it on each of them.
struct LdsOnce {
  std::atomic<uint64_t> done{0};  // bit d: set on device d
};
inline hipError_t reserve_lds(LdsOnce& once, const void* kernel, int bytes) {
  int dev = -1;
  const bool known = hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64;
  if (known && (once.done.load(std::memory_order_acquire) >> dev & 1ull)) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && known) once.done.fetch_or(1ull << dev, std::memory_order_release);
  return e;
}

int launch_fwd_generic(const mi355_sdpa_fwd_params& p, hipStream_t s);
int launch_fwd_mfma(const mi355_sdpa_fwd_params& p, hipStream_t s);
size_t fwd_mfma_workspace(const mi355_sdpa_fwd_params& p);  // with which the call would split its keys (0: it would not)
bool fwd_mfma_supported(const mi355_sdpa_fwd_params& p, const char** why);
int launch_bwd_generic(const mi355_sdpa_bwd_params& p, hipStream_t s);
int launch_bwd_mfma(const mi355_sdpa_bwd_params& p, hipStream_t s);
bool bwd_mfma_supported(const mi355_sdpa_bwd_params& p, const char** why);
size_t bwd_generic_workspace(const mi355_sdpa_bwd_params& p);
// d sink_logit = - sum_i exp(sink_logit - lse_i) delta_i per (batch, head); lse natural log, delta = rowsum(dO * O)
// (n_sinks logits per head, each with a gradient of its own)
int launch_sink_grad(const float* lse, const float* delta, const float* sink_logit, float* grad, int64_t heads, int L,
                     int n_sinks, hipStream_t s);
size_t bwd_mfma_workspace(const mi355_sdpa_bwd_params& p);
// float32 inputs on the float32 matrix op (f32_mfma.hip)
bool fwd_f32_mfma_supported(const mi355_sdpa_fwd_params& p, const char** why);
int launch_fwd_f32_mfma(const mi355_sdpa_fwd_params& p, hipStream_t s);
size_t fwd_f32_mfma_workspace(const mi355_sdpa_fwd_params& p);  // with which the call would split its keys (0: it would not)
bool bwd_f32_mfma_supported(const mi355_sdpa_bwd_params& p, const char** why);
int launch_bwd_f32_mfma(const mi355_sdpa_bwd_params& p, hipStream_t s);
size_t bwd_f32_mfma_workspace(const mi355_sdpa_bwd_params& p);
int launch_decode_fp8kv(const mi355_sdpa_decode_params& p, hipStream_t s);
size_t decode_workspace(const mi355_sdpa_decode_params& p);
int decode_pick_splits(const mi355_sdpa_decode_params& p);
int decode_static_scratch(void** device_ptr);

// device side -----------------------------------------------------------------------------
typedef __bf16 bf16_t;
typedef _Float16 f16_t;

struct T4 {  // device view of a 4-D tensor, strides in elements
  const void* data;
  int64_t st[4];
};

// extent of a mask over dim i (batch or head) as far as its data goes: a broadcast dim counts once
static inline int live_extent(const mi355_sdpa_tensor& t, int i) {
  return (t.size[i] > 1 && t.stride[i] != 0) ? (int)t.size[i] : 1;
}

static inline T4 view(const mi355_sdpa_tensor& t) {
  T4 r;
  r.data = t.data;
  for (int i = 0; i < 4; ++i) r.st[i] = t.stride[i];
  return r;
}

// The mask arguments of a call as a kernel body sees them: the parameter block's own, or what a
// verdict about the call's bias (written by mi355_sdpa_mask_verdict) puts in their place.  A verdict
// that names the keep-everything or the causal pattern, or a sliding window with sink keys, each with
// or without right padding, turns the call into one with the causal flag, the window and per-batch key
// counts and no bias (verdict_pattern returns true), and the kernel goes on in its variant for such calls.  Uniform scalar loads, ahead of everything
// else; every kernel of a call applies the same rule to the same block, so they agree.  (Passed
// beside the block rather than written into it: a kernel that modifies its parameter block keeps
// all of it in registers.)
struct MaskArgs {
  int causal, bias_kind;
  const int32_t* kv_lens;
  int window, sink_keys;
};
template <typename P>
__device__ __forceinline__ MaskArgs mask_args_of(const P& p) {
  return MaskArgs{p.causal, p.bias_kind, p.kv_lens, p.window, p.sink_keys};
}
template <typename P>
__device__ __forceinline__ bool verdict_pattern(const P& p, MaskArgs& m) {
  if (!p.verdict) return false;
  const int kind = p.verdict[0];
  // (the variants with dropout have no window: such a mask stays a mask there - one rule for every
  // kernel of a call, the merge kernels included)
  if (kind < 1 || kind > (p.keep_scale != 0.f ? 2 : 3)) return false;
  m.causal = kind >= 2, m.bias_kind = 0, m.kv_lens = p.verdict + 8;
  if (kind == 3) m.window = p.verdict[1], m.sink_keys = p.verdict[2];
  return true;
}

template <typename T>
__device__ __forceinline__ float to_f32(T x) {
  return (float)x;
}

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
  return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
  return x;
}

}  // namespace mi355
