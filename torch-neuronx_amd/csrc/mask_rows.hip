// Row summary of an attention mask: the run-time stand-in for the graph pass that recovers
// causality from an explicit mask
// (torch_neuronx/neuron_dynamo_backend/fx/passes/sdpa_causal_mask.py:162-289).  That pass proves at
// trace time that a mask is lower-triangular and rewrites the call to is_causal=True, so that the
// fused kernel stays eligible; here the mask only exists as a tensor, so one small kernel reads it
// once and the host decides from four numbers per row whether the mask is a pattern that a kernel
// can generate by itself (causal, sliding window with sink keys, keep-everything).
//
// One wavefront per row.  An element counts as kept if it is a non-zero bool or a float 0, as
// dropped if it is a zero bool or a float -inf; any other float value means that the tensor is a
// real bias, not a mask.  Per row: { last kept key, number of kept keys (-1: not a mask), length of
// the kept run that starts at key 0, first key of the kept run that ends at the last kept key }.
#include "common.h"

namespace mi355 {
namespace {

template <typename T>
__device__ __forceinline__ int classify(T x) {  // 1 kept, 0 dropped, -1 neither
  const float f = (float)x;
  return f == 0.f ? 1 : (f == -INFINITY ? 0 : -1);
}
template <>
__device__ __forceinline__ int classify<uint8_t>(uint8_t x) {
  return x ? 1 : 0;
}

template <typename T>
__global__ __launch_bounds__(256) void mask_rows_kernel(const T* mask, int64_t row_stride, int L, int S, int32_t* out) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= L) return;
  const T* m = mask + (int64_t)row * row_stride;
  int hi = -1, cnt = 0, lead = S, bad = 0;
  for (int j = lane; j < S; j += 64) {
    const int c = classify<T>(m[j]);
    if (c < 0) bad = 1;
    if (c == 1) hi = j, ++cnt;
    else lead = min(lead, j);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    hi = max(hi, __shfl_xor(hi, o, 64));
    cnt += __shfl_xor(cnt, o, 64);
    lead = min(lead, __shfl_xor(lead, o, 64));
    bad |= __shfl_xor(bad, o, 64);
  }
  int gap = -1;  // last dropped key below the last kept one
  for (int j = lane; j < hi; j += 64)
    if (classify<T>(m[j]) != 1) gap = j;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) gap = max(gap, __shfl_xor(gap, o, 64));
  if (lane == 0) {
    out[row * 4 + 0] = hi;
    out[row * 4 + 1] = bad ? -1 : cnt;
    out[row * 4 + 2] = lead;
    out[row * 4 + 3] = gap + 1;
  }
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int mi355_sdpa_mask_rows(const void* mask, int32_t dtype, int64_t L, int64_t S, int64_t row_stride,
                                    int32_t* rows_out, void* stream) {
  if (!mask || !rows_out) return set_error("SDPA: mask_rows needs a mask and an output buffer"), MI355_SDPA_ERR_INVALID;
  if (L < 0 || S < 0 || L > 0x7fffffff / 4 || S > 0x7fffffff) return set_error("SDPA: mask_rows: bad sizes"), MI355_SDPA_ERR_INVALID;
  if (L == 0) return MI355_SDPA_OK;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)((L + 3) / 4)), block(256);
  switch (dtype) {
    case MI355_SDPA_BOOL:
      hipLaunchKernelGGL((mask_rows_kernel<uint8_t>), grid, block, 0, s, (const uint8_t*)mask, row_stride, (int)L, (int)S, rows_out);
      break;
    case MI355_SDPA_F32:
      hipLaunchKernelGGL((mask_rows_kernel<float>), grid, block, 0, s, (const float*)mask, row_stride, (int)L, (int)S, rows_out);
      break;
    case MI355_SDPA_F16:
      hipLaunchKernelGGL((mask_rows_kernel<f16_t>), grid, block, 0, s, (const f16_t*)mask, row_stride, (int)L, (int)S, rows_out);
      break;
    case MI355_SDPA_BF16:
      hipLaunchKernelGGL((mask_rows_kernel<bf16_t>), grid, block, 0, s, (const bf16_t*)mask, row_stride, (int)L, (int)S, rows_out);
      break;
    default:
      return set_error("SDPA: mask_rows: mask dtype must be bool, float32, float16 or bfloat16"), MI355_SDPA_ERR_INVALID;
  }
  return check_launch("mask_rows_kernel");
}
