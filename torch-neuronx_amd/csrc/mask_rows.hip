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

// ---- the verdict, on the device -------------------------------------------------------------------
// The same decision without a trip to the host: a row summary of every (mask batch, row), and one
// workgroup that holds the summaries against the patterns.  The verdict stays in device memory, where
// the masked variants of the forward and backward kernels read it in their prologue and, for a mask
// that is a pattern, drop the mask in favour of the causal flag and per-batch key counts.  Nothing
// here synchronises, so the whole sequence records into a HIP graph and follows a mask that is
// updated in place between replays.
//   verdict[0] kind: 0 not a pattern, 1 keep-everything, 2 causal, 3 sliding window with sink keys
//   verdict[1] window   verdict[2] sink keys   verdict[3] 1 if some batch keeps fewer than S keys
//   verdict[8 + b] keys of batch b that take part (right padding becomes a key count)
// and behind them the row summaries, four ints per (mask batch, row), and one int per mask batch (the
// key count that a window pattern would have there).
namespace mi355 {
namespace {

struct VerdictArgs {
  const void* mask;
  int64_t sb, sl;  // strides of the mask's batch and row dims in elements (0: broadcast)
  int B, Bm, L, Lm, S;
  int32_t* verdict;
  int32_t* rows;
  int32_t* n_win;  // per mask batch
};

template <typename T>
__global__ __launch_bounds__(256) void mask_rows_batched_kernel(VerdictArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= (int64_t)a.Bm * a.Lm) return;
  const int bm = (int)(row / a.Lm), l = (int)(row % a.Lm);
  const T* m = (const T*)a.mask + bm * a.sb + l * a.sl;
  const int S = a.S;
  // (elements are read sixteen bytes at a time where the row allows it)
  constexpr int E = 16 / (int)sizeof(T);
  const bool wide = ((uintptr_t)m & 15) == 0 && S % E == 0;
  int hi = -1, cnt = 0, lead = S, bad = 0;
  auto scan = [&](auto&& visit) {
    if (wide) {
      for (int j = lane * E; j < S; j += 64 * E) {
        const uint4 w = *(const uint4*)(m + j);
        T e[E];
        __builtin_memcpy(e, &w, 16);
#pragma unroll
        for (int i = 0; i < E; ++i) visit(j + i, classify<T>(e[i]));
      }
    } else {
      for (int j = lane; j < S; j += 64) visit(j, classify<T>(m[j]));
    }
  };
  scan([&](int j, int c) {
    if (c < 0) bad = 1;
    if (c == 1) hi = max(hi, j), ++cnt;
    else lead = min(lead, j);
  });
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    hi = max(hi, __shfl_xor(hi, o, 64));
    cnt += __shfl_xor(cnt, o, 64);
    lead = min(lead, __shfl_xor(lead, o, 64));
    bad |= __shfl_xor(bad, o, 64);
  }
  int gap = -1;  // last dropped key below the last kept one
  if (cnt != hi + 1) {  // (a row that is one run from key 0 has none)
    scan([&](int j, int c) {
      if (j < hi && c != 1) gap = max(gap, j);
    });
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) gap = max(gap, __shfl_xor(gap, o, 64));
  }
  if (lane == 0) {
    int32_t* out = a.rows + row * 4;
    out[0] = hi, out[1] = bad ? -1 : cnt, out[2] = lead, out[3] = gap + 1;
  }
}

// One workgroup: the rules of mask_patterns.py (lens_pattern_from_rows, window_lens_pattern_from_rows),
// held against the row summaries of every mask batch.  Its threads share out the (mask batch, row)
// pairs as one range, so the time does not grow with the batch size on its own.
__global__ __launch_bounds__(1024) void mask_verdict_kernel(VerdictArgs a) {
  const int tid = threadIdx.x;
  const int L = a.L, Lm = a.Lm, S = a.S;
  const bool per_row = Lm == L;  // (otherwise one row stands for every query: no causal, no window)
  const bool windows = per_row && L > 1;
  const int64_t pairs = (int64_t)a.Bm * Lm;
  __shared__ int red_s[16];
  auto block_max = [&](int v) {  // (called by every thread)
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
    __syncthreads();
    if ((tid & 63) == 0) red_s[tid >> 6] = v;
    __syncthreads();
    int r = red_s[0];
#pragma unroll
    for (int w = 1; w < 16; ++w) r = max(r, red_s[w]);
    return r;
  };
  int ok_all = 1, ok_causal = windows, ok_mask = 1;
  const int npairs = (int)pairs;  // (verdict_shape keeps it below 2^29)
  for (int idx = tid; idx < npairs; idx += 1024) {
    const int bm = (int)((unsigned)idx / (unsigned)Lm), i = idx - bm * Lm;
    const int hi_last = a.rows[((int64_t)bm * Lm + Lm - 1) * 4];
    const int n_all = hi_last + 1;
    const int n_causal = hi_last == min(L - 1, S - 1) ? S : hi_last + 1;  // the last row reaches its diagonal: no key is known to be padding
    const int32_t* row = a.rows + (int64_t)idx * 4;
    const int hi = row[0], cnt = row[1], lo = row[3];
    if (cnt < 0) ok_mask = 0;
    if (lo != 0 || hi != n_all - 1 || cnt != n_all) ok_all = 0;
    const int hc = min(min(i, S - 1), n_causal - 1);
    if (lo != 0 || hi != hc || cnt != hc + 1) ok_causal = 0;
  }
  ok_mask = __syncthreads_and(ok_mask);
  ok_all = __syncthreads_and(ok_all) && ok_mask;
  ok_causal = __syncthreads_and(ok_causal) && ok_mask;
  int kind = ok_all ? 1 : ok_causal ? 2 : 0, window = 0, sinks = 0;
  if (!kind && ok_mask && windows) {
    // Sliding window with sink keys, with or without right padding: query i of a batch with n keys
    // keeps the keys of i-W+1 .. i and of the first N that lie below n (all S keys when some row reaches
    // the last diagonal element).  W and N are read where they show: in the last row that has keys of
    // its own, in the (first) batch with the most keys.
    // (the keys of a batch are those up to the last one any of its rows keeps: a maximum per batch, for
    // which a wavefront whose rows belong to one batch, the usual case, adds its own once)
    for (int bm = tid; bm < a.Bm; bm += 1024) a.n_win[bm] = -1;
    __syncthreads();
    for (int base = 0; base < npairs; base += 1024) {  // (every thread makes every trip: the wavefront votes)
      const int idx = base + tid;
      const int bm = idx < npairs ? (int)((unsigned)idx / (unsigned)Lm) : -1;
      int top = idx < npairs ? a.rows[(int64_t)idx * 4] : -1;
      const int bm0 = __builtin_amdgcn_readfirstlane(bm);
      if (__builtin_amdgcn_ballot_w64(bm == bm0) == ~0ull) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) top = max(top, __shfl_xor(top, o, 64));
        if ((tid & 63) == 0 && bm0 >= 0 && top >= 0) atomicMax(&a.n_win[bm0], top);
      } else if (bm >= 0 && top >= 0) {
        atomicMax(&a.n_win[bm], top);
      }
    }
    __syncthreads();
    int n_mine = 0;
    for (int bm = tid; bm < a.Bm; bm += 1024) {
      const int top = a.n_win[bm];
      const int n = top == min(L - 1, S - 1) ? S : top + 1;
      a.n_win[bm] = n;
      n_mine = max(n_mine, n);
    }
    const int n_max = block_max(n_mine);  // (its barriers also publish n_win)
    int b_mine = -0x7fffffff;
    for (int bm = tid; bm < a.Bm; bm += 1024)
      if (a.n_win[bm] == n_max) b_mine = max(b_mine, -bm);
    const int b_sel = -block_max(b_mine);
    int W = 0, N = 0, ok = n_max > 0;
    if (ok) {
      const int32_t* row = a.rows + ((int64_t)b_sel * Lm + min(n_max, L) - 1) * 4;
      const int hi_r = row[0], lead_r = row[2], lo_r = row[3];
      W = hi_r - lo_r + 1, N = lead_r < lo_r ? lead_r : 0;
      ok = W > 0 && lo_r != 0;
    }
    for (int idx = tid; idx < npairs && ok; idx += 1024) {
      const int bm = (int)((unsigned)idx / (unsigned)Lm), i = idx - bm * Lm;
      const int n = a.n_win[bm];
      const int32_t* row = a.rows + (int64_t)idx * 4;
      const int hi = row[0], cnt = row[1], lead = row[2], lo = row[3];
      const int top = min(min(i, S - 1), n - 1), lo_w = max(i - W + 1, 0);
      int e_hi, e_cnt, e_lead, e_lo = 0;
      if (lo_w > top) {  // the window lies behind the batch's keys: the sink keys below n are what is left
        const int m = max(min(N, top + 1), 0);
        e_hi = m - 1, e_cnt = m, e_lead = m;
      } else if (lo_w <= N) {  // the window reaches into the sink keys (or to key 0): one run from key 0
        e_hi = top, e_cnt = top + 1, e_lead = top + 1;
      } else {
        e_hi = top, e_cnt = top - lo_w + 1 + N, e_lead = N, e_lo = lo_w;
      }
      if (hi != e_hi || cnt != e_cnt || lead != e_lead || lo != e_lo) ok = 0;
    }
    if (__syncthreads_and(ok)) kind = 3, window = W, sinks = N;
  }
  // key counts per batch (a mask without a batch dim counts for every batch)
  int short_any = 0;
  for (int b = tid; b < a.B; b += 1024) {
    const int bm = a.Bm > 1 ? b : 0;
    const int hi_last = a.rows[((int64_t)bm * Lm + Lm - 1) * 4];
    int n = S;
    if (kind == 1) n = hi_last + 1;
    else if (kind == 2) n = hi_last == min(L - 1, S - 1) ? S : hi_last + 1;
    else if (kind == 3) n = a.n_win[bm];
    a.verdict[8 + b] = n;
    short_any |= n != S;
  }
  short_any = __syncthreads_or(short_any);
  if (tid == 0) {
    a.verdict[0] = kind, a.verdict[1] = window, a.verdict[2] = sinks, a.verdict[3] = short_any;
    a.verdict[4] = a.verdict[5] = a.verdict[6] = a.verdict[7] = 0;
  }
}

// what a verdict needs of the mask: no dependence on the head, unit stride over keys, a known dtype
bool verdict_shape(const mi355_sdpa_tensor& t, int32_t dtype, int* Bm, int* Lm) {
  if (!t.data) return false;
  if (dtype != MI355_SDPA_BOOL && dtype != MI355_SDPA_F32 && dtype != MI355_SDPA_F16 && dtype != MI355_SDPA_BF16) return false;
  const int64_t B = t.size[0], L = t.size[2], S = t.size[3];
  if (B < 1 || L < 1 || S < 1 || B > (1 << 20) || L > (1 << 24) || S > 0x7fffffff) return false;
  if (t.size[1] > 1 && t.stride[1] != 0) return false;
  if (S > 1 && t.stride[3] != 1) return false;
  *Bm = live_extent(t, 0);
  *Lm = (L > 1 && t.stride[2] == 0) ? 1 : (int)L;
  return (int64_t)*Bm * *Lm * 4 < 0x7fffffff;
}

}  // namespace
}  // namespace mi355

extern "C" size_t mi355_sdpa_mask_verdict_words(const mi355_sdpa_tensor* mask, int32_t dtype) {
  int Bm, Lm;
  if (!mask || !verdict_shape(*mask, dtype, &Bm, &Lm)) return 0;
  return (size_t)8 + (size_t)mask->size[0] + (size_t)Bm * Lm * 4 + (size_t)Bm;
}

extern "C" int mi355_sdpa_mask_verdict(const mi355_sdpa_tensor* mask, int32_t dtype, int32_t* verdict, void* stream) {
  int Bm, Lm;
  if (!mask || !verdict) return set_error("SDPA: mask_verdict needs a mask and an output buffer"), MI355_SDPA_ERR_INVALID;
  if (!verdict_shape(*mask, dtype, &Bm, &Lm))
    return set_error("SDPA: mask_verdict: this mask cannot have a verdict (it depends on the head, its keys are not unit-stride, or its dtype)"),
           MI355_SDPA_ERR_UNSUPPORTED;
  VerdictArgs a;
  a.mask = mask->data;
  a.sb = Bm > 1 ? mask->stride[0] : 0, a.sl = Lm > 1 ? mask->stride[2] : 0;
  a.B = (int)mask->size[0], a.Bm = Bm, a.L = (int)mask->size[2], a.Lm = Lm, a.S = (int)mask->size[3];
  a.verdict = verdict, a.rows = verdict + 8 + a.B, a.n_win = a.rows + (int64_t)Bm * Lm * 4;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)(((int64_t)Bm * Lm + 3) / 4)), block(256);
  switch (dtype) {
    case MI355_SDPA_BOOL: hipLaunchKernelGGL((mask_rows_batched_kernel<uint8_t>), grid, block, 0, s, a); break;
    case MI355_SDPA_F32: hipLaunchKernelGGL((mask_rows_batched_kernel<float>), grid, block, 0, s, a); break;
    case MI355_SDPA_F16: hipLaunchKernelGGL((mask_rows_batched_kernel<f16_t>), grid, block, 0, s, a); break;
    default: hipLaunchKernelGGL((mask_rows_batched_kernel<bf16_t>), grid, block, 0, s, a); break;
  }
  if (int rc = check_launch("mask_rows_batched_kernel")) return rc;
  hipLaunchKernelGGL(mask_verdict_kernel, dim3(1), dim3(1024), 0, s, a);
  return check_launch("mask_verdict_kernel");
}

// ---- tile skip tables ------------------------------------------------------------------------------
// The run-time counterpart of the reference's static tile elimination
// (torch_neuronx/neuron_dynamo_backend/flex_attention/flex_attention.py.jinja:15-33): there the mask
// is a function known when the kernel is rendered, here it is a tensor, so one pass over it records
// which 64-row x 32-key blocks hold at least one kept score.  The forward then walks only those key
// tiles; the dK/dV kernel, whose lanes are keys, gets the transposed map (128 keys x 64 rows).
//
// One workgroup per (mask batch, mask head, 64-row block); a wavefront owns 16 of the rows and reads
// them a dword per lane (4 bool, 2 half, 1 float elements), 16 rows per column of dwords, so every
// element of the mask is read once, 256 contiguous bytes per load.
namespace mi355 {
namespace {

template <int KIND>  // 1 float32, 2 float16, 3 bfloat16, 4 bool: does the dword hold a kept element?
__device__ __forceinline__ bool any_kept(uint32_t w) {
  if constexpr (KIND == 1) return w != 0xff800000u;
  else if constexpr (KIND == 2) return (w & 0xffffu) != 0xfc00u || (w >> 16) != 0xfc00u;
  else if constexpr (KIND == 3) return (w & 0xffffu) != 0xff80u || (w >> 16) != 0xff80u;
  else return w != 0u;
}

struct TileMapArgs {
  const uint32_t* mask;       // dword view of the mask
  int64_t sb, sh, sl;         // strides in dwords
  int Hm, L, S, nrb, words;   // mask heads, rows, keys, 64-row blocks, words per row block
  uint32_t* out;
};

template <int KIND>
__global__ __launch_bounds__(256) void mask_tiles_kernel(TileMapArgs a) {
  constexpr int KP = KIND == 1 ? 1 : KIND == 4 ? 4 : 2;  // keys per dword
  constexpr int LPT = 32 / KP;                           // lanes per 32-key tile
  constexpr int TPC = 64 / LPT;                          // tiles per 64-dword column chunk
  __shared__ uint32_t bits[32];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rb = blockIdx.x % a.nrb, hm = (blockIdx.x / a.nrb) % a.Hm, bm = blockIdx.x / (a.nrb * a.Hm);
  if (tid < 32) bits[tid] = 0u;
  __syncthreads();
  const uint32_t* base = a.mask + bm * a.sb + hm * a.sh;
  const int row0 = rb * 64 + wave * 16;
  const int nd = a.S / KP;  // dwords per row
  for (int c = 0; c * 64 < nd; ++c) {
    const int d = c * 64 + lane;
    bool kept = false;
    if (d < nd) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (row0 + r < a.L) kept |= any_kept<KIND>(base[(int64_t)(row0 + r) * a.sl + d]);
    }
    const uint64_t m = __builtin_amdgcn_ballot_w64(kept);
    if (lane < TPC) {
      const uint64_t part = (m >> (lane * LPT)) & (LPT == 32 ? 0xffffffffull : ((1ull << LPT) - 1));
      const int tile = c * TPC + lane;
      if (part && !((bits[tile >> 5] >> (tile & 31)) & 1u)) atomicOr(&bits[tile >> 5], 1u << (tile & 31));
    }
  }
  __syncthreads();
  if (tid < a.words) a.out[((int64_t)(bm * a.Hm + hm) * a.nrb + rb) * a.words + tid] = bits[tid];
}

// live_t[(batch, head)][key block of 128][word]: bit q = some key tile of the block is live for row block q
__global__ __launch_bounds__(256) void mask_tiles_transpose_kernel(const uint32_t* live, uint32_t* live_t, int heads, int nrb,
                                                                   int words, int nkb, int words_t) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)heads * nkb * words_t) return;
  const int w = (int)(idx % words_t), kb = (int)((idx / words_t) % nkb), bh = (int)(idx / ((int64_t)words_t * nkb));
  uint32_t r = 0u;
  for (int q = w * 32; q < min(w * 32 + 32, nrb); ++q) {
    const uint32_t x = live[((int64_t)bh * nrb + q) * words + (kb >> 3)];
    if ((x >> ((kb & 7) * 4)) & 0xfu) r |= 1u << (q & 31);
  }
  live_t[idx] = r;
}

// the mask's own extents (a broadcast dim counts once) and what a table needs of its layout
bool tile_map_shape(const mi355_sdpa_tensor& t, int32_t dtype, int* Bm, int* Hm, int* nrb, int* words, int* nkb, int* words_t) {
  const int esz = dtype == MI355_SDPA_F32 ? 4 : dtype == MI355_SDPA_BOOL ? 1 : (dtype == MI355_SDPA_F16 || dtype == MI355_SDPA_BF16) ? 2 : 0;
  if (!esz || !t.data) return false;
  const int64_t L = t.size[2], S = t.size[3];
  const int gran = 4 / esz;
  if (L < 1 || S < 1 || S > 32768 || L > (1 << 24)) return false;
  if ((S > 1 && t.stride[3] != 1) || ((uintptr_t)t.data & 3) != 0 || S % gran != 0) return false;
  for (int i = 0; i < 3; ++i)
    if (t.size[i] > 1 && (t.stride[i] % gran) != 0) return false;
  if (L > 1 && t.stride[2] == 0) return false;  // a mask per key: nothing to skip by row block
  *Bm = live_extent(t, 0), *Hm = live_extent(t, 1);
  *nrb = (int)((L + 63) / 64), *words = (int)(((S + 31) / 32 + 31) / 32);
  *nkb = (int)((S + 127) / 128), *words_t = (*nrb + 31) / 32;
  return true;
}

}  // namespace
}  // namespace mi355

extern "C" int mi355_sdpa_mask_tiles_words(const mi355_sdpa_tensor* bias, int32_t bias_dtype, size_t* words, size_t* words_t) {
  if (!bias || !words || !words_t) return set_error("SDPA: mask_tiles_words needs a mask and two outputs"), MI355_SDPA_ERR_INVALID;
  int Bm, Hm, nrb, w, nkb, wt;
  *words = *words_t = 0;
  if (!tile_map_shape(*bias, bias_dtype, &Bm, &Hm, &nrb, &w, &nkb, &wt)) return MI355_SDPA_OK;
  *words = (size_t)Bm * Hm * nrb * w, *words_t = (size_t)Bm * Hm * nkb * wt;
  return MI355_SDPA_OK;
}

extern "C" int mi355_sdpa_mask_tiles(const mi355_sdpa_tensor* bias, int32_t bias_dtype, uint32_t* live_tiles,
                                     uint32_t* live_tiles_t, void* stream) {
  if (!bias || !live_tiles) return set_error("SDPA: mask_tiles needs a mask and an output buffer"), MI355_SDPA_ERR_INVALID;
  int Bm, Hm, nrb, w, nkb, wt;
  if (!tile_map_shape(*bias, bias_dtype, &Bm, &Hm, &nrb, &w, &nkb, &wt))
    return set_error("SDPA: mask_tiles: this mask cannot have tile tables (dtype, alignment, a row stride of 0, or more than 32768 keys)"),
           MI355_SDPA_ERR_UNSUPPORTED;
  const int esz = bias_dtype == MI355_SDPA_F32 ? 4 : bias_dtype == MI355_SDPA_BOOL ? 1 : 2;
  const int gran = 4 / esz;
  TileMapArgs a;
  a.mask = (const uint32_t*)bias->data;
  a.sb = Bm > 1 ? bias->stride[0] / gran : 0, a.sh = Hm > 1 ? bias->stride[1] / gran : 0, a.sl = bias->stride[2] / gran;
  a.Hm = Hm, a.L = (int)bias->size[2], a.S = (int)bias->size[3], a.nrb = nrb, a.words = w, a.out = live_tiles;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)(Bm * Hm * nrb)), block(256);
  switch (bias_dtype) {
    case MI355_SDPA_F32: hipLaunchKernelGGL((mask_tiles_kernel<1>), grid, block, 0, s, a); break;
    case MI355_SDPA_F16: hipLaunchKernelGGL((mask_tiles_kernel<2>), grid, block, 0, s, a); break;
    case MI355_SDPA_BF16: hipLaunchKernelGGL((mask_tiles_kernel<3>), grid, block, 0, s, a); break;
    default: hipLaunchKernelGGL((mask_tiles_kernel<4>), grid, block, 0, s, a); break;
  }
  if (int rc = check_launch("mask_tiles_kernel")) return rc;
  if (live_tiles_t) {
    const int64_t n = (int64_t)Bm * Hm * nkb * wt;
    hipLaunchKernelGGL(mask_tiles_transpose_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, live_tiles, live_tiles_t,
                       Bm * Hm, nrb, w, nkb, wt);
    return check_launch("mask_tiles_transpose_kernel");
  }
  return MI355_SDPA_OK;
}
