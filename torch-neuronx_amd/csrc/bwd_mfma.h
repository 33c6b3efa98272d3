// Parameter block shared by the MFMA backward kernels.
#pragma once

#include "mfma_common.h"
#include "score_mod.h"

namespace mi355 {

struct BwdM {
  const void *go, *q, *k, *v, *out;
  const float* lse;
  void *gq, *gk, *gv;
  float* delta;  // workspace: rowsum(dO * O) per query row (B, Hq, L)
  float* lse2;   // workspace: the log-sum-exp in the log2 domain, +inf for rows without a live key
  int64_t go_sb, go_sh, go_sl, q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl;
  int64_t o_sb, o_sh, o_sl, gq_sb, gq_sh, gq_sl, gk_sb, gk_sh, gk_sl, gv_sb, gv_sh, gv_sl;
  int B, Hq, Hkv, L, S;
  int n_qt, n_kt;
  int causal, xcd_map;
  float scale;
  // masked calls (the two-wavefronts-per-SIMD kernels only): a bias or bool keep-mask (unit stride
  // over keys; strides in elements; bias_sl = 0 for one that does not depend on the query row)
  // and per-batch key counts
  const void* bias = nullptr;
  int64_t bias_sb = 0, bias_sh = 0, bias_sl = 0;
  int bias_kind = 0;  // 0 none, 1 float32, 2 float16, 3 bfloat16, 4 bool
  // dropout (with or without a bias): nonzero = 1 / (1 - p) (1 for p = 1), and the
  // (B, Hq, L, S) contiguous keep bytes
  float keep_scale = 0.f;
  const void* keep = nullptr;
  int64_t keep_ld = 0;  // bytes from one row of keep bytes to the next (S, or more where the caller padded the rows)
  const int32_t* kv_lens = nullptr;
  // gradient of the bias (the dQ kernel writes it): P (dP - delta) in the input dtype, one element
  // per score, unit stride over keys, rows a whole number of 8-byte words (zeros where a score
  // takes no part: above the causal diagonal, past a batch's keys)
  void* gbias = nullptr;
  int64_t gbias_sb = 0, gbias_sh = 0, gbias_sl = 0;
  // Elements per row that exist (a multiple of 8).  Below the head dim a kernel is built for, the
  // masked variants treat the rest of every Q / K / V / dO / O row as zeros and leave it out of
  // the gradients; 0 means the full width.
  int d_real = 0;
  // ... of V, dO, O and dV when they are narrower than Q and K (bwd_wide.hip only); 0 means d_real
  int dv_real = 0;
  // 1: the dQ kernel of bwd_dq_w32.hip computes delta and lse2 itself and writes them to the
  // workspace for the dK/dV kernel that follows it (bwd_delta_kernel is then not launched)
  int make_delta = 0;
  // sliding window (causal calls, masked variants without a per-score bias): query i sees keys
  // i-window+1 .. i and the first sink_keys keys; tiles that the window drops whole are skipped
  int window = 0, sink_keys = 0;
  // score functors and document ids (the functor variants of bwd_dq_w32.hip and bwd_dkdv_w32.hip)
  ScoreMod sm;
  // sorted document ids: workspace for the order in which the dK/dV kernel takes the key blocks of a
  // batch, heaviest first ((B, n_kt) ints, written by bwd_key_order_kernel ahead of it); nullptr: 0, 1, 2 ...
  int32_t* kt_order = nullptr;
  // tile skip table of a per-score bias / keep-mask for the dK/dV kernel: per (mask batch, mask head,
  // block of 128 keys) a bitmap of the 64-row query tiles with a kept score, live_t_words words each;
  // live_hm = the mask's own head extent
  const uint32_t* live_t = nullptr;
  int live_t_words = 0, live_hm = 1;
  // ... and for the dQ kernel (unless a bias gradient is asked for): per (mask batch, mask head, 64-row
  // block) a bitmap of the 32-key tiles with a kept score, live_words words each
  const uint32_t* live_tiles = nullptr;
  int live_words = 0;
  // dK/dV kernel of bwd_dkdv_w32.hip with too few key blocks for the 256 compute units (few kv heads,
  // short keys): the items of a key block (query tile x head of the group) go to `parts` workgroups,
  // each of which leaves float32 partial rows in the workspace - part_dk / part_dv, indexed
  // [part][batch][kv head][key][d_real or dv_real] - and bwd_dkdv_merge_kernel adds them up
  // (bwd_wide.hip's kernel deals out whole query tiles in the same way)
  int parts = 1;
  int parts_h = 1;  // bwd_dkdv_w32.hip: of these, shares of the group's heads (a divisor of Hq / Hkv and of parts)
  float *part_dk = nullptr, *part_dv = nullptr;
  // bwd_dkdv_w32.hip without a skip table: items per part (the same for every key block, so that a
  // block with fewer items - a causal mask, a window, a batch with fewer keys - fills fewer parts;
  // the others are neither written nor read).  0: every key block uses all `parts`, in equal shares.
  int chunk_items = 0;
  // The dQ kernel of bwd_dq_w32.hip for few query rows against many keys (cross attention over a long
  // memory): its workgroups are (batch, head, 256 rows), too few to fill the GPU, each walking every
  // key.  The key tiles are then split over blockIdx.y, dq_split_tiles tiles of 32 keys per part, the
  // parts leave float32 rows (dq_n_split, B, Hq, L, d_real) in part_dq and a second kernel adds them.
  int dq_split_tiles = 0, dq_n_split = 1;
  float* part_dq = nullptr;
  // a verdict about the bias (mask_rows.hip), read by the variants with a per-score bias in their
  // prologue: see apply_verdict
  const int32_t* verdict = nullptr;
};

// parts the dK/dV kernel of bwd_dkdv_w32.hip / of bwd_wide.hip would use for this call
int bwd_dkdv_w32_parts(const BwdM& g);
int bwd_wide_parts(const BwdM& g);
// adds up the parts' rows (g.parts, g.part_dk with d_real columns, g.part_dv with dv_real) into dK and dV
int launch_bwd_dkdv_merge(const BwdM& g, int dtype, hipStream_t s);

// dot product of eight packed elements, float32 accumulation
template <typename T>
__device__ __forceinline__ float dot8(u32x4 a, u32x4 b) {
  typedef __attribute__((ext_vector_type(8))) T v8;
  const v8 x = __builtin_bit_cast(v8, a), y = __builtin_bit_cast(v8, b);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) s = fmaf((float)x[i], (float)y[i], s);
  return s;
}


// bias element as a float (bool: 0 or -inf)
__device__ __forceinline__ float bias_value(const void* base, int64_t idx, int kind) {
  if (kind == 1) return ((const float*)base)[idx];
  if (kind == 4) return ((const uint8_t*)base)[idx] ? 0.f : -INFINITY;
  const uint32_t w = ((const uint16_t*)base)[idx];
  if (kind == 3) return __builtin_bit_cast(float, w << 16);
  return (float)__builtin_bit_cast(_Float16, (uint16_t)w);
}

// Instruction order of a tile, spelled out for the scheduler: a wavefront issues in order, and
// left alone the compiler emits a tile's matrix ops in solid runs with all of the vector work
// between them, which leaves the overlap to the other wavefront of the SIMD alone.  A pipeline
// is GROUPS groups of 1 matrix op + READS LDS reads + VALU vector instructions, in that order.
template <int GROUPS, int READS, int VALU>
__device__ __forceinline__ void pipeline() {
#pragma unroll
  for (int g = 0; g < GROUPS; ++g) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (READS > 0) __builtin_amdgcn_sched_group_barrier(0x100, READS, 0);
    if constexpr (VALU > 0) __builtin_amdgcn_sched_group_barrier(0x002, VALU, 0);
  }
}

// dK / dV with two wavefronts per SIMD (bwd_dkdv_w32.hip), head dim 64 or 128; `fits` is false
// when the tensors do not fit its 32-bit addressing and the caller must use bwd_mfma.hip
bool bwd_dkdv_w32_fits(const BwdM& g, int head_dim);
int launch_bwd_dkdv_w32(const BwdM& g, int dtype, int head_dim, hipStream_t s);
// dQ with two wavefronts per SIMD (bwd_dq_w32.hip), same convention
bool bwd_dq_w32_fits(const BwdM& g, int head_dim);
int launch_bwd_dq_w32(const BwdM& g, int dtype, int head_dim, hipStream_t s);
// head dims above 128 and D_qk != D_v (D_v <= D_qk <= 256), without masks (bwd_wide.hip)
int launch_bwd_wide(const BwdM& g, int dtype, hipStream_t s);

}  // namespace mi355
