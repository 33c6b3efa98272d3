// Parameter block and workgroup-to-tile mapping shared by the MFMA forward kernels.
#pragma once

#include "mfma_common.h"
#include "score_mod.h"

namespace mi355 {

struct FwdM {
  const void *q, *k, *v;
  void* out;
  float* lse;
  int64_t q_sb, q_sh, q_sl;
  int64_t k_sb, k_sh, k_sl;
  int64_t v_sb, v_sh, v_sl;
  int64_t o_sb, o_sh, o_sl;
  int B, Hq, Hkv, L, S;
  int n_qt;    // query tiles per head
  int causal;
  int xcd_map;  // 1: (batch, kv head) streams are pinned to XCDs
  float scale;
  // masked calls (fwd_mfma_w32.hip only): additive bias or bool keep-mask with unit stride on the
  // key dim, strides in elements (0 on broadcast dims), and per-batch key counts
  const void* bias = nullptr;
  int64_t bias_sb = 0, bias_sh = 0, bias_sl = 0;
  int bias_kind = 0;  // 0 none, 1 float32, 2 float16, 3 bfloat16, 4 bool
  // dropout (fwd_mfma_w32.hip; with or without a bias): nonzero = 1 / (1 - p)
  // (1 for p = 1), and the (B, Hq, L, S) contiguous keep bytes
  float keep_scale = 0.f;
  const void* keep = nullptr;
  int64_t keep_ld = 0;  // bytes from one row of keep bytes to the next (S, or more where the caller padded the rows)
  // Short query sequences under grouped-query attention (fwd_mfma_w32.hip; no dropout, no bias that
  // depends on the head): one workgroup serves `grouped` query heads of a kv group (all Hq / Hkv of
  // them where they fit its wavefronts; a divisor of that otherwise, with Hq / Hkv / grouped
  // workgroups per kv head): wavefront w the rows 32 * (w / grouped) .. +31 of the workgroup's head
  // w % grouped, so that a K / V tile is fetched once for all of them (decode-like calls are bound
  // by exactly that traffic).  0 = off.
  int grouped = 0;
  // ... and, when that leaves most compute units without a workgroup, the keys are split: n_split
  // workgroups per group of heads, each over split_tiles key tiles, leave their normalised output
  // (float32, (B, Hq, n_split, L, dv_real)) and log-sum-exp ((B, Hq, n_split, L)) in the workspace,
  // and fwd_split_merge_kernel combines them.  Grouped calls without a window, a sink logit, a skip
  // table or the causal flag; with a bias, head dims up to 128 only.  0 = off.
  int split_tiles = 0, n_split = 1;
  float* part_o = nullptr;   // the workspace (part_bytes bytes of it)
  float* part_lse = nullptr;
  size_t part_bytes = 0;
  const int32_t* kv_lens = nullptr;
  // Elements per row that exist (a multiple of 8).  Below the head dim a kernel is built for, the
  // masked variant treats the rest of every Q / K / V row as zeros and leaves it out of the output
  // (head dims 8 .. 56 in the 64 kernel, 72 .. 120 in the 128 kernel); 0 means the full width.
  // dv_real: the same for V and the output, which may be narrower than Q and K (192 / 128).
  int d_real = 0, dv_real = 0;
  // mask functors (masked variant without a bias only): with window > 0 (causal calls) query i sees
  // keys i-window+1 .. i and the first sink_keys keys; sink_logit (B, Hq) is one more logit per row
  // that joins the softmax and carries no value
  int window = 0, sink_keys = 0;
  const float* sink_logit = nullptr;
  int n_sinks = 1;  // logits per (batch, head) behind sink_logit
  // score functors and document ids (fwd_mfma_w32.hip, the functor variant: no bias)
  ScoreMod sm;
  // tile skip table of the bias / keep-mask (variant with a bias, no causal flag): per (mask batch,
  // mask head, 64-row block) a bitmap of the key tiles with a kept score, live_words words each;
  // live_hm = the mask's own head extent
  const uint32_t* live_tiles = nullptr;
  int live_words = 0, live_hm = 1;
  // a verdict about the bias (mask_rows.hip), read by the variants with a per-score bias in their
  // prologue: see apply_verdict
  const int32_t* verdict = nullptr;
};

// Decode blockIdx.x -> (batch, query head, query tile).  Tiles are issued heaviest first
// (for causal attention the last query tile walks the most keys).  With xcd_map the eight
// XCDs (blocks are dealt round-robin, block i -> XCD i % 8) each serve a fixed subset of
// (batch, kv head) streams, so the K/V of a stream stay in one XCD's L2.
__device__ __forceinline__ void decode_block(const FwdM& p, int& b, int& h, int& qt) {
  const int bid = blockIdx.x;
  const int rep = p.Hq / p.Hkv;
  if (p.xcd_map) {
    const int streams = p.B * p.Hkv;  // multiple of 8
    const int per_xcd = streams / 8;
    const int xcd = bid & 7;
    int r = bid >> 3;  // index within this XCD: [qt desc][stream in xcd][head in group]
    const int hg = r % rep;
    r /= rep;
    const int sl = r % per_xcd;
    r /= per_xcd;
    qt = p.n_qt - 1 - r;
    const int stream = sl * 8 + xcd;
    b = stream / p.Hkv;
    h = (stream % p.Hkv) * rep + hg;
  } else {
    const int heads = p.B * p.Hq;
    qt = p.n_qt - 1 - bid / heads;
    const int bh = bid % heads;
    b = bh / p.Hq;
    h = bh % p.Hq;
  }
}


// head_dim 64, 128 or 256: the width the kernel is built for (g.d_real: the width of the data);
// waves = 4 or 8 wavefronts (128 or 256 query rows) per workgroup, 4 only at head dim 256
int launch_fwd_mfma_w32(const FwdM& g, int dtype, int head_dim, int waves, hipStream_t s);
// bytes of workspace with which that launch would split the keys of the call (0: it would not)
size_t fwd_w32_workspace(const FwdM& g, int head_dim, int waves);

}  // namespace mi355
