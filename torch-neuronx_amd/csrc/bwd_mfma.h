// Parameter block shared by the MFMA backward kernels.
#pragma once

#include "mfma_common.h"

namespace mi355 {

struct BwdM {
  const void *go, *q, *k, *v, *out;
  const float* lse;
  void *gq, *gk, *gv;
  float* delta;
  int64_t go_sb, go_sh, go_sl, q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl;
  int64_t o_sb, o_sh, o_sl, gq_sb, gq_sh, gq_sl, gk_sb, gk_sh, gk_sl, gv_sb, gv_sh, gv_sl;
  int B, Hq, Hkv, L, S;
  int n_qt, n_kt;
  int causal, xcd_map;
  float scale;
};

// dK / dV for head dim 128 with two wavefronts per SIMD (bwd_dkdv_w32.hip); false when the
// tensors do not fit its 32-bit addressing and the caller must use the kernel in bwd_mfma.hip
bool bwd_dkdv_w32_fits(const BwdM& g);
int launch_bwd_dkdv_w32(const BwdM& g, int dtype, hipStream_t s);
// dQ for head dim 128 with two wavefronts per SIMD (bwd_dq_w32.hip), same convention
bool bwd_dq_w32_fits(const BwdM& g);
int launch_bwd_dq_w32(const BwdM& g, int dtype, hipStream_t s);

}  // namespace mi355
