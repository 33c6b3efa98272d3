// Flash-attention backward for gfx950 on the 32x32x16 bf16/f16 MFMA.  Three kernels, no
// atomics, deterministic; P is recomputed from the saved log-sum-exp:
//
//   bwd_delta_kernel   delta_i = sum_d dO_id O_id  (float32).  This is the whole row term of
//                      torch_neuronx/_sdpa_math.py:160-163: its two P-dependent parts cancel.
//                      (Not launched when the dQ kernel of bwd_dq_w32.hip serves the call: that
//                      one goes first and leaves the row terms behind itself.)
//   bwd_dkdv_kernel    one workgroup per 128 keys of a (batch, kv head); loops over the query
//                      heads of the group (the GQA sum of decompositions.py:2595-2598 happens
//                      in registers) and over 64-row query tiles:
//                        S = Q K^T, dP = dO V^T      (A = Q / dO tile from LDS, B = K / V in registers)
//                        P = exp2(c S - lse), dS = P (dP - delta)
//                        dV^T += dO^T P, dK^T += Q^T dS  (A = transposed tile from LDS, B = P / dS
//                                                         packed straight from the accumulators)
//   bwd_dq_kernel      one workgroup per 128 query rows; loops over 64-key tiles:
//                        S^T = K Q^T, dP^T = V dO^T, dS^T = P^T (dP^T - delta), dQ^T += K^T dS^T
//
// In both main kernels the softmax statistics a lane needs are either per-lane scalars or four
// consecutive floats, and no probability ever goes through LDS.  Row-major tiles are XOR
// swizzled, transposed tiles are written with byte permutes (see mfma_common.h).  Math follows
// _sdpa_math.py:98-176: everything accumulates in float32, rows with lse = -inf give zero
// gradients, scale multiplies dQ and dK once at the end.
#include <type_traits>

#include "bwd_mfma.h"

namespace mi355 {
namespace {

template <typename T, int D>
__global__ __launch_bounds__(256) void bwd_delta_kernel(BwdM p) {
  constexpr int LPR = D / 8, RPB = 256 / LPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LPR;
  const int sub = threadIdx.x % LPR;
  const int64_t rows = (int64_t)p.B * p.Hq * p.L;
  float s = 0.f;
  if (row < rows) {
    const int i = (int)(row % p.L), h = (int)((row / p.L) % p.Hq), b = (int)(row / ((int64_t)p.L * p.Hq));
    const uint16_t* g = (const uint16_t*)p.go + b * p.go_sb + h * p.go_sh + (int64_t)i * p.go_sl + sub * 8;
    const uint16_t* o = (const uint16_t*)p.out + b * p.o_sb + h * p.o_sh + (int64_t)i * p.o_sl + sub * 8;
    if (sub * 8 < p.d_real) s = dot8<T>(*(const u32x4*)g, *(const u32x4*)o);
  }
#pragma unroll
  for (int off = LPR / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  if (row < rows && sub == 0) {
    p.delta[row] = s;
    // (+inf turns exp2(x - lse) into 0 for rows without a live key)
    const float l = p.lse[row];
    p.lse2[row] = l != -INFINITY ? l * kLog2eF : INFINITY;
  }
}

// ================================================================================================
template <typename T, int D>
__global__ __launch_bounds__(256, 1) void bwd_dkdv_kernel(BwdM p) {
  constexpr int BQ = 64, BK = 128;
  constexpr int KS = D / 16, DB = D / 32, NCH = D / 8;
  constexpr int TP = BQ + 8;            // pitch of the transposed tiles (elements)
  constexpr int U = 16 * NCH;           // 4-row x 8-d units per tile
  constexpr int NU = (2 * U) / 256;     // units per thread over the Q and dO tiles
  __shared__ __attribute__((aligned(16))) uint16_t q_rm[2][BQ * D];
  __shared__ __attribute__((aligned(16))) uint16_t do_rm[2][BQ * D];
  __shared__ __attribute__((aligned(16))) uint16_t q_t[2][D * TP];
  __shared__ __attribute__((aligned(16))) uint16_t do_t[2][D * TP];
  __shared__ __attribute__((aligned(16))) float lse_s[2][BQ];
  __shared__ __attribute__((aligned(16))) float dl_s[2][BQ];

  const int streams = p.B * p.Hkv;
  const int kt = blockIdx.x / streams;  // low key tiles see the most queries under a causal mask: first
  const int st = blockIdx.x % streams;
  const int b = st / p.Hkv, hk = st % p.Hkv;
  const int rep = p.Hq / p.Hkv;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int col = lane & 31, half = lane >> 5;
  const int k0 = kt * BK, kw0 = k0 + wave * 32;
  const int key = kw0 + col;

  // K and V fragments of this lane's key: B operands of S = Q K^T and dP = dO V^T
  u32x4 kf[KS], vf[KS];
  {
    const int kc = min(key, p.S - 1);
    const uint16_t* kr = (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh + (int64_t)kc * p.k_sl + half * 8;
    const uint16_t* vr = (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh + (int64_t)kc * p.v_sl + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kf[ks] = *(const u32x4*)(kr + ks * 16), vf[ks] = *(const u32x4*)(vr + ks * 16);
  }

  const int nqs = (p.L + BQ - 1) / BQ;
  const int qs_begin = p.causal ? min(k0 / BQ, nqs) : 0;
  const int per_head = nqs - qs_begin;
  const int n_items = rep * per_head;

  u32x4 stage[NU][4];
  float lse_r = 0.f, dl_r = 0.f;
  auto item_head = [&](int it) { return hk * rep + it / per_head; };
  auto item_q0 = [&](int it) { return (qs_begin + it % per_head) * BQ; };
  auto load_item = [&](int it) {
    const int h = item_head(it), q0 = item_q0(it);
#pragma unroll
    for (int n = 0; n < NU; ++n) {
      const int u = tid + n * 256, tile = u / U, uu = u % U, g = uu & 15, dc = uu >> 4;
      const uint16_t* base = tile ? (const uint16_t*)p.go + b * p.go_sb + h * p.go_sh
                                  : (const uint16_t*)p.q + b * p.q_sb + h * p.q_sh;
      const int64_t sl = tile ? p.go_sl : p.q_sl;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = min(q0 + 4 * g + i, p.L - 1);
        stage[n][i] = *(const u32x4*)(base + (int64_t)r * sl + dc * 8);
      }
    }
    if (tid < BQ) {
      const int qi = q0 + tid;
      const int64_t idx = ((int64_t)b * p.Hq + h) * p.L + min(qi, p.L - 1);
      const float l = p.lse[idx];
      // +inf turns exp2(x - lse) into 0 for rows past L and for rows without a live key
      lse_r = (qi < p.L && l != -INFINITY) ? l * kLog2eF : INFINITY;
      dl_r = qi < p.L ? p.delta[idx] : 0.f;
    }
  };
  auto store_item = [&](int buf) {
#pragma unroll
    for (int n = 0; n < NU; ++n) {
      const int u = tid + n * 256, tile = u / U, uu = u % U, g = uu & 15, dc = uu >> 4;
      uint16_t* rm = tile ? do_rm[buf] : q_rm[buf];
      uint16_t* tt = tile ? do_t[buf] : q_t[buf];
#pragma unroll
      for (int i = 0; i < 4; ++i) *(u32x4*)(&rm[rm_off<D>(4 * g + i, dc)]) = stage[n][i];
      tr_store<TP>(tt, stage[n], g, dc * 8);
    }
    if (tid < BQ) lse_s[buf][tid] = lse_r, dl_s[buf][tid] = dl_r;
  };

  f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) zero(dkacc[i]), zero(dvacc[i]);
  const float c = p.scale * kLog2eF;

  if (n_items > 0) {
    load_item(0);
    store_item(0);
    __syncthreads();
    if (n_items > 1) load_item(1);
  }
  for (int it = 0; it < n_items; ++it) {
    const int buf = it & 1;
    const int q0 = item_q0(it);
    // register classes, stated once per item: the dK / dV accumulators are touched by matrix ops
    // only and live in accumulation registers; the K / V fragments feed every matrix op as a
    // source operand and must stay in ordinary vector registers
#pragma unroll
    for (int i = 0; i < DB; ++i) {
      asm volatile("" : "+a"(dkacc[i]));
      asm volatile("" : "+a"(dvacc[i]));
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      asm volatile("" : "+v"(kf[ks]));
      asm volatile("" : "+v"(vf[ks]));
    }
    const bool active = !p.causal || q0 + BQ - 1 >= kw0;
    if (active) {
      const bool edge = (p.causal && q0 < kw0 + 31) || (kw0 + 31 >= p.S);
      uint32_t pP[2][8], pS[2][8];
      // A operands stream from LDS through a small register ring, kRing reads ahead of the
      // matrix op that consumes them: with one wavefront per SIMD nothing else hides LDS latency.
      constexpr int kRing = 8;
      u32x4 ring[kRing];
      // S / dP operand i of query-row block mq: (i even) Q rows for S, (i odd) dO rows for dP
      auto read_rows = [&](int mq, int i) -> u32x4 {
        const uint16_t* t = (i & 1) ? do_rm[buf] : q_rm[buf];
        return *(const u32x4*)(&t[rm_off<D>(mq * 32 + col, 2 * (i >> 1) + half)]);
      };
      // dV / dK operand i: step ks = i / (2 DB), d block db, (i even) dO^T for dV, (i odd) Q^T for dK
      auto read_cols = [&](int i) -> u32x4 {
        const uint16_t* t = (i & 1) ? q_t[buf] : do_t[buf];
        const int ks = i / (2 * DB), db = (i >> 1) % DB;
        return *(const u32x4*)(&t[(db * 32 + col) * TP + ks * 16 + half * 8]);
      };
      // P = exp2(c S - lse), dS = P (dP - delta) for 32 query rows x this lane's key
      auto softmax = [&](int mq, const f32x16& sacc, const f32x16& dpacc, auto edge_c) {
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const f32x4 l4 = *(const f32x4*)(&lse_s[buf][mq * 32 + r4 * 8 + half * 4]);
          const f32x4 d4 = *(const f32x4*)(&dl_s[buf][mq * 32 + r4 * 8 + half * 4]);
          float pr[4], ds[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int r = r4 * 4 + e;
            pr[e] = __builtin_amdgcn_exp2f(fmaf(sacc[r], c, -l4[e]));
            if (decltype(edge_c)::value) {
              const int qi = q0 + mq * 32 + r4 * 8 + half * 4 + e;
              pr[e] = ((p.causal && key > qi) || key >= p.S) ? 0.f : pr[e];
            }
            ds[e] = pr[e] * (dpacc[r] - d4[e]);
          }
          pP[mq][r4 * 2] = Mma<T>::pack(pr[0], pr[1]), pP[mq][r4 * 2 + 1] = Mma<T>::pack(pr[2], pr[3]);
          pS[mq][r4 * 2] = Mma<T>::pack(ds[0], ds[1]), pS[mq][r4 * 2 + 1] = Mma<T>::pack(ds[2], ds[3]);
        }
      };
#pragma unroll
      for (int i = 0; i < kRing; ++i) ring[i] = read_rows(0, i);
#pragma unroll
      for (int mq = 0; mq < 2; ++mq) {
        f32x16 sacc, dpacc;  // written by the matrix ops below into ordinary vector registers
#pragma unroll
        for (int i = 0; i < 2 * KS; ++i) {
          if (i & 1) {
            if (i == 1) MmaV<T>::first(dpacc, ring[i % kRing], vf[i >> 1]);
            else MmaV<T>::next(dpacc, ring[i % kRing], vf[i >> 1]);
          } else {
            if (i == 0) MmaV<T>::first(sacc, ring[i % kRing], kf[i >> 1]);
            else MmaV<T>::next(sacc, ring[i % kRing], kf[i >> 1]);
          }
          if (i + kRing < 2 * KS) ring[i % kRing] = read_rows(mq, i + kRing);
          else if (mq == 0) ring[i % kRing] = read_rows(1, i + kRing - 2 * KS);
          else ring[i % kRing] = read_cols(i + kRing - 2 * KS);
        }
        mfma_to_valu_gap(sacc, dpacc);
        if (edge) softmax(mq, sacc, dpacc, std::true_type{});
        else softmax(mq, sacc, dpacc, std::false_type{});
      }
      // dV^T += dO^T P, dK^T += Q^T dS
#pragma unroll
      for (int i = 0; i < 8 * DB; ++i) {
        const int ks = i / (2 * DB), db = (i >> 1) % DB, mq = ks >> 1, r0 = (ks & 1) * 4;
        if (i & 1) {
          const u32x4 bS = {pS[mq][r0], pS[mq][r0 + 1], pS[mq][r0 + 2], pS[mq][r0 + 3]};
          dkacc[db] = Mma<T>::run(ring[i % kRing], bS, dkacc[db]);
        } else {
          const u32x4 bP = {pP[mq][r0], pP[mq][r0 + 1], pP[mq][r0 + 2], pP[mq][r0 + 3]};
          dvacc[db] = Mma<T>::run(ring[i % kRing], bP, dvacc[db]);
        }
        if (i + kRing < 8 * DB) ring[i % kRing] = read_cols(i + kRing);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (it + 1 < n_items) store_item(buf ^ 1);
    __syncthreads();
    if (it + 2 < n_items) load_item(it + 2);
  }

  if (key < p.S) {
    uint16_t* gk = (uint16_t*)p.gk + b * p.gk_sb + hk * p.gk_sh + (int64_t)key * p.gk_sl;
    uint16_t* gv = (uint16_t*)p.gv + b * p.gv_sb + hk * p.gv_sh + (int64_t)key * p.gv_sl;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        w[0] = Mma<T>::pack(dkacc[db][g * 4] * p.scale, dkacc[db][g * 4 + 1] * p.scale);
        w[1] = Mma<T>::pack(dkacc[db][g * 4 + 2] * p.scale, dkacc[db][g * 4 + 3] * p.scale);
        *(u32x2*)(gk + db * 32 + g * 8 + half * 4) = w;
        w[0] = Mma<T>::pack(dvacc[db][g * 4], dvacc[db][g * 4 + 1]);
        w[1] = Mma<T>::pack(dvacc[db][g * 4 + 2], dvacc[db][g * 4 + 3]);
        *(u32x2*)(gv + db * 32 + g * 8 + half * 4) = w;
      }
  }
}

// ================================================================================================
// NB = query-row blocks of 32 per wavefront.  NB = 2 (256 rows per workgroup) lets every K / V /
// K^T fragment read from LDS feed two matrix ops, which halves the LDS bytes per flop, the bound of
// this kernel; the Q and dO fragments of 64 rows (128 registers) are then parked in accumulation
// registers, which the score matrix ops can read directly as their B operand.
template <typename T, int D, int NB>
__global__ __launch_bounds__(256, 1) void bwd_dq_kernel(BwdM p) {
  constexpr int BM = 128 * NB, BN = 64;
  constexpr int KS = D / 16, DB = D / 32, NCH = D / 8;
  constexpr int TP = BN + 8;
  constexpr int U = 16 * NCH;               // K units (4 keys x 8 d)
  constexpr int VLD = (BN * NCH) / 256;     // V chunks per thread
  __shared__ __attribute__((aligned(16))) uint16_t k_rm[2][BN * D];
  __shared__ __attribute__((aligned(16))) uint16_t v_rm[2][BN * D];
  __shared__ __attribute__((aligned(16))) uint16_t k_t[2][D * TP];

  int b, h, qt;
  {
    const int bid = blockIdx.x, rep = p.Hq / p.Hkv;
    const int n_qt = (p.L + BM - 1) / BM;
    if (p.xcd_map) {
      const int per_xcd = (p.B * p.Hkv) / 8, xcd = bid & 7;
      int r = bid >> 3;
      const int hg = r % rep;
      r /= rep;
      const int sl = r % per_xcd;
      r /= per_xcd;
      qt = n_qt - 1 - r;
      const int stream = sl * 8 + xcd;
      b = stream / p.Hkv, h = (stream % p.Hkv) * rep + hg;
    } else {
      const int heads = p.B * p.Hq;
      qt = n_qt - 1 - bid / heads;
      b = (bid % heads) / p.Hq, h = (bid % heads) % p.Hq;
    }
  }
  const int hk = h / (p.Hq / p.Hkv);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int col = lane & 31, half = lane >> 5;
  const int q0 = qt * BM, qw0 = q0 + wave * 32 * NB;
  int qrow[NB], qc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) qrow[nb] = qw0 + 32 * nb + col, qc[nb] = min(qrow[nb], p.L - 1);

  u32x4 qf[NB][KS], dof[NB][KS];
  float lse2[NB], dl[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const uint16_t* qr = (const uint16_t*)p.q + b * p.q_sb + h * p.q_sh + (int64_t)qc[nb] * p.q_sl + half * 8;
    const uint16_t* gr = (const uint16_t*)p.go + b * p.go_sb + h * p.go_sh + (int64_t)qc[nb] * p.go_sl + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[nb][ks] = *(const u32x4*)(qr + ks * 16), dof[nb][ks] = *(const u32x4*)(gr + ks * 16);
    const int64_t idx = ((int64_t)b * p.Hq + h) * p.L + qc[nb];
    const float l = p.lse[idx];
    lse2[nb] = (qrow[nb] < p.L && l != -INFINITY) ? l * kLog2eF : INFINITY;
    dl[nb] = p.delta[idx];
  }

  int nt = (p.S + BN - 1) / BN;
  if (p.causal) nt = min(nt, (min(q0 + BM, p.L) - 1) / BN + 1);

  const uint16_t* kp = (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh;
  const uint16_t* vp = (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh;
  u32x4 kst[4], vst[VLD];
  const int k_g = tid & 15, k_dc = tid >> 4;
  const bool k_loader = tid < U;
  const int v_ch = tid % NCH, v_r0 = tid / NCH;
  auto load_tile = [&](int t) {
    const int kv0 = t * BN;
    if (k_loader) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        kst[i] = *(const u32x4*)(kp + (int64_t)min(kv0 + 4 * k_g + i, p.S - 1) * p.k_sl + k_dc * 8);
    }
#pragma unroll
    for (int i = 0; i < VLD; ++i)
      vst[i] = *(const u32x4*)(vp + (int64_t)min(kv0 + v_r0 + i * (256 / NCH), p.S - 1) * p.v_sl + v_ch * 8);
  };
  auto store_tile = [&](int buf) {
    if (k_loader) {
#pragma unroll
      for (int i = 0; i < 4; ++i) *(u32x4*)(&k_rm[buf][rm_off<D>(4 * k_g + i, k_dc)]) = kst[i];
      tr_store<TP>(k_t[buf], kst, k_g, k_dc * 8);
    }
#pragma unroll
    for (int i = 0; i < VLD; ++i) *(u32x4*)(&v_rm[buf][rm_off<D>(v_r0 + i * (256 / NCH), v_ch)]) = vst[i];
  };

  f32x16 dqacc[DB][NB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) zero(dqacc[i][nb]);
  const float c = p.scale * kLog2eF;

  load_tile(0);
  store_tile(0);
  __syncthreads();
  if (nt > 1) load_tile(1);
  for (int t = 0; t < nt; ++t) {
    const int buf = t & 1, kv0 = t * BN;
    const bool active = !p.causal || kv0 <= qw0 + 32 * NB - 1;
    // register classes, stated once per tile (see bwd_dkdv_kernel)
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) asm volatile("" : "+a"(dqacc[i][nb]));
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (NB == 2) {
          asm volatile("" : "+a"(qf[nb][ks]));
          asm volatile("" : "+a"(dof[nb][ks]));
        } else {
          asm volatile("" : "+v"(qf[nb][ks]));
          asm volatile("" : "+v"(dof[nb][ks]));
        }
      }
    if (active) {
      const bool edge = (p.causal && kv0 + BN - 1 > qw0) || (kv0 + BN > p.S);
      uint32_t pS[NB][2][8];
      constexpr int kRing = 8;
      u32x4 ring[kRing];
      // S^T / dP^T operand i of key block mb: (i even) K rows, (i odd) V rows
      auto read_rows = [&](int mb, int i) -> u32x4 {
        const uint16_t* t_ = (i & 1) ? v_rm[buf] : k_rm[buf];
        return *(const u32x4*)(&t_[rm_off<D>(mb * 32 + col, 2 * (i >> 1) + half)]);
      };
      // dQ^T operand i: step ks = i / DB, d block db = i % DB of K^T
      auto read_cols = [&](int i) -> u32x4 {
        return *(const u32x4*)(&k_t[buf][((i % DB) * 32 + col) * TP + (i / DB) * 16 + half * 8]);
      };
      auto softmax = [&](int nb, int mb, const f32x16& sacc, const f32x16& dpacc, auto edge_c) {
        const int lim = p.causal ? min(qrow[nb], p.S - 1) : p.S - 1;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          float ds[2];
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            float pr = __builtin_amdgcn_exp2f(fmaf(sacc[r + e], c, -lse2[nb]));
            if (decltype(edge_c)::value) {
              const int kv = kv0 + mb * 32 + ((r + e) >> 2) * 8 + half * 4 + ((r + e) & 3);
              pr = kv > lim ? 0.f : pr;
            }
            ds[e] = pr * (dpacc[r + e] - dl[nb]);
          }
          pS[nb][mb][r >> 1] = Mma<T>::pack(ds[0], ds[1]);
        }
      };
#pragma unroll
      for (int i = 0; i < kRing; ++i) ring[i] = read_rows(0, i);
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        f32x16 sacc[NB], dpacc[NB];  // written by the matrix ops below into ordinary vector registers
#pragma unroll
        for (int i = 0; i < 2 * KS; ++i) {
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            f32x16& acc = (i & 1) ? dpacc[nb] : sacc[nb];
            const u32x4& frag = (i & 1) ? dof[nb][i >> 1] : qf[nb][i >> 1];
            if (NB == 2) {
              if (i < 2) MmaV<T>::first_ba(acc, ring[i % kRing], frag);
              else MmaV<T>::next_ba(acc, ring[i % kRing], frag);
            } else {
              if (i < 2) MmaV<T>::first(acc, ring[i % kRing], frag);
              else MmaV<T>::next(acc, ring[i % kRing], frag);
            }
          }
          if (i + kRing < 2 * KS) ring[i % kRing] = read_rows(mb, i + kRing);
          else if (mb == 0) ring[i % kRing] = read_rows(1, i + kRing - 2 * KS);
          else ring[i % kRing] = read_cols(i + kRing - 2 * KS);
        }
        if constexpr (NB == 2) mfma_to_valu_gap(sacc[0], dpacc[0], sacc[NB - 1], dpacc[NB - 1]);
        else mfma_to_valu_gap(sacc[0], dpacc[0]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          if (edge) softmax(nb, mb, sacc[nb], dpacc[nb], std::true_type{});
          else softmax(nb, mb, sacc[nb], dpacc[nb], std::false_type{});
        }
      }
#pragma unroll
      for (int i = 0; i < 4 * DB; ++i) {
        const int ks = i / DB, db = i % DB, mb = ks >> 1, r0 = (ks & 1) * 4;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const u32x4 bS = {pS[nb][mb][r0], pS[nb][mb][r0 + 1], pS[nb][mb][r0 + 2], pS[nb][mb][r0 + 3]};
          dqacc[db][nb] = Mma<T>::run(ring[i % kRing], bS, dqacc[db][nb]);
        }
        if (i + kRing < 4 * DB) ring[i % kRing] = read_cols(i + kRing);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (t + 1 < nt) store_tile(buf ^ 1);
    __syncthreads();
    if (t + 2 < nt) load_tile(t + 2);
  }

#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    if (qrow[nb] < p.L) {
      uint16_t* gq = (uint16_t*)p.gq + b * p.gq_sb + h * p.gq_sh + (int64_t)qrow[nb] * p.gq_sl;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          u32x2 w;
          w[0] = Mma<T>::pack(dqacc[db][nb][g * 4] * p.scale, dqacc[db][nb][g * 4 + 1] * p.scale);
          w[1] = Mma<T>::pack(dqacc[db][nb][g * 4 + 2] * p.scale, dqacc[db][nb][g * 4 + 3] * p.scale);
          *(u32x2*)(gq + db * 32 + g * 8 + half * 4) = w;
        }
    }
  }
}

template <typename T, int D>
int launch_td(const BwdM& g, hipStream_t s) {
  const int64_t rows = (int64_t)g.B * g.Hq * g.L;
  constexpr int RPB = 256 / (D / 8);
  // dQ: 256-row workgroups when D = 128 and there is at least one for every compute unit
  const int64_t wg256 = (int64_t)g.B * g.Hq * ((g.L + 255) / 256);
  const bool dq_w32 = (wg256 >= 256 || g.bias_kind || g.keep_scale != 0.f || g.kv_lens || g.gbias || g.d_real != D || g.window > 0 || g.sm.any || g.dq_split_tiles) && bwd_dq_w32_fits(g, D);  // (a masked call has no other kernel)
  int rc;
  if (dq_w32) {
    // that kernel holds every row of dO in registers anyway: it goes first and leaves the row
    // terms (delta, log2-domain LSE) behind for the dK/dV kernel, which saves the pass over dO
    // and O of bwd_delta_kernel
    BwdM g2 = g;
    g2.make_delta = 1;
    rc = launch_bwd_dq_w32(g2, std::is_same<T, bf16_t>::value ? MI355_SDPA_BF16 : MI355_SDPA_F16, D, s);
  } else {
    hipLaunchKernelGGL((bwd_delta_kernel<T, D>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, s, g);
    rc = check_launch("bwd_delta_kernel");
  }
  if (rc) return rc;
  if (bwd_dkdv_w32_fits(g, D)) {
    rc = launch_bwd_dkdv_w32(g, std::is_same<T, bf16_t>::value ? MI355_SDPA_BF16 : MI355_SDPA_F16, D, s);
  } else {
    hipLaunchKernelGGL((bwd_dkdv_kernel<T, D>), dim3((unsigned)(g.B * g.Hkv * g.n_kt)), dim3(256), 0, s, g);
    rc = check_launch("bwd_dkdv_kernel");
  }
  if (rc || dq_w32) return rc;
  if (D == 128 && wg256 >= 256) {
    hipLaunchKernelGGL((bwd_dq_kernel<T, D, D == 128 ? 2 : 1>), dim3((unsigned)wg256), dim3(256), 0, s, g);
  } else {
    hipLaunchKernelGGL((bwd_dq_kernel<T, D, 1>), dim3((unsigned)(g.B * g.Hq * g.n_qt)), dim3(256), 0, s, g);
  }
  return check_launch("bwd_dq_kernel");
}

}  // namespace

static void fill(BwdM& g, const mi355_sdpa_bwd_params& p) {
  g.go = p.grad_out.data, g.q = p.q.data, g.k = p.k.data, g.v = p.v.data, g.out = p.out.data;
  g.lse = p.lse, g.gq = p.grad_q.data, g.gk = p.grad_k.data, g.gv = p.grad_v.data;
  g.delta = (float*)p.workspace;
  g.lse2 = g.delta + p.q.size[0] * p.q.size[1] * p.q.size[2];
#define SET3(dst, src) g.dst##_sb = p.src.stride[0], g.dst##_sh = p.src.stride[1], g.dst##_sl = p.src.stride[2]
  SET3(go, grad_out);
  SET3(q, q);
  SET3(k, k);
  SET3(v, v);
  SET3(o, out);
  SET3(gq, grad_q);
  SET3(gk, grad_k);
  SET3(gv, grad_v);
#undef SET3
  g.B = (int)p.q.size[0], g.Hq = (int)p.q.size[1], g.Hkv = (int)p.k.size[1];
  g.L = (int)p.q.size[2], g.S = (int)p.k.size[2];
  g.n_qt = (g.L + 127) / 128, g.n_kt = (g.S + 127) / 128;
  g.causal = p.is_causal, g.scale = p.scale;
  g.xcd_map = ((g.B * g.Hkv) % 8 == 0) ? 1 : 0;
  g.kv_lens = p.kv_lens;
  g.d_real = (int)p.q.size[3], g.dv_real = (int)p.v.size[3];
  g.window = p.mask.window, g.sink_keys = p.mask.sink_keys;
  g.sm = score_mod_of(p.mask);
  if (p.grad_bias.data) {
    g.gbias = p.grad_bias.data;
    g.gbias_sb = p.grad_bias.stride[0], g.gbias_sh = p.grad_bias.stride[1], g.gbias_sl = p.grad_bias.stride[2];
  }
  if (p.bias.data) {
    g.bias = p.bias.data;
    g.bias_sb = p.bias.stride[0], g.bias_sh = p.bias.stride[1];
    g.bias_sl = p.q.size[2] > 1 ? p.bias.stride[2] : 0;
    g.bias_kind = p.bias_dtype == MI355_SDPA_F32 ? 1 : p.bias_dtype == MI355_SDPA_F16 ? 2 : p.bias_dtype == MI355_SDPA_BF16 ? 3 : 4;
    const int words_t = ((g.L + 63) / 64 + 31) / 32;
    if (p.mask.live_tiles_t && !p.is_causal && g.bias_sl != 0 && g.S <= 32768 && (g.Hq / g.Hkv) * words_t <= 256 && p.dropout_p == 0.f) {
      g.live_t = p.mask.live_tiles_t;
      g.live_t_words = words_t, g.live_hm = live_extent(p.bias, 1);
    }
    if (p.mask.live_tiles && !p.is_causal && g.bias_sl != 0 && g.S <= 32768 && !p.grad_bias.data && p.dropout_p == 0.f) {
      g.live_tiles = p.mask.live_tiles;
      g.live_words = ((g.S + 31) / 32 + 31) / 32, g.live_hm = live_extent(p.bias, 1);
    }
  }
  // (a verdict about the bias is for calls in which nothing else shapes the scores; dropout may come on top)
  if (p.mask.mask_verdict && g.bias_kind && p.q.size[2] > 1 && !p.is_causal && !p.kv_lens && !g.live_t &&
      !g.live_tiles && !g.gbias && g.window == 0 && !g.sm.any && p.q.size[3] <= 128 && p.v.size[3] == p.q.size[3])
    g.verdict = p.mask.mask_verdict;
  if (p.dropout_p > 0.f) {  // (B, Hq, L, S) contiguous bytes, 1 = keep
    g.keep = p.dropout_keep;
    g.keep_ld = (p.dropout_keep_ld > 0 ? p.dropout_keep_ld : p.k.size[2]);
    g.keep_scale = p.dropout_p < 1.f ? 1.f / (1.f - p.dropout_p) : 1.f;
  }
}

bool bwd_mfma_supported(const mi355_sdpa_bwd_params& p, const char** why) {
  *why = "";
  const int64_t E = p.q.size[3], Dv = p.v.size[3];
  if (p.dtype != MI355_SDPA_BF16 && p.dtype != MI355_SDPA_F16) return *why = "dtype is not bf16/f16", false;
  if (E < 8 || E > 256 || E % 8 != 0 || Dv < 8 || Dv > E || Dv % 8 != 0)
    return *why = "head dims are not multiples of 8 up to 256 with D_v <= D_qk", false;
  // head dims above 128 and D_qk != D_v: the kernels of bwd_wide.hip, which take key counts and a
  // bias / keep-mask, but no bias gradient and no window
  const bool wide = E > 128 || Dv != E;
  const bool smod = score_mod_of(p.mask).any;
  if (smod && (p.bias.data || p.grad_bias.data || p.dropout_p > 0.f))
    return *why = "score functor together with attn_bias or dropout", false;
  const bool padded = E != 64 && E != 128;  // served by the next wider kernels' masked variants
  if (p.grad_bias.data) {  // written by the dQ kernel four keys (8 bytes) at a time
    const int64_t S = p.k.size[2];
    if (!p.bias.data) return *why = "grad_attn_bias without attn_bias", false;
    // (a row stride of at least S rounded up to four says that every row - the last one of the tensor
    // included - has room for whole words: the words that cross the end of a row then land in its padding)
    const bool room = S % 4 == 0 || (p.q.size[2] > 1 && p.grad_bias.stride[2] >= ((S + 3) & ~(int64_t)3));
    if (!room || (S > 1 && p.grad_bias.stride[3] != 1) || ((uintptr_t)p.grad_bias.data & 7) != 0)
      return *why = "grad_attn_bias rows are not whole 8-byte words", false;
    for (int i = 0; i < 3; ++i)
      if (p.grad_bias.size[i] > 1 && (p.grad_bias.stride[i] % 4) != 0) return *why = "grad_attn_bias stride not 8-byte aligned", false;
  }
  // masked calls: a bias / bool keep-mask whose rows can be read four keys at a time and that one
  // (batch, head) addresses with 32 bits, and per-batch key counts, in the kernels with 32-bit
  // addressing
  if (p.bias.data) {
    const int esz = p.bias_dtype == MI355_SDPA_F32 ? 4 : p.bias_dtype == MI355_SDPA_BOOL ? 1
                    : (p.bias_dtype == MI355_SDPA_F16 || p.bias_dtype == MI355_SDPA_BF16) ? 2 : 0;
    if (!esz) return *why = "attn_bias dtype", false;
    const int64_t S = p.k.size[2];
    const int gran = 4 / esz;
    if (S > 1 && p.bias.stride[3] != 1) return *why = "attn_bias keys are not unit-stride", false;
    if (((uintptr_t)p.bias.data & 3) != 0 || S % gran != 0) return *why = "attn_bias not dword aligned", false;
    for (int i = 0; i < 3; ++i)
      if (p.bias.size[i] > 1 && (p.bias.stride[i] % gran) != 0) return *why = "attn_bias stride not dword aligned", false;
    if (p.q.size[2] > 1 && p.bias.stride[2] < 0) return *why = "attn_bias row stride is negative", false;
    if (((p.q.size[2] + 64) * (p.q.size[2] > 1 ? p.bias.stride[2] : 0) + S + 64) * esz >= (1ll << 31))
      return *why = "attn_bias rows beyond 32-bit offsets", false;
  }
  if (p.dropout_p > 0.f) {
    // the keep-mask takes a bool bias's way into the kernels (one dword = four keys of a row)
    const int64_t S = p.k.size[2];
    if (p.mask.window > 0) return *why = "dropout together with a window functor", false;
    if (!p.dropout_keep || ((uintptr_t)p.dropout_keep & 3) != 0 || (p.dropout_keep_ld > 0 ? p.dropout_keep_ld : p.k.size[2]) % 4 != 0) return *why = "dropout keep-mask rows do not start on dwords", false;
    if ((p.q.size[2] + 64) * S + S + 64 >= (1ll << 31)) return *why = "dropout keep-mask rows beyond 32-bit offsets", false;
  }
  if (!(p.scale > 0.f)) return *why = "scale <= 0", false;
  if (p.q.size[2] < 1 || p.k.size[2] < 1) return *why = "empty sequence", false;
  if (p.mask.window > 0 && p.bias.data) return *why = "window functor together with attn_bias", false;
  const mi355_sdpa_tensor* ts[8] = {&p.grad_out, &p.q, &p.k, &p.v, &p.out, &p.grad_q, &p.grad_k, &p.grad_v};
  for (const mi355_sdpa_tensor* t : ts) {
    if (t->stride[3] != 1) return *why = "head dim is not unit-stride", false;
    if (((uintptr_t)t->data & 15) != 0) return *why = "pointer not 16-byte aligned", false;
    for (int i = 0; i < 3; ++i)
      if (t->size[i] > 1 && (t->stride[i] % 8) != 0) return *why = "stride not a multiple of 8 elements", false;
  }
  if ((int64_t)p.q.size[0] * p.q.size[1] * ((p.q.size[2] + 127) / 128) > 0x7fffffff) return *why = "too many tiles", false;
  if (!wide && (p.bias.data || p.kv_lens || padded || p.mask.window > 0 || p.dropout_p > 0.f || smod)) {
    BwdM g;
    fill(g, p);
    const int D = E <= 64 ? 64 : 128;
    if (!bwd_dkdv_w32_fits(g, D) || !bwd_dq_w32_fits(g, D)) return *why = "masked call / padded head dim beyond 32-bit offsets", false;
  }
  return true;
}

// delta and lse2, rounded up to 256 bytes, and behind them the partial dK / dV rows of a call whose
// dK/dV kernel splits its items
static size_t row_stats_bytes(const mi355_sdpa_bwd_params& p) {
  return ((size_t)(p.q.size[0] * p.q.size[1] * p.q.size[2]) * 2 * sizeof(float) + 255) & ~(size_t)255;
}
// (behind them, for a call with sorted document ids: the order in which the dK/dV kernel takes the key
// blocks of each batch, one int per block)
static size_t key_order_bytes(const mi355_sdpa_bwd_params& p) {
  if (!p.mask.doc_ids_sorted || !p.mask.doc_ids_q || !p.mask.doc_ids_k) return 0;
  return ((size_t)p.q.size[0] * ((p.k.size[2] + 127) / 128) * sizeof(int32_t) + 255) & ~(size_t)255;
}
static size_t row_terms_bytes(const mi355_sdpa_bwd_params& p) { return row_stats_bytes(p) + key_order_bytes(p); }
static int parts_of(const BwdM& g, const mi355_sdpa_bwd_params& p) {
  if (p.k.size[2] <= 0 || p.k.size[1] <= 0) return 1;
  if (p.q.size[3] > 128 || p.v.size[3] != p.q.size[3]) return bwd_wide_parts(g);
  return bwd_dkdv_w32_fits(g, p.q.size[3] <= 64 ? 64 : 128) ? bwd_dkdv_w32_parts(g) : 1;
}
static size_t part_rows_bytes(const BwdM& g, int parts) {  // dK rows, then dV rows
  const size_t bytes = parts > 1 ? (size_t)parts * g.B * g.Hkv * g.S * (g.d_real + g.dv_real) * sizeof(float) : 0;
  return (bytes + 255) & ~(size_t)255;
}
// Few query rows against many keys (cross attention over a long memory): parts into which the dQ
// kernel of bwd_dq_w32.hip splits its keys - at least 1024 keys each, about two workgroups per compute
// unit in all - and the tiles of 32 keys per part.  1: no split (and for every call with a bias, dropout,
// a functor, a window or a verdict, which that kernel's variant for split keys does not take).
static int dq_splits(const BwdM& g, const mi355_sdpa_bwd_params& p, int* split_tiles) {
  *split_tiles = 0;
  if (p.q.size[3] > 128 || p.v.size[3] != p.q.size[3] || g.bias_kind || g.gbias || g.keep_scale != 0.f || g.sm.any ||
      g.window > 0 || g.verdict || g.live_tiles || g.live_t || p.force_kernel == MI355_SDPA_KERNEL_GENERIC)
    return 1;
  if (!bwd_dq_w32_fits(g, p.q.size[3] <= 64 ? 64 : 128)) return 1;
  const int64_t blocks = (int64_t)g.B * g.Hq * ((g.L + 255) / 256);
  const int nt = (g.S + 31) / 32;
  if (blocks >= 128 || nt < 64) return 1;
  const int want = (int)std::min<int64_t>(std::min<int64_t>((512 + blocks - 1) / blocks, nt / 32), 64);
  if (want <= 1) return 1;
  *split_tiles = (nt + want - 1) / want;
  return (nt + *split_tiles - 1) / *split_tiles;
}
static size_t dq_part_bytes(const BwdM& g, int n_split) {
  return n_split > 1 ? (size_t)n_split * g.B * g.Hq * g.L * g.d_real * sizeof(float) : 0;
}
size_t bwd_mfma_workspace(const mi355_sdpa_bwd_params& p) {
  if (p.dtype != MI355_SDPA_BF16 && p.dtype != MI355_SDPA_F16) return row_terms_bytes(p);
  BwdM g;
  fill(g, p);
  int split_tiles;
  return row_terms_bytes(p) + part_rows_bytes(g, parts_of(g, p)) + dq_part_bytes(g, dq_splits(g, p, &split_tiles));
}

int launch_bwd_mfma(const mi355_sdpa_bwd_params& p, hipStream_t s) {
  const char* why;
  if (!bwd_mfma_supported(p, &why)) {
    set_error("SDPA: MFMA backward kernel cannot take this call: %s", why);
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  BwdM g;
  fill(g, p);
  const int parts = parts_of(g, p);
  if (parts > 1 && p.workspace_bytes >= row_terms_bytes(p) + part_rows_bytes(g, parts)) {
    g.parts = parts;
    g.part_dk = (float*)((char*)p.workspace + row_terms_bytes(p));
    g.part_dv = g.part_dk + (size_t)parts * g.B * g.Hkv * g.S * g.d_real;
  }
  {
    int split_tiles;
    const int n_split = dq_splits(g, p, &split_tiles);
    const size_t at = row_terms_bytes(p) + part_rows_bytes(g, parts);
    if (n_split > 1 && p.workspace_bytes >= at + dq_part_bytes(g, n_split))
      g.dq_split_tiles = split_tiles, g.dq_n_split = n_split, g.part_dq = (float*)((char*)p.workspace + at);
  }
  if (key_order_bytes(p) && p.workspace_bytes >= row_terms_bytes(p)) g.kt_order = (int32_t*)((char*)p.workspace + row_stats_bytes(p));
  const int D = p.q.size[3] <= 64 ? 64 : 128;  // the kernels' width
  int rc;
  if (p.q.size[3] > 128 || p.v.size[3] != p.q.size[3]) rc = launch_bwd_wide(g, p.dtype, s);
  else if (p.dtype == MI355_SDPA_BF16) rc = D == 128 ? launch_td<bf16_t, 128>(g, s) : launch_td<bf16_t, 64>(g, s);
  else rc = D == 128 ? launch_td<f16_t, 128>(g, s) : launch_td<f16_t, 64>(g, s);
  // (a sink logit changes nothing in these kernels: the probabilities come from the saved
  // log-sum-exp, which includes it; only its own gradient is one more small reduction)
  if (rc == MI355_SDPA_OK && p.grad_sink_logit && p.mask.sink_logit)
    rc = launch_sink_grad(p.lse, g.delta, p.mask.sink_logit, p.grad_sink_logit, (int64_t)g.B * g.Hq, g.L, p.mask.n_sink_logits, s);
  return rc;
}

}  // namespace mi355
