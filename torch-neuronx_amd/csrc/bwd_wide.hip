// Flash-attention backward for head dims above 128 and for D_qk != D_v (D_v <= D_qk <= 256,
// multiples of 8; e.g. 192 / 128 of multi-head latent attention, or 256 / 256), bf16/f16, on the
// 32x32x16 MFMA.  Two kernels built for the widest case, rows narrower than 256 counting as zero
// padded; one wavefront per SIMD with the 512-register budget, compiler-scheduled: the point of
// these kernels is to keep such calls on the matrix pipe (the float32 generic kernels that served
// them run at 1-2 TFLOP/s), not to match the hand-pipelined kernels for head dims 64 / 128.
//
//   bwd_wide_dq_kernel    128 query rows per workgroup (4 wavefronts x 32 rows), 32-key tiles:
//                           S^T = K Q^T, dP^T = V dO^T, dS^T = P^T (dP^T - delta), dQ^T += K^T dS^T
//                         it also forms delta = rowsum(dO * O) and leaves it, with the log2-domain
//                         log-sum-exp, in the workspace for the second kernel
//   bwd_wide_dkdv_kernel  128 keys per workgroup (4 wavefronts x 32 keys); loops over the query
//                         heads of the group (the GQA sum of decompositions.py:2595-2598 happens in
//                         registers) and over 32-row query tiles:
//                           S = Q K^T, dP = dO V^T, P = exp2(c S - lse), dS = P (dP - delta)
//                           dV^T += dO^T P, dK^T += Q^T dS
//
// Tiles sit in LDS row-major with a padded pitch; transposed operands come out of the transposing
// LDS read.  Math follows torch_neuronx/_sdpa_math.py:98-176: float32 accumulation, rows with
// lse = -inf give zero gradients, scale multiplies dQ and dK once at the end.
#include "bwd_mfma.h"

namespace mi355 {
namespace {

constexpr int DW = 256;           // the width the kernels are built for
constexpr int KS = DW / 16;       // contraction steps over the head dim
constexpr int DB = DW / 32;       // 32-row blocks of a transposed product
constexpr int PITCH = DW + 8;     // LDS row pitch in elements: 16-byte row reads of 16 lanes hit every bank once
constexpr int BT = 32;            // rows of a staged tile

typedef short s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 tr_read(const uint16_t* ptr) {
  const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(ptr));
  return __builtin_bit_cast(u32x2, v);
}

// A 32-row tile of a (rows, width) matrix on its way to LDS, zero beyond `width` and beyond
// `rows_left` rows: fetched into registers one tile ahead (the loads travel under the matrix ops
// of the current tile) and written to LDS between two barriers.  256 threads, 16-byte chunks:
// chunk c of row r at r * PITCH + 8 c.
constexpr int NST = (BT * (DW / 8)) / 256;  // chunks per thread and tile
struct TileRegs {
  u32x4 w[NST];
  __device__ __forceinline__ void fetch(const uint16_t* base, int64_t row_stride, int rows_left, int width, int tid) {
#pragma unroll
    for (int n = 0; n < NST; ++n) {
      const int u = tid + n * 256, r = u / (DW / 8), ch = u % (DW / 8);
      w[n] = u32x4{0u, 0u, 0u, 0u};
      if (r < rows_left && ch * 8 < width) w[n] = *(const u32x4*)(base + (int64_t)r * row_stride + ch * 8);
    }
  }
  __device__ __forceinline__ void put(uint16_t* lds, int tid) const {
#pragma unroll
    for (int n = 0; n < NST; ++n) {
      const int u = tid + n * 256, r = u / (DW / 8), ch = u % (DW / 8);
      *(u32x4*)(lds + r * PITCH + ch * 8) = w[n];
    }
  }
};

// element offsets of the transposing reads of a tile, [second read of a pair][d block]
struct TrOff {
  int off[2][DB];
  __device__ __forceinline__ void init(int lane) {
    const int jj = lane & 15, g = lane >> 4;
#pragma unroll
    for (int sec = 0; sec < 2; ++sec)
#pragma unroll
      for (int db = 0; db < DB; ++db)
        off[sec][db] = (8 * sec + (g >> 1) * 4 + (jj >> 2)) * PITCH + db * 32 + 16 * (g & 1) + 4 * (jj & 3);
  }
  // operand i = DB * (16-row step) + d block of the transposed tile
  __device__ __forceinline__ u32x4 cols(const uint16_t* tile, int i) const {
    const u32x2 lo = tr_read(tile + off[0][i % DB] + (i / DB) * 16 * PITCH);
    const u32x2 hi = tr_read(tile + off[1][i % DB] + (i / DB) * 16 * PITCH);
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
  }
};

template <typename T>
__global__ __launch_bounds__(256, 1) void bwd_wide_dq_kernel(BwdM p) {
  __shared__ __attribute__((aligned(16))) uint16_t k_t[BT * PITCH];
  __shared__ __attribute__((aligned(16))) uint16_t v_t[BT * PITCH];
  const int n_qt = (p.L + 127) / 128;
  const int qt = n_qt - 1 - blockIdx.x / (p.B * p.Hq);  // heavy query tiles first
  const int bh = blockIdx.x % (p.B * p.Hq), b = bh / p.Hq, h = bh % p.Hq, hk = h / (p.Hq / p.Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 31, half = lane >> 5;
  const int q0 = qt * 128, qw0 = q0 + wave * 32, qrow = qw0 + col, qc = min(qrow, p.L - 1);
  const int er = p.d_real, dvr = p.dv_real;

  u32x4 qf[KS], dof[KS];
  float lse2, dl;
  {
    const uint16_t* qr = (const uint16_t*)p.q + b * p.q_sb + h * p.q_sh + (int64_t)qc * p.q_sl + half * 8;
    const uint16_t* gr = (const uint16_t*)p.go + b * p.go_sb + h * p.go_sh + (int64_t)qc * p.go_sl + half * 8;
    const uint16_t* orow = (const uint16_t*)p.out + b * p.o_sb + h * p.o_sh + (int64_t)qc * p.o_sl + half * 8;
    float dsum = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = half * 8 + ks * 16 < er ? *(const u32x4*)(qr + ks * 16) : u32x4{0u, 0u, 0u, 0u};
      if (half * 8 + ks * 16 < dvr) {
        dof[ks] = *(const u32x4*)(gr + ks * 16);
        dsum += dot8<T>(dof[ks], *(const u32x4*)(orow + ks * 16));
      } else {
        dof[ks] = u32x4{0u, 0u, 0u, 0u};
      }
    }
    dsum += __shfl_xor(dsum, 32, 64);
    const int64_t idx = ((int64_t)b * p.Hq + h) * p.L + qc;
    const float l = p.lse[idx];
    // +inf turns exp2(x - lse) into 0 for rows past L and for rows without a live key
    lse2 = (qrow < p.L && l != -INFINITY) ? l * kLog2eF : INFINITY;
    dl = dsum;
    if (qrow < p.L && half == 0) p.delta[idx] = dsum, p.lse2[idx] = l != -INFINITY ? l * kLog2eF : INFINITY;
  }
  TrOff tr;
  tr.init(lane);
  f32x16 dqacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) zero(dqacc[i]);
  const float c = p.scale * kLog2eF;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const uint16_t* kp = (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh;
  const uint16_t* vp = (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh;
  int nt = (p.S + BT - 1) / BT;
  if (p.causal) nt = min(nt, (min(q0 + 128, p.L) - 1) / BT + 1);
  const int nt_w = p.causal ? min(nt, (qw0 + 31) / BT + 1) : nt;  // tiles with work for this wavefront
  const int lim = p.causal ? min(qrow, p.S - 1) : p.S - 1;

  TileRegs kn, vn;
  if (nt > 0) kn.fetch(kp, p.k_sl, p.S, er, tid), vn.fetch(vp, p.v_sl, p.S, dvr, tid);
  for (int t = 0; t < nt; ++t) {
    __syncthreads();  // the previous tile has been read by every wavefront
    kn.put(k_t, tid), vn.put(v_t, tid);
    __syncthreads();
    if (t + 1 < nt) {
      kn.fetch(kp + (int64_t)(t + 1) * BT * p.k_sl, p.k_sl, p.S - (t + 1) * BT, er, tid);
      vn.fetch(vp + (int64_t)(t + 1) * BT * p.v_sl, p.v_sl, p.S - (t + 1) * BT, dvr, tid);
    }
    if (t >= nt_w) continue;
    f32x16 sacc = zero16, dpacc = zero16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      sacc = Mma<T>::run(*(const u32x4*)(k_t + col * PITCH + ks * 16 + half * 8), qf[ks], sacc);
      dpacc = Mma<T>::run(*(const u32x4*)(v_t + col * PITCH + ks * 16 + half * 8), dof[ks], dpacc);
    }
    uint32_t pS[8];
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      float ds[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int kv = t * BT + ((r + e) >> 2) * 8 + half * 4 + ((r + e) & 3);
        float pr = __builtin_amdgcn_exp2f(fmaf(sacc[r + e], c, -lse2));
        pr = kv > lim ? 0.f : pr;
        ds[e] = pr * (dpacc[r + e] - dl);
      }
      pS[r >> 1] = Mma<T>::pack(ds[0], ds[1]);
    }
#pragma unroll
    for (int i = 0; i < 2 * DB; ++i) {
      const int r0 = (i / DB) * 4;
      const u32x4 bS = {pS[r0], pS[r0 + 1], pS[r0 + 2], pS[r0 + 3]};
      dqacc[i % DB] = Mma<T>::run(tr.cols(k_t, i), bS, dqacc[i % DB]);
    }
  }
  if (qrow < p.L) {
    uint16_t* gq = (uint16_t*)p.gq + b * p.gq_sb + h * p.gq_sh + (int64_t)qrow * p.gq_sl;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        w[0] = Mma<T>::pack(dqacc[db][g * 4] * p.scale, dqacc[db][g * 4 + 1] * p.scale);
        w[1] = Mma<T>::pack(dqacc[db][g * 4 + 2] * p.scale, dqacc[db][g * 4 + 3] * p.scale);
        if (db * 32 + g * 8 + half * 4 < er) *(u32x2*)(gq + db * 32 + g * 8 + half * 4) = w;
      }
  }
}

template <typename T>
__global__ __launch_bounds__(256, 1) void bwd_wide_dkdv_kernel(BwdM p) {
  __shared__ __attribute__((aligned(16))) uint16_t q_t[BT * PITCH];
  __shared__ __attribute__((aligned(16))) uint16_t do_t[BT * PITCH];
  __shared__ __attribute__((aligned(16))) float lse_s[BT];
  __shared__ __attribute__((aligned(16))) float dl_s[BT];
  const int streams = p.B * p.Hkv;
  const int kt = blockIdx.x / streams;  // low key tiles see the most queries under a causal mask: first
  const int st = blockIdx.x % streams, b = st / p.Hkv, hk = st % p.Hkv, rep = p.Hq / p.Hkv;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 31, half = lane >> 5;
  const int k0 = kt * 128, kw0 = k0 + wave * 32, key = kw0 + col;
  const int er = p.d_real, dvr = p.dv_real;

  u32x4 kf[KS], vf[KS];
  {
    const int kc = min(key, p.S - 1);
    const uint16_t* kr = (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh + (int64_t)kc * p.k_sl + half * 8;
    const uint16_t* vr = (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh + (int64_t)kc * p.v_sl + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kf[ks] = half * 8 + ks * 16 < er ? *(const u32x4*)(kr + ks * 16) : u32x4{0u, 0u, 0u, 0u};
      vf[ks] = half * 8 + ks * 16 < dvr ? *(const u32x4*)(vr + ks * 16) : u32x4{0u, 0u, 0u, 0u};
    }
  }
  TrOff tr;
  tr.init(lane);
  f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) zero(dkacc[i]), zero(dvacc[i]);
  const float c = p.scale * kLog2eF;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int nqs = (p.L + BT - 1) / BT;
  const int qs_begin = p.causal ? min(k0 / BT, nqs) : 0;

  // (no fetch ahead here: the two accumulators and the two fragments fill the register file, and the
  // 32 registers of a tile in flight spill)
  // Query tile by query tile from the last one down, heads inside: the workgroups of a kv head, which
  // share an XCD, then want the same Q / dO tile at about the same time and find it in its L2.
  for (int qs = nqs - 1; qs >= qs_begin; --qs) {
    for (int hg = 0; hg < rep; ++hg) {
      const int h = hk * rep + hg;
      const uint16_t* qb = (const uint16_t*)p.q + b * p.q_sb + h * p.q_sh;
      const uint16_t* gb = (const uint16_t*)p.go + b * p.go_sb + h * p.go_sh;
      const int64_t row0 = ((int64_t)b * p.Hq + h) * p.L;
      const int q0 = qs * BT;
      __syncthreads();  // the previous tile has been read by every wavefront
      {
        TileRegs qn;
        qn.fetch(qb + (int64_t)q0 * p.q_sl, p.q_sl, p.L - q0, er, tid);
        qn.put(q_t, tid);
        qn.fetch(gb + (int64_t)q0 * p.go_sl, p.go_sl, p.L - q0, dvr, tid);
        qn.put(do_t, tid);
      }
      if (tid < BT) {
        const int qi = q0 + tid;
        // rows past L are switched off through lse = +inf
        lse_s[tid] = qi < p.L ? p.lse2[row0 + qi] : INFINITY;
        dl_s[tid] = qi < p.L ? p.delta[row0 + qi] : 0.f;
      }
      __syncthreads();
      if ((p.causal && q0 + BT - 1 < kw0) || kw0 >= p.S) continue;  // (uniform per wavefront)
      // the accumulators are touched by matrix ops only: accumulation registers; the K / V fragments
      // feed every matrix op as a source operand: ordinary vector registers
#pragma unroll
      for (int i = 0; i < DB; ++i) {
        asm volatile("" : "+a"(dkacc[i]));
        asm volatile("" : "+a"(dvacc[i]));
      }
      f32x16 sacc = zero16, dpacc = zero16;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        sacc = Mma<T>::run(*(const u32x4*)(q_t + col * PITCH + ks * 16 + half * 8), kf[ks], sacc);
        dpacc = Mma<T>::run(*(const u32x4*)(do_t + col * PITCH + ks * 16 + half * 8), vf[ks], dpacc);
      }
      uint32_t pP[8], pS[8];
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const f32x4 l4 = *(const f32x4*)(&lse_s[r4 * 8 + half * 4]);
        const f32x4 d4 = *(const f32x4*)(&dl_s[r4 * 8 + half * 4]);
        float pr[4], ds[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = r4 * 4 + e, qi = q0 + r4 * 8 + half * 4 + e;
          pr[e] = __builtin_amdgcn_exp2f(fmaf(sacc[r], c, -l4[e]));
          pr[e] = ((p.causal && key > qi) || key >= p.S) ? 0.f : pr[e];
          ds[e] = pr[e] * (dpacc[r] - d4[e]);
        }
        pP[r4 * 2] = Mma<T>::pack(pr[0], pr[1]), pP[r4 * 2 + 1] = Mma<T>::pack(pr[2], pr[3]);
        pS[r4 * 2] = Mma<T>::pack(ds[0], ds[1]), pS[r4 * 2 + 1] = Mma<T>::pack(ds[2], ds[3]);
      }
#pragma unroll
      for (int i = 0; i < 2 * DB; ++i) {
        const int r0 = (i / DB) * 4;
        const u32x4 bP = {pP[r0], pP[r0 + 1], pP[r0 + 2], pP[r0 + 3]};
        const u32x4 bS = {pS[r0], pS[r0 + 1], pS[r0 + 2], pS[r0 + 3]};
        dvacc[i % DB] = Mma<T>::run(tr.cols(do_t, i), bP, dvacc[i % DB]);
        dkacc[i % DB] = Mma<T>::run(tr.cols(q_t, i), bS, dkacc[i % DB]);
      }
    }
  }
  if (key < p.S) {
    uint16_t* gk = (uint16_t*)p.gk + b * p.gk_sb + hk * p.gk_sh + (int64_t)key * p.gk_sl;
    uint16_t* gv = (uint16_t*)p.gv + b * p.gv_sb + hk * p.gv_sh + (int64_t)key * p.gv_sl;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 wk, wv;
        wk[0] = Mma<T>::pack(dkacc[db][g * 4] * p.scale, dkacc[db][g * 4 + 1] * p.scale);
        wk[1] = Mma<T>::pack(dkacc[db][g * 4 + 2] * p.scale, dkacc[db][g * 4 + 3] * p.scale);
        wv[0] = Mma<T>::pack(dvacc[db][g * 4], dvacc[db][g * 4 + 1]);
        wv[1] = Mma<T>::pack(dvacc[db][g * 4 + 2], dvacc[db][g * 4 + 3]);
        if (db * 32 + g * 8 + half * 4 < er) *(u32x2*)(gk + db * 32 + g * 8 + half * 4) = wk;
        if (db * 32 + g * 8 + half * 4 < dvr) *(u32x2*)(gv + db * 32 + g * 8 + half * 4) = wv;
      }
  }
}

template <typename T>
int launch_t(const BwdM& g, hipStream_t s) {
  const int64_t q_blocks = (int64_t)g.B * g.Hq * ((g.L + 127) / 128), k_blocks = (int64_t)g.B * g.Hkv * ((g.S + 127) / 128);
  if (q_blocks > 0x7fffffff || k_blocks > 0x7fffffff) {
    set_error("SDPA: too many tiles for the wide backward kernels");
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  hipLaunchKernelGGL((bwd_wide_dq_kernel<T>), dim3((unsigned)q_blocks), dim3(256), 0, s, g);
  int rc = check_launch("bwd_wide_dq_kernel");
  if (rc) return rc;
  hipLaunchKernelGGL((bwd_wide_dkdv_kernel<T>), dim3((unsigned)k_blocks), dim3(256), 0, s, g);
  return check_launch("bwd_wide_dkdv_kernel");
}

}  // namespace

int launch_bwd_wide(const BwdM& g, int dtype, hipStream_t s) {
  return dtype == MI355_SDPA_BF16 ? launch_t<bf16_t>(g, s) : launch_t<f16_t>(g, s);
}

}  // namespace mi355
