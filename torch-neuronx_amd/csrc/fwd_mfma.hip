// Flash-attention forward for gfx950 on the 32x32x16 bf16/f16 MFMA.
//
// Work split: one workgroup = 4 wavefronts = 128 query rows of one (batch, query head);
// each wavefront owns 32 query rows and walks the keys in tiles of 64.  Two workgroups fit
// one compute unit (<=256 VGPRs, 2 x ~35 KB LDS), so while one wavefront is in its softmax
// the matrix pipe is fed by its neighbour.
//
// Both products are computed TRANSPOSED so that the softmax needs no shuffle and P never
// leaves registers:
//   S^T = K * Q^T   (A = K tile from LDS,   B = Q fragment held in registers)
//   O^T = V^T * P^T (A = V^T tile from LDS, B = P^T = exp2(S^T ...) re-packed in registers)
// In the 32x32 accumulator layout a lane then holds one query column (lane % 32) and 16 key
// rows per 32-key block, so the row max / row sum of a query are per-lane scalars plus one
// exchange with lane ^ 32, and the accumulator registers of S^T are, pairwise packed, exactly
// the B operand of the second product.  The order in which the contraction index is spread
// over lanes is free as long as A and B agree; V^T is stored in LDS in the matching order.
//
// K tile in LDS: row-major [key][d], rows padded by 16 bytes (conflict-free 128-bit reads).
// V tile in LDS: transposed [d][key] in groups of four keys, built from 4x(8 d) register
// blocks with byte permutes; row padded by 16 bytes.  Both tiles are double buffered; the
// global loads of tile j+2 are in flight while tile j is consumed.
//
// Numerics follow torch_neuronx/_sdpa_math.py:51-95: raw dot products accumulate in
// float32, the scale is applied in float32 inside the exponent, probabilities are rounded
// to the input dtype only as the operand of P*V while the row sum uses the float32 values,
// a row without a live key yields zeros and lse = -inf.
#include "common.h"

namespace mi355 {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr int BM = 128;  // query rows per workgroup
constexpr int BN = 64;   // keys per tile
constexpr int PAD = 8;   // elements of row padding in LDS (16 bytes)
constexpr float kLog2e = 1.4426950408889634f;

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
};

template <typename T>
struct Mma;
template <>
struct Mma<bf16_t> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
    bf16x2 r = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, r);
  }
};
template <>
struct Mma<f16_t> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
    f16x2 r = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, r);
  }
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

template <typename T, int D>
__global__ __launch_bounds__(256, 2) void fwd_mfma_kernel(FwdM p) {
  constexpr int KS = D / 16;       // contraction steps of S^T = K Q^T
  constexpr int DB = D / 32;       // 32-row blocks of O^T
  constexpr int KROW = D + PAD;    // K tile row pitch (elements)
  constexpr int VROW = BN + PAD;   // V^T tile row pitch (elements)
  constexpr int KCH = D / 8;       // 16-byte chunks per K row
  constexpr int KLD = (BN * KCH) / 256;  // K chunks per thread
  __shared__ __attribute__((aligned(16))) uint16_t k_lds[2][BN * KROW];
  __shared__ __attribute__((aligned(16))) uint16_t v_lds[2][D * VROW];

  int b, h, qt;
  decode_block(p, b, h, qt);
  const int hk = h / (p.Hq / p.Hkv);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int col = lane & 31, half = lane >> 5;
  const int q0 = qt * BM;
  const int qw0 = q0 + wave * 32;  // first query row of this wavefront
  const int qrow = qw0 + col;      // this lane's query row

  const uint16_t* qp = (const uint16_t*)p.q + b * p.q_sb + h * p.q_sh;
  const uint16_t* kp = (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh;
  const uint16_t* vp = (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh;

  // ---- Q fragment (B operand): lane = query column, 8 consecutive d per step ------------
  u32x4 qf[KS];
  {
    const uint16_t* qr = qp + (int64_t)min(qrow, p.L - 1) * p.q_sl + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const u32x4*)(qr + ks * 16);
  }

  // number of key tiles this workgroup walks
  int nt = (p.S + BN - 1) / BN;
  if (p.causal) nt = min(nt, (min(q0 + BM, p.L) - 1) / BN + 1);

  // ---- global -> register staging of one K/V tile -------------------------------------------
  u32x4 kreg[KLD], vreg[4];
  const int k_chunk = tid % KCH, k_row0 = tid / KCH;  // rows k_row0 + i * (256 / KCH)
  const int v_g = tid & 15, v_dc = tid >> 4;           // key group of 4, d chunk of 8
  const bool v_loader = v_dc < D / 8;
  auto load_tile = [&](int t) {
    const int kv0 = t * BN;
#pragma unroll
    for (int i = 0; i < KLD; ++i) {
      const int r = min(kv0 + k_row0 + i * (256 / KCH), p.S - 1);
      kreg[i] = *(const u32x4*)(kp + (int64_t)r * p.k_sl + k_chunk * 8);
    }
    if (v_loader) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = min(kv0 + v_g * 4 + i, p.S - 1);
        vreg[i] = *(const u32x4*)(vp + (int64_t)r * p.v_sl + v_dc * 8);
      }
    }
  };
  // position (in 4-key units) of key group g inside a V^T row: within every 16 keys the
  // groups are stored 0,2,1,3 so that the 8 keys one lane needs are contiguous
  const int v_pos = (v_g & ~3) | ((v_g & 1) << 1) | ((v_g >> 1) & 1);
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < KLD; ++i) {
      const int r = k_row0 + i * (256 / KCH);
      *(u32x4*)(&k_lds[buf][r * KROW + k_chunk * 8]) = kreg[i];
    }
    if (v_loader) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {  // dword c of each row holds d = 2c, 2c+1
        const uint32_t a0 = vreg[0][c], a1 = vreg[1][c], a2 = vreg[2][c], a3 = vreg[3][c];
        u32x2 even, odd;
        even[0] = __builtin_amdgcn_perm(a1, a0, 0x05040100);  // (a0.lo, a1.lo)
        even[1] = __builtin_amdgcn_perm(a3, a2, 0x05040100);
        odd[0] = __builtin_amdgcn_perm(a1, a0, 0x07060302);   // (a0.hi, a1.hi)
        odd[1] = __builtin_amdgcn_perm(a3, a2, 0x07060302);
        const int d = v_dc * 8 + 2 * c;
        *(u32x2*)(&v_lds[buf][d * VROW + v_pos * 4]) = even;
        *(u32x2*)(&v_lds[buf][(d + 1) * VROW + v_pos * 4]) = odd;
      }
    }
  };

  f32x16 oacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
  float m_run = -INFINITY;  // running max of the raw dot products of this lane's query
  float l_run = 0.f;        // this lane's share of the running row sum
  const float c = p.scale * kLog2e;

  load_tile(0);
  store_tile(0);
  __syncthreads();
  if (nt > 1) load_tile(1);

  for (int t = 0; t < nt; ++t) {
    const int buf = t & 1;
    const int kv0 = t * BN;
    // causal: this wavefront has nothing to do once the tile starts past its last row
    const bool active = !p.causal || kv0 <= qw0 + 31;
    if (active) {
      // ---- S^T = K Q^T ------------------------------------------------------------------
      f32x16 sacc[2];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[mb][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
          const u32x4 a =
              *(const u32x4*)(&k_lds[buf][(mb * 32 + col) * KROW + ks * 16 + half * 8]);
          sacc[mb] = Mma<T>::run(a, qf[ks], sacc[mb]);
        }
      }
      // ---- masks --------------------------------------------------------------------------
      const bool edge = (p.causal && kv0 + BN - 1 > qw0) || (kv0 + BN > p.S);
      if (edge) {
        const int lim = p.causal ? min(qrow, p.S - 1) : p.S - 1;  // last key this query sees
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int kv = kv0 + mb * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
            if (kv > lim) sacc[mb][r] = -INFINITY;
          }
      }
      // ---- online softmax -----------------------------------------------------------------
      float tmax = sacc[0][0];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, sacc[mb][r]);
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(m_run, tmax);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);
      m_run = m_new;
      const float mc = m_use * c;
      float psum = 0.f;
      uint32_t pk[2][8];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const float p0 = __builtin_amdgcn_exp2f(fmaf(sacc[mb][r], c, -mc));
          const float p1 = __builtin_amdgcn_exp2f(fmaf(sacc[mb][r + 1], c, -mc));
          psum += p0 + p1;
          pk[mb][r >> 1] = Mma<T>::pack(p0, p1);
        }
      l_run = l_run * alpha + psum;
#pragma unroll
      for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
      // ---- O^T += V^T P^T -----------------------------------------------------------------
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        u32x4 bfrag;
        const int mb = ks >> 1, r0 = (ks & 1) * 4;
        bfrag[0] = pk[mb][r0], bfrag[1] = pk[mb][r0 + 1];
        bfrag[2] = pk[mb][r0 + 2], bfrag[3] = pk[mb][r0 + 3];
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const u32x4 a =
              *(const u32x4*)(&v_lds[buf][(db * 32 + col) * VROW + ks * 16 + half * 8]);
          oacc[db] = Mma<T>::run(a, bfrag, oacc[db]);
        }
      }
    }
    if (t + 1 < nt) store_tile(buf ^ 1);
    __syncthreads();
    if (t + 2 < nt) load_tile(t + 2);
  }

  // ---- epilogue -----------------------------------------------------------------------------
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (qrow < p.L) {
    uint16_t* orow = (uint16_t*)p.out + b * p.o_sb + h * p.o_sh + (int64_t)qrow * p.o_sl;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        w[0] = Mma<T>::pack(oacc[db][g * 4 + 0] * inv, oacc[db][g * 4 + 1] * inv);
        w[1] = Mma<T>::pack(oacc[db][g * 4 + 2] * inv, oacc[db][g * 4 + 3] * inv);
        *(u32x2*)(orow + db * 32 + g * 8 + half * 4) = w;
      }
    if (p.lse && half == 0)
      p.lse[((int64_t)b * p.Hq + h) * p.L + qrow] =
          l_tot > 0.f ? m_run * p.scale + __builtin_logf(l_tot) : -INFINITY;
  }
}

}  // namespace

bool fwd_mfma_supported(const mi355_sdpa_fwd_params& p, const char** why) {
  static const char* ok = "";
  *why = ok;
  const int64_t E = p.q.size[3], Dv = p.v.size[3];
  if (p.dtype != MI355_SDPA_BF16 && p.dtype != MI355_SDPA_F16) return *why = "dtype is not bf16/f16", false;
  if (E != Dv || (E != 64 && E != 128)) return *why = "head dim is not 64 or 128", false;
  if (p.bias.data) return *why = "attn_bias present", false;
  if (p.kv_lens) return *why = "kv_lens present", false;
  if (p.dropout_p > 0.f) return *why = "dropout", false;
  if (!(p.scale > 0.f)) return *why = "scale <= 0", false;
  if (p.q.size[2] < 1 || p.k.size[2] < 1) return *why = "empty sequence", false;
  if (p.q.stride[3] != 1 || p.k.stride[3] != 1 || p.v.stride[3] != 1 || p.out.stride[3] != 1)
    return *why = "head dim is not unit-stride", false;
  const mi355_sdpa_tensor* ts[4] = {&p.q, &p.k, &p.v, &p.out};
  for (const mi355_sdpa_tensor* t : ts) {
    if (((uintptr_t)t->data & 15) != 0) return *why = "pointer not 16-byte aligned", false;
    for (int i = 0; i < 3; ++i)
      if (t->size[i] > 1 && (t->stride[i] % 8) != 0) return *why = "stride not a multiple of 8 elements", false;
  }
  return true;
}

int launch_fwd_mfma(const mi355_sdpa_fwd_params& p, hipStream_t s) {
  const char* why;
  if (!fwd_mfma_supported(p, &why)) {
    set_error("SDPA: MFMA forward kernel cannot take this call: %s", why);
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  FwdM g;
  g.q = p.q.data, g.k = p.k.data, g.v = p.v.data, g.out = p.out.data, g.lse = p.lse;
  g.q_sb = p.q.stride[0], g.q_sh = p.q.stride[1], g.q_sl = p.q.stride[2];
  g.k_sb = p.k.stride[0], g.k_sh = p.k.stride[1], g.k_sl = p.k.stride[2];
  g.v_sb = p.v.stride[0], g.v_sh = p.v.stride[1], g.v_sl = p.v.stride[2];
  g.o_sb = p.out.stride[0], g.o_sh = p.out.stride[1], g.o_sl = p.out.stride[2];
  g.B = (int)p.q.size[0], g.Hq = (int)p.q.size[1], g.Hkv = (int)p.k.size[1];
  g.L = (int)p.q.size[2], g.S = (int)p.k.size[2];
  g.n_qt = (g.L + BM - 1) / BM;
  g.causal = p.is_causal, g.scale = p.scale;
  g.xcd_map = ((g.B * g.Hkv) % 8 == 0) ? 1 : 0;
  const int64_t blocks = (int64_t)g.B * g.Hq * g.n_qt;
  if (blocks == 0) return MI355_SDPA_OK;
  if (blocks > 0x7fffffff) {
    set_error("SDPA: too many query tiles (%lld)", (long long)blocks);
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  dim3 grid((unsigned)blocks), block(256);
  const int D = (int)p.q.size[3];
  if (p.dtype == MI355_SDPA_BF16) {
    if (D == 128) hipLaunchKernelGGL((fwd_mfma_kernel<bf16_t, 128>), grid, block, 0, s, g);
    else hipLaunchKernelGGL((fwd_mfma_kernel<bf16_t, 64>), grid, block, 0, s, g);
  } else {
    if (D == 128) hipLaunchKernelGGL((fwd_mfma_kernel<f16_t, 128>), grid, block, 0, s, g);
    else hipLaunchKernelGGL((fwd_mfma_kernel<f16_t, 64>), grid, block, 0, s, g);
  }
  return check_launch("fwd_mfma_kernel");
}

}  // namespace mi355
