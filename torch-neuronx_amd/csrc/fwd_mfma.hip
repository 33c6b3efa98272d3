// Flash-attention forward for gfx950 on the 32x32x16 bf16/f16 MFMA.
//
// Work split: one workgroup = 4 wavefronts; each wavefront owns NB blocks of 32 query rows
// (NB = 2: 256 query rows per workgroup, one workgroup per compute unit with the full 512
// registers per lane; NB = 1: 128 rows, two workgroups per compute unit, for short sequences)
// and walks the keys in tiles of 64.  This is the first generation of the forward kernel; it
// serves only tensors whose strides are too large for the 32-bit addressing of fwd_mfma_w32.hip.
//
// With NB = 2 each K or V^T fragment read from LDS feeds two MFMAs (two query blocks held in
// registers), which halves the LDS reads per flop.
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
// The key loop is software pipelined by hand inside each wavefront: S^T of tile t+1 runs on
// the matrix pipe while the vector pipe turns S^T of tile t into probabilities, and V^T P^T of
// tile t runs while the vector pipe finds the row max of tile t+1.  The instruction interleave
// is pinned with scheduling-group barriers.  K therefore runs one tile ahead of V through the
// two LDS buffers each of them has; global loads run two to three tiles ahead.
//
// K tile in LDS: row-major [key][d], rows padded by 16 bytes (conflict-free 128-bit reads).
// V tile in LDS: transposed [d][key] in groups of four keys, built from 4x(8 d) register
// blocks with byte permutes; rows padded by 16 bytes.
//
// Numerics follow torch_neuronx/_sdpa_math.py:51-95: raw dot products accumulate in
// float32, the scale is applied in float32 inside the exponent, probabilities are rounded
// to the input dtype only as the operand of P*V while the row sum uses the float32 values,
// a row without a live key yields zeros and lse = -inf.
#include "fwd_mfma.h"

namespace mi355 {
namespace {

constexpr int BN = 64;   // keys per tile
constexpr int PAD = 8;   // elements of row padding in LDS (16 bytes)
constexpr float kLazy = 8.f;  // log2 headroom before the accumulator is rescaled

template <typename T, int D, int NB>
__global__ __launch_bounds__(256, NB == 1 ? 2 : 1) void fwd_mfma_kernel(FwdM p) {
  constexpr int BM = 128 * NB;     // query rows per workgroup
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
  const int qw0 = q0 + wave * (32 * NB);  // first query row of this wavefront
  int qrow[NB];                           // this lane's query rows
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) qrow[nb] = qw0 + nb * 32 + col;
  const int qw_last = qw0 + 32 * NB - 1;

  const uint16_t* qp = (const uint16_t*)p.q + b * p.q_sb + h * p.q_sh;
  const uint16_t* kp = (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh;
  const uint16_t* vp = (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh;

  // ---- Q fragments (B operand): lane = query column, 8 consecutive d per step -------------
  u32x4 qf[NB][KS];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const uint16_t* qr = qp + (int64_t)min(qrow[nb], p.L - 1) * p.q_sl + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[nb][ks] = *(const u32x4*)(qr + ks * 16);
  }

  // number of key tiles this workgroup walks
  int nt = (p.S + BN - 1) / BN;
  if (p.causal) nt = min(nt, (min(q0 + BM, p.L) - 1) / BN + 1);

  // ---- global -> register staging of one K/V tile -------------------------------------------
  u32x4 kreg[KLD], vreg[4];
  const int k_chunk = tid % KCH, k_row0 = tid / KCH;  // rows k_row0 + i * (256 / KCH)
  const int v_g = tid & 15, v_dc = tid >> 4;           // key group of 4, d chunk of 8
  const bool v_loader = v_dc < D / 8;
  auto load_tile_k = [&](int t) {
    const int kv0 = t * BN;
#pragma unroll
    for (int i = 0; i < KLD; ++i) {
      const int r = min(kv0 + k_row0 + i * (256 / KCH), p.S - 1);
      kreg[i] = *(const u32x4*)(kp + (int64_t)r * p.k_sl + k_chunk * 8);
    }
  };
  auto load_tile_v = [&](int t) {
    const int kv0 = t * BN;
    if (v_loader) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = min(kv0 + v_g * 4 + i, p.S - 1);
        vreg[i] = *(const u32x4*)(vp + (int64_t)r * p.v_sl + v_dc * 8);
      }
    }
  };
  auto store_tile_k = [&](int buf) {
#pragma unroll
    for (int i = 0; i < KLD; ++i) {
      const int r = k_row0 + i * (256 / KCH);
      *(u32x4*)(&k_lds[buf][r * KROW + k_chunk * 8]) = kreg[i];
    }
  };
  auto store_tile_v = [&](int buf) {
    if (v_loader) tr_store<VROW>(v_lds[buf], vreg, v_g, v_dc * 8);
  };

  f32x16 oacc[DB][NB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) zero(oacc[i][nb]);
  float m_run[NB], l_run[NB];  // running max of the raw dot products / this lane's share of the row sum
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) m_run[nb] = -INFINITY, l_run[nb] = 0.f;
  const float c = p.scale * kLog2eF;

  const int nt_w = p.causal ? min(nt, qw_last / BN + 1) : nt;  // tiles with work for this wavefront
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  int lim[NB];  // last key each of this lane's queries sees
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) lim[nb] = p.causal ? min(qrow[nb], p.S - 1) : p.S - 1;

  auto mask_tile = [&](f32x16 (&sacc)[2][NB], int kv0) {
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int kv = kv0 + mb * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
          if (kv > lim[nb]) sacc[mb][nb][r] = -INFINITY;
        }
  };
  auto is_edge = [&](int kv0) { return (p.causal && kv0 + BN - 1 > qw0) || (kv0 + BN > p.S); };

  // statistics of the tile whose probabilities are formed next (set by the row-max step)
  float m_new[NB], mc[NB], alpha[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) m_new[nb] = -INFINITY, mc[nb] = 0.f, alpha[nb] = 1.f;
  bool need_rescale = false;
  auto row_max_step = [&](const f32x16 (&sacc)[2][NB]) {
    bool moved = false;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float tmax = fmaxf(sacc[0][nb][0], sacc[1][nb][0]);
#pragma unroll
      for (int r = 1; r < 16; ++r) tmax = fmaxf(fmaxf(tmax, sacc[0][nb][r]), sacc[1][nb][r]);  // v_max3
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      // lazy reference max: raised only when a tile beats it by more than kLazy in the exponent,
      // so O is rescaled a few times per row; probabilities stay below 2^kLazy (exact arithmetic)
      const bool up = (tmax - m_run[nb]) * c > kLazy;  // false for NaN (-inf minus -inf)
      m_new[nb] = up ? tmax : m_run[nb];
      const float m_use = (m_new[nb] == -INFINITY) ? 0.f : m_new[nb];
      moved |= up;
      alpha[nb] = __builtin_amdgcn_exp2f((m_run[nb] - m_use) * c);
      mc[nb] = m_use * c;
    }
    // the running max moves only a handful of times per row: O is rescaled only when it did
    need_rescale = __builtin_amdgcn_ballot_w64(moved) != 0;
  };

  load_tile_k(0);
  load_tile_v(0);
  store_tile_k(0);
  store_tile_v(0);
  if (nt > 1) {
    load_tile_k(1);
    store_tile_k(1);
  }
  __syncthreads();
  if (nt > 1) load_tile_v(1);
  if (nt > 2) load_tile_k(2);

  f32x16 scur[2][NB];
  if (nt_w > 0) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        const u32x4 a = *(const u32x4*)(&k_lds[0][(mb * 32 + col) * KROW + ks * 16 + half * 8]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          scur[mb][nb] = Mma<T>::run(a, qf[nb][ks], ks == 0 ? zero16 : scur[mb][nb]);
      }
    row_max_step(scur);
  }
  __syncthreads();  // tile 0 of K is overwritten at the end of the first iteration

  for (int t = 0; t < nt; ++t) {
    if (t < nt_w) {
      // rare paths first, so that everything after them is one straight-line region: a tile that
      // crosses the causal diagonal or the end of the keys is masked here and its row max redone
      if (is_edge(t * BN)) {
        mask_tile(scur, t * BN);
        row_max_step(scur);
      }
      if (need_rescale) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          l_run[nb] *= alpha[nb];
#pragma unroll
          for (int i = 0; i < DB; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][nb][r] *= alpha[nb];
          m_run[nb] = m_new[nb];
        }
      }
      // ---- phase A: S^T of tile t+1 on the matrix pipe, probabilities of tile t on the VALU ----
      // (for the last tile S^T of a tile that is not there is computed and dropped)
      const uint16_t* kt = k_lds[(t + 1) & 1];
      f32x16 snext[2][NB];
      uint32_t pk[2][NB][8];
      float ps0[NB], ps1[NB];  // the row sum uses the unrounded float32 probabilities
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) ps0[nb] = 0.f, ps1[nb] = 0.f;
      constexpr int EPS = 32 / KS;  // elements per query block handled per contraction step
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
          const u32x4 a = *(const u32x4*)(&kt[(mb * 32 + col) * KROW + ks * 16 + half * 8]);
#pragma unroll
          for (int nb = 0; nb < NB; ++nb)
            snext[mb][nb] = Mma<T>::run(a, qf[nb][ks], ks == 0 ? zero16 : snext[mb][nb]);
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int e = 0; e < EPS; e += 2) {
            const int idx = ks * EPS + e, mb = idx >> 4, r = idx & 15;
            const float p0 = __builtin_amdgcn_exp2f(fmaf(scur[mb][nb][r], c, -mc[nb]));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(scur[mb][nb][r + 1], c, -mc[nb]));
            ps0[nb] += p0, ps1[nb] += p1;
            pk[mb][nb][r >> 1] = Mma<T>::pack(p0, p1);
          }
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) l_run[nb] += ps0[nb] + ps1[nb];
      // ---- phase B: O^T += V^T P^T on the matrix pipe, row max of tile t+1 on the VALU ---------
      const uint16_t* vt = v_lds[t & 1];
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        u32x4 bfrag[NB];
        const int mb = ks >> 1, r0 = (ks & 1) * 4;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          bfrag[nb][0] = pk[mb][nb][r0], bfrag[nb][1] = pk[mb][nb][r0 + 1];
          bfrag[nb][2] = pk[mb][nb][r0 + 2], bfrag[nb][3] = pk[mb][nb][r0 + 3];
        }
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const u32x4 a = *(const u32x4*)(&vt[(db * 32 + col) * VROW + ks * 16 + half * 8]);
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) oacc[db][nb] = Mma<T>::run(a, bfrag[nb], oacc[db][nb]);
        }
      }
      row_max_step(snext);
      // pin the interleave of the whole region: LDS operand fetches two steps ahead, then per
      // fetch NB MFMAs, each followed by its share of the VALU work
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
      for (int i = 0; i < 2 * KS; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // LDS read
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
          __builtin_amdgcn_sched_group_barrier(0x002, (112 + 2 * KS - 1) / (2 * KS), 0);  // VALU
        }
      }
#pragma unroll
      for (int i = 0; i < 4 * DB; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
        }
      }
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) scur[mb][nb] = snext[mb][nb];
    }
    if (t + 2 < nt) store_tile_k(t & 1);
    if (t + 1 < nt) store_tile_v((t + 1) & 1);
    __syncthreads();
    if (t + 3 < nt) load_tile_k(t + 3);
    if (t + 2 < nt) load_tile_v(t + 2);
  }

  // ---- epilogue -----------------------------------------------------------------------------
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const float l_tot = l_run[nb] + __shfl_xor(l_run[nb], 32, 64);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (qrow[nb] < p.L) {
      uint16_t* orow = (uint16_t*)p.out + b * p.o_sb + h * p.o_sh + (int64_t)qrow[nb] * p.o_sl;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          u32x2 w;
          w[0] = Mma<T>::pack(oacc[db][nb][g * 4 + 0] * inv, oacc[db][nb][g * 4 + 1] * inv);
          w[1] = Mma<T>::pack(oacc[db][nb][g * 4 + 2] * inv, oacc[db][nb][g * 4 + 3] * inv);
          *(u32x2*)(orow + db * 32 + g * 8 + half * 4) = w;
        }
      if (p.lse && half == 0)
        p.lse[((int64_t)b * p.Hq + h) * p.L + qrow[nb]] =
            l_tot > 0.f ? m_run[nb] * p.scale + __builtin_logf(l_tot) : -INFINITY;
    }
  }
}

}  // namespace

bool fwd_mfma_supported(const mi355_sdpa_fwd_params& p, const char** why) {
  static const char* ok = "";
  *why = ok;
  const int64_t E = p.q.size[3], Dv = p.v.size[3];
  if (p.dtype != MI355_SDPA_BF16 && p.dtype != MI355_SDPA_F16) return *why = "dtype is not bf16/f16", false;
  // (V may be narrower than Q and K, as in multi-head latent attention's 192 / 128)
  if (E < 8 || E > 256 || E % 8 != 0 || Dv < 8 || Dv > E || Dv % 8 != 0)
    return *why = "head dims are not multiples of 8 up to 256 with D_v <= D_qk", false;
  const bool padded = (E != 64 && E != 128 && E != 256) || Dv != E;  // served by the next wider kernel's masked variant
  const bool w32_only = padded || E > 128;
  // masked calls (bias, bool keep-mask, per-batch key counts) and padded head dims: the kernels
  // with 32-bit row addressing only, and a bias whose rows can be read four keys at a time
  if (p.bias.data || p.kv_lens || w32_only || p.mask.window > 0 || p.mask.sink_logit || score_mod_of(p.mask).any) {
    if ((int64_t)p.k.size[2] * p.k.stride[2] * 2 >= (1ll << 31) || (int64_t)p.k.size[2] * p.v.stride[2] * 2 >= (1ll << 31))
      return *why = "attn_bias / kv_lens / padded head dim with rows beyond 32-bit offsets", false;
  }
  if (p.bias.data) {
    const int esz = p.bias_dtype == MI355_SDPA_F32 ? 4 : p.bias_dtype == MI355_SDPA_BOOL ? 1
                    : (p.bias_dtype == MI355_SDPA_F16 || p.bias_dtype == MI355_SDPA_BF16) ? 2 : 0;
    if (!esz) return *why = "attn_bias dtype", false;
    const int64_t S = p.k.size[2], L = p.q.size[2];
    const int gran = 4 / esz;  // elements per dword
    if (S > 1 && p.bias.stride[3] != 1) return *why = "attn_bias keys are not unit-stride", false;
    if (((uintptr_t)p.bias.data & 3) != 0 || S % gran != 0) return *why = "attn_bias not dword aligned", false;
    for (int i = 0; i < 3; ++i)
      if (p.bias.size[i] > 1 && (p.bias.stride[i] % gran) != 0) return *why = "attn_bias stride not dword aligned", false;
    if ((31 * p.bias.stride[2] + S) * esz >= (1ll << 31)) return *why = "attn_bias rows beyond 32-bit offsets", false;
    (void)L;
  }
  if (p.dropout_p > 0.f) {
    // the keep-mask takes a bool bias's way into the kernel (one dword = four keys of a row)
    const int64_t S = p.k.size[2];
    if (p.mask.window > 0 || p.mask.sink_logit || score_mod_of(p.mask).any) return *why = "dropout together with a functor", false;
    if (!p.dropout_keep || ((uintptr_t)p.dropout_keep & 3) != 0 || (p.dropout_keep_ld > 0 ? p.dropout_keep_ld : p.k.size[2]) % 4 != 0) return *why = "dropout keep-mask rows do not start on dwords", false;
    if (32 * S >= (1ll << 31)) return *why = "dropout keep-mask rows beyond 32-bit offsets", false;
    if ((int64_t)p.k.size[2] * p.k.stride[2] * 2 >= (1ll << 31) || (int64_t)p.k.size[2] * p.v.stride[2] * 2 >= (1ll << 31))
      return *why = "dropout with rows beyond 32-bit offsets", false;
  }
  if (!(p.scale > 0.f)) return *why = "scale <= 0", false;
  if (p.q.size[2] < 1 || p.k.size[2] < 1) return *why = "empty sequence", false;
  if ((p.mask.window > 0 || p.mask.sink_logit || score_mod_of(p.mask).any) && p.bias.data)
    return *why = "window / sink / score functor together with attn_bias", false;
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

// launches the call, or (ws_only) reports the workspace with which it would split its keys
static int launch_or_size(const mi355_sdpa_fwd_params& p, hipStream_t s, size_t* ws_only) {
  const char* why;
  if (ws_only) *ws_only = 0;
  if (!fwd_mfma_supported(p, &why)) {
    if (ws_only) return MI355_SDPA_OK;
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
  g.causal = p.is_causal, g.scale = p.scale;
  g.xcd_map = ((g.B * g.Hkv) % 8 == 0) ? 1 : 0;
  g.kv_lens = p.kv_lens;
  if (p.bias.data) {
    g.bias = p.bias.data;
    g.bias_sb = p.bias.stride[0], g.bias_sh = p.bias.stride[1], g.bias_sl = p.bias.stride[2];
    g.bias_kind = p.bias_dtype == MI355_SDPA_F32 ? 1 : p.bias_dtype == MI355_SDPA_F16 ? 2 : p.bias_dtype == MI355_SDPA_BF16 ? 3 : 4;
  }
  if (p.dropout_p > 0.f) {  // (B, Hq, L, S) contiguous bytes, 1 = keep
    g.keep = p.dropout_keep;
    g.keep_ld = (p.dropout_keep_ld > 0 ? p.dropout_keep_ld : p.k.size[2]);
    g.keep_scale = p.dropout_p < 1.f ? 1.f / (1.f - p.dropout_p) : 1.f;
  }
  g.d_real = (int)p.q.size[3], g.dv_real = (int)p.v.size[3];
  g.window = p.mask.window, g.sink_keys = p.mask.sink_keys, g.sink_logit = p.mask.sink_logit;
  g.n_sinks = p.mask.n_sink_logits > 0 ? p.mask.n_sink_logits : 1;
  g.sm = score_mod_of(p.mask);
  if (p.bias.data && p.mask.live_tiles && !p.is_causal && g.S <= 32768 && p.bias.stride[2] != 0 && p.dropout_p == 0.f) {
    g.live_tiles = p.mask.live_tiles;
    g.live_words = ((g.S + 31) / 32 + 31) / 32, g.live_hm = live_extent(p.bias, 1);
  }
  // (a verdict about the bias is for calls in which nothing else shapes the scores; dropout may come on top)
  if (p.mask.mask_verdict && p.bias.data && g.L > 1 && !p.is_causal && !p.kv_lens &&
      !g.live_tiles && !g.sink_logit && g.window == 0 && !g.sm.any)
    g.verdict = p.mask.mask_verdict;
  if (p.workspace && ((uintptr_t)p.workspace & 255) == 0) g.part_o = (float*)p.workspace, g.part_bytes = p.workspace_bytes;
  const int D = g.d_real <= 64 ? 64 : g.d_real <= 128 ? 128 : 256;  // the kernel's width
  const int64_t wg256 = (int64_t)g.B * g.Hq * ((g.L + 255) / 256);
  const int force_tile = p.force_kernel == MI355_SDPA_KERNEL_MFMA_T256 ? 256
                         : p.force_kernel == MI355_SDPA_KERNEL_MFMA_T128 ? 128 : 0;
  // The kernels of fwd_mfma_w32.hip address K / V rows with 32-bit byte offsets from the start of
  // a (batch, head).  Head dim 128: 256-row workgroups (one per compute unit) once every compute
  // unit gets at least one (two when the causal mask makes half of them light) and the key loop
  // is long, 128-row workgroups (two per compute unit) for short or few sequences.  Head dim 64:
  // 128-row workgroups always (measured crossovers on MI355X).
  if ((int64_t)g.S * g.k_sl * 2 < (1ll << 31) && (int64_t)g.S * g.v_sl * 2 < (1ll << 31)) {
    const bool big = D == 128 && ((g.S >= 2048 && wg256 >= (g.causal ? 512 : 256)) || (!g.causal && g.S >= 1024 && wg256 >= 512));
    // (a short window: the keys a workgroup walks are window + rows, so smaller workgroups waste less:
    // B=2, S=4096, window 1024: 160 -> 144 us; window 2048: 208 -> 201; window 4096: 243 -> 249)
    const bool short_window = g.window > 0 && g.window <= 2048;
    // (with a tile skip table at head dim 128: 256 rows, whose LDS has room for the tile list at two
    // wavefronts per SIMD)
    const bool listed = g.live_tiles && D == 128;
    // (sorted document ids: a workgroup's keys are those of its rows' documents, again fewer for fewer rows:
    // 8 documents of 512 in S=4096, B=2: 75 -> 67 us; 4 of 1024: 98 -> 96)
    const bool packed = g.sm.doc_q && g.sm.doc_k && g.sm.doc_sorted;
    const int rows = D == 256 ? 128 : listed ? 256 : force_tile ? force_tile : (big && !short_window && !packed) ? 256 : 128;
    if (ws_only) return *ws_only = fwd_w32_workspace(g, D, rows / 32), MI355_SDPA_OK;
    return launch_fwd_mfma_w32(g, p.dtype, D, rows / 32, s);
  }
  if (ws_only) return MI355_SDPA_OK;
  // strides beyond 32-bit offsets: the kernel above (64-bit addressing)
  int NB = (D == 64 && (force_tile == 256 || (force_tile == 0 && wg256 >= 256 && g.S >= 2048))) ? 2 : 1;
  const int BM = 128 * NB;
  g.n_qt = (g.L + BM - 1) / BM;
  const int64_t blocks = (int64_t)g.B * g.Hq * g.n_qt;
  if (blocks == 0) return MI355_SDPA_OK;
  if (blocks > 0x7fffffff) {
    set_error("SDPA: too many query tiles (%lld)", (long long)blocks);
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  dim3 grid((unsigned)blocks), block(256);
  if (p.dtype == MI355_SDPA_BF16) {
    if (D == 128) hipLaunchKernelGGL((fwd_mfma_kernel<bf16_t, 128, 1>), grid, block, 0, s, g);
    else if (NB == 2) hipLaunchKernelGGL((fwd_mfma_kernel<bf16_t, 64, 2>), grid, block, 0, s, g);
    else hipLaunchKernelGGL((fwd_mfma_kernel<bf16_t, 64, 1>), grid, block, 0, s, g);
  } else {
    if (D == 128) hipLaunchKernelGGL((fwd_mfma_kernel<f16_t, 128, 1>), grid, block, 0, s, g);
    else if (NB == 2) hipLaunchKernelGGL((fwd_mfma_kernel<f16_t, 64, 2>), grid, block, 0, s, g);
    else hipLaunchKernelGGL((fwd_mfma_kernel<f16_t, 64, 1>), grid, block, 0, s, g);
  }
  return check_launch("fwd_mfma_kernel");
}

int launch_fwd_mfma(const mi355_sdpa_fwd_params& p, hipStream_t s) { return launch_or_size(p, s, nullptr); }

size_t fwd_mfma_workspace(const mi355_sdpa_fwd_params& p) {
  size_t bytes = 0;
  launch_or_size(p, nullptr, &bytes);
  return bytes;
}

}  // namespace mi355
