// Flash-attention forward for gfx950, head dim 128, bf16/f16: the variant for long sequences.
//
// One workgroup = 4 wavefronts = 256 query rows of one (batch, query head); ONE workgroup per
// compute unit, so a wavefront has the whole 512-register budget: 64 query rows (two 32-column
// blocks) per wavefront, O^T in the accumulation registers, keys in tiles of 32.
//
// Why 64 rows per wavefront: the kernel is bound by LDS bandwidth before it is bound by the
// matrix pipe.  Every 32x32x16 MFMA consumes a fresh 1 KB A operand (a K or V^T fragment) out
// of LDS, a compute unit delivers about 64 B/clk of LDS reads, and four SIMDs at full MFMA rate
// would ask for twice that.  Holding two query blocks per wavefront lets each fragment feed two
// MFMAs.
//
// With one wavefront per SIMD nothing hides latency but the instruction stream itself, so the
// key loop is software pipelined and its order pinned by hand (see `iteration` below): the
// softmax of a tile is split in two halves that ride on the matrix ops of two different phases,
// LDS operands are fetched three MFMA pairs ahead through a four-entry register ring, and a
// scheduling barrier after every MFMA pair keeps the compiler from regrouping the stream.  The
// vector unit, not the matrix pipe, is the scarce resource (v_exp_f32 alone costs half the
// matrix time), so the loop carries no row maximum at all: see kTrig.
// Products are computed transposed (S^T = K Q^T, O^T = V^T P^T) as in fwd_mfma.hip, so the
// softmax statistics are per-lane scalars and P goes from accumulator to B operand in registers.
//
// Numerics: torch_neuronx/_sdpa_math.py:51-95 (float32 accumulation and softmax, probabilities
// rounded to the input dtype for P*V only, dead rows give zeros and lse = -inf).
#include <type_traits>

#include "fwd_mfma.h"

namespace mi355 {
namespace {

constexpr int D = 128;
constexpr int BM = 256, BN = 32, NB = 2;
constexpr int KS = D / 16, DB = D / 32;
constexpr int KROW = D + 8;   // K tile row pitch (elements): conflict-free 128-bit reads
constexpr int VROW = BN + 8;  // V^T tile row pitch
constexpr int KCH = D / 8;    // 16-byte chunks per K row
constexpr float kLazy = 8.f;  // log2 headroom before the accumulator is rescaled

template <typename T>
__global__ __launch_bounds__(256, 1) void fwd_w64_kernel(FwdM p) {
  __shared__ __attribute__((aligned(16))) uint16_t k_lds[2][BN * KROW];
  __shared__ __attribute__((aligned(16))) uint16_t v_lds[2][D * VROW];

  int b, h, qt;
  decode_block(p, b, h, qt);
  const int hk = h / (p.Hq / p.Hkv);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int col = lane & 31, half = lane >> 5;
  const int q0 = qt * BM;
  const int qw0 = q0 + wave * 64;
  const int qrow[NB] = {qw0 + col, qw0 + 32 + col};
  const int qw_last = qw0 + 63;

  const uint16_t* qp = (const uint16_t*)p.q + b * p.q_sb + h * p.q_sh;
  const uint16_t* kp = (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh;
  const uint16_t* vp = (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh;

  u32x4 qf[NB][KS];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const uint16_t* qr = qp + (int64_t)min(qrow[nb], p.L - 1) * p.q_sl + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[nb][ks] = *(const u32x4*)(qr + ks * 16);
  }

  int nt = (p.S + BN - 1) / BN;
  if (p.causal) nt = min(nt, (min(q0 + BM, p.L) - 1) / BN + 1);
  const int nt_w = p.causal ? min(nt, qw_last / BN + 1) : nt;

  // ---- staging: every thread moves two 16-byte K chunks and a 4-key x 4-d block of V ----------
  // Two staging sets each: a tile is fetched from global memory two iterations before it is
  // written to LDS, so a fetch has about two tile times to land.
  u32x4 kreg[2][2];
  u32x2 vreg[2][4];
  const int k_chunk = tid & 15, k_row0 = tid >> 4;  // K rows k_row0, k_row0 + 16
  const int v_g = tid & 7, v_dq = tid >> 3;         // keys 4 v_g .. +3, d = 4 v_dq .. +3
  // K and V are read through buffer resources: the per-thread byte offset inside a tile is fixed
  // (one register each, set up once) and the tile offset is a scalar, so a fetch is a single
  // instruction with no address arithmetic on the vector unit.  S is a multiple of BN here (the
  // launcher guarantees it), so no row needs clamping.
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)kp, 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)vp, 0, 0x7fffffff, 0x00020000);
  uint32_t k_off[2], v_off[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) k_off[i] = (uint32_t)(((k_row0 + 16 * i) * p.k_sl + k_chunk * 8) * 2);
#pragma unroll
  for (int i = 0; i < 4; ++i) v_off[i] = (uint32_t)(((4 * v_g + i) * p.v_sl + v_dq * 4) * 2);
  const int k_tile_bytes = (int)(BN * p.k_sl * 2), v_tile_bytes = (int)(BN * p.v_sl * 2);
  auto load_k = [&](int set, int t) {
    const int base = min(t, nt - 1) * k_tile_bytes;
#pragma unroll
    for (int i = 0; i < 2; ++i) kreg[set][i] = __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, k_off[i], base, 0);
  };
  auto load_v = [&](int set, int t) {
    const int base = min(t, nt - 1) * v_tile_bytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) vreg[set][i] = __builtin_amdgcn_raw_buffer_load_b64(v_rsrc, v_off[i], base, 0);
  };
  auto store_k = [&](int set, int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      *(u32x4*)(&k_lds[buf][(k_row0 + 16 * i) * KROW + k_chunk * 8]) = kreg[set][i];
  };
  // transpose the 4x4 block with byte permutes: one 8-byte write of four keys per d
  auto store_v_half = [&](int set, int buf, int c) {  // dword c of each row holds d = 2c, 2c+1
    const int pos = tr_pos(v_g) * 4;
    const uint32_t a0 = vreg[set][0][c], a1 = vreg[set][1][c], a2 = vreg[set][2][c], a3 = vreg[set][3][c];
    u32x2 even, odd;
    even[0] = __builtin_amdgcn_perm(a1, a0, 0x05040100);
    even[1] = __builtin_amdgcn_perm(a3, a2, 0x05040100);
    odd[0] = __builtin_amdgcn_perm(a1, a0, 0x07060302);
    odd[1] = __builtin_amdgcn_perm(a3, a2, 0x07060302);
    const int d = v_dq * 4 + 2 * c;
    *(u32x2*)(&v_lds[buf][d * VROW + pos]) = even;
    *(u32x2*)(&v_lds[buf][(d + 1) * VROW + pos]) = odd;
  };

  f32x16 oacc[DB][NB];
#pragma unroll
  for (int i = 0; i < DB; ++i)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) zero(oacc[i][nb]);
  float m_run[NB] = {-INFINITY, -INFINITY}, l_run[NB] = {0.f, 0.f};
  const float c = p.scale * kLog2eF;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int lim[NB] = {p.causal ? min(qrow[0], p.S - 1) : p.S - 1, p.causal ? min(qrow[1], p.S - 1) : p.S - 1};

  auto mask_tile = [&](f32x16 (&s)[NB], int kv0) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kv = kv0 + (r >> 2) * 8 + half * 4 + (r & 3);
        if (kv > lim[nb]) s[nb][r] = -INFINITY;
      }
  };
  auto is_edge = [&](int kv0) { return (p.causal && kv0 + BN - 1 > qw0) || (kv0 + BN > p.S); };

  float m_new[NB] = {-INFINITY, -INFINITY}, mc[NB] = {0.f, 0.f}, alpha[NB] = {1.f, 1.f};
  bool need_rescale = false;
  auto tile_max = [&](const f32x16& s) {
    float t = fmaxf(s[0], s[1]);
#pragma unroll
    for (int r = 2; r < 16; r += 2) t = fmaxf(fmaxf(t, s[r]), s[r + 1]);  // v_max3
    return t;
  };
  // The softmax reference of a row (m_run, folded into mc) is NOT the running maximum.  The fast
  // path never looks for a maximum at all: probabilities are formed against the current reference
  // and only their sum is watched.  A lane's sum over its 16 keys above kTrig means that some
  // probability outgrew 2^kLazy-ish headroom (or that there is no reference yet): then, and only
  // then, the slow path finds the true tile maximum, raises the reference of every row that beat
  // it by more than kLazy in the exponent, rescales those rows' accumulators and redoes the
  // tile's probabilities.  Exact arithmetic: numerator and row sum always carry the same
  // reference, and lse = reference * scale + ln(sum).
  constexpr float kTrig = 8192.f;  // 16 probabilities of at most 2^kLazy stay below this
  auto raise_reference = [&](float t0, float t1) {
    const float tm[NB] = {fmaxf(t0, __shfl_xor(t0, 32, 64)), fmaxf(t1, __shfl_xor(t1, 32, 64))};
    bool moved = false;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      const bool up = (tm[nb] - m_run[nb]) * c > kLazy;  // false for NaN (-inf minus -inf)
      m_new[nb] = up ? tm[nb] : m_run[nb];
      const float m_use = (m_new[nb] == -INFINITY) ? 0.f : m_new[nb];
      moved |= up;
      alpha[nb] = __builtin_amdgcn_exp2f((m_run[nb] - m_use) * c);
      mc[nb] = m_use * c;
    }
    need_rescale = __builtin_amdgcn_ballot_w64(moved) != 0;
  };

  // Softmax of one register pair, in three stages so that consecutive pairs can be staggered by
  // hand (the chain read S -> fma -> exp2 -> add/pack is strictly dependent and a wavefront
  // issues in order).  Pair j of 16: query block j / 8, accumulator registers 2 (j % 8), +1.
  float xs[3][2], pv[2][2];
  auto stage1 = [&](const f32x16 (&sv)[NB], int j, int q) {
    const int nb = j >> 3, r = (j & 7) * 2;
    xs[q % 3][0] = fmaf(sv[nb][r], c, -mc[nb]);
    xs[q % 3][1] = fmaf(sv[nb][r + 1], c, -mc[nb]);
  };
  auto stage2 = [&](int q) {
    pv[q & 1][0] = __builtin_amdgcn_exp2f(xs[q % 3][0]);
    pv[q & 1][1] = __builtin_amdgcn_exp2f(xs[q % 3][1]);
  };
  auto stage3 = [&](int j, int q, uint32_t (&pk)[NB][8], float (&ps)[NB]) {
    const int nb = j >> 3, r = (j & 7) * 2;
    ps[nb] += pv[q & 1][0] + pv[q & 1][1];
    asm volatile("" : "+v"(ps[nb]));  // keeps the add in its slot (left alone it sinks below the loop body)
    pk[nb][r >> 1] = Mma<T>::pack(pv[q & 1][0], pv[q & 1][1]);
  };
  // The 16 pairs of a tile are split in two halves by key: pairs whose registers 0..7 hold the
  // tile's first 16 keys (the first contraction step of P*V) and those of the last 16 keys.
  auto early_pair = [](int q) { return q < 4 ? q : q + 4; };      // 0..3, 8..11
  auto late_pair = [](int q) { return q < 4 ? q + 4 : q + 8; };   // 4..7, 12..15

  // ---- prologue ----------------------------------------------------------------------------------
  load_k(0, 0);
  load_v(0, 0);
  load_k(1, 1);
  store_k(0, 0);
  store_v_half(0, 0, 0);
  store_v_half(0, 0, 1);
  store_k(1, 1);
  __syncthreads();
  load_k(0, 2);
  load_k(1, 3);
  load_v(1, 1);
  load_v(0, 2);
  f32x16 s_a[NB], s_b[NB];
  uint32_t pk_a[NB][8], pk_b[NB][8];
  float ps_a[NB] = {0.f, 0.f}, ps_b[NB] = {0.f, 0.f};
  bool first = true;  // no reference yet: the first tile goes through the slow path whatever its sums
  if (nt_w > 0) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const u32x4 a = *(const u32x4*)(&k_lds[0][col * KROW + ks * 16 + half * 8]);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        if (ks == 0) MmaV<T>::first(s_a[nb], a, qf[nb][ks]);
        else MmaV<T>::next(s_a[nb], a, qf[nb][ks]);
      }
    }
    mfma_to_valu_gap();
    if (is_edge(0)) mask_tile(s_a, 0);
#pragma unroll
    for (int q = 0; q < 8; ++q) {  // first half of tile 0 (redone by the slow path of iteration 0)
      stage1(s_a, early_pair(q), q);
      stage2(q);
      stage3(early_pair(q), q, pk_a, ps_a);
    }
  }
  __syncthreads();  // K buffer 0 is rewritten during the first iteration

  // One pipelined iteration.  On entry scur holds S^T of tile t and pk / ps the probabilities of its
  // first 16 keys; snext receives S^T of tile t+1 and pkn / psn the first half of ITS probabilities.
  //   phase A   S^T(t+1) = K(t+1) Q^T on the matrix pipe  |  softmax of the last 16 keys of tile t
  //   check     sums of tile t against kTrig; rare slow path
  //   phase B   O^T += V^T(t) P^T(t) on the matrix pipe    |  softmax of the first 16 keys of tile
  //             t+1, LDS stores of tiles t+2 / t+1, fetches of tiles t+4 / t+3
  auto iteration = [&](int t, auto parity, f32x16 (&scur)[NB], f32x16 (&snext)[NB], uint32_t (&pk)[NB][8],
                       uint32_t (&pkn)[NB][8], float (&ps)[NB], float (&psn)[NB]) {
    constexpr int par = decltype(parity)::value;  // t & 1, known at compile time
    const uint16_t* kt = &k_lds[par ^ 1][col * KROW + half * 8];
    const uint16_t* vt = &v_lds[par][col * VROW + half * 8];
    auto read_k = [&](int ks) { return *(const u32x4*)(kt + ks * 16); };
    auto read_v = [&](int i) { return *(const u32x4*)(vt + (i & 3) * 32 * VROW + (i >> 2) * 16); };
    u32x4 ring[4];
    __builtin_amdgcn_sched_barrier(0);
    // the first operand fetches are in flight while the first probabilities are formed
    ring[0] = read_k(0), ring[1] = read_k(1), ring[2] = read_k(2);
    stage1(scur, late_pair(0), 0);
    stage1(scur, late_pair(1), 1);
    stage2(0);
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase A -------------------------------------------------------------------------------
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + 3 < KS) ring[(ks + 3) & 3] = read_k(ks + 3);
      else ring[(ks + 3) & 3] = read_v(ks + 3 - KS);
      if (ks == 0) MmaV<T>::first(snext[0], ring[ks & 3], qf[0][ks]);
      else MmaV<T>::next(snext[0], ring[ks & 3], qf[0][ks]);
      if (ks + 2 < 8) stage1(scur, late_pair(ks + 2), ks + 2);
      if (ks + 1 < 8) stage2(ks + 1);
      if (ks == 0) MmaV<T>::first(snext[1], ring[ks & 3], qf[1][ks]);
      else MmaV<T>::next(snext[1], ring[ks & 3], qf[1][ks]);
      stage3(late_pair(ks), ks, pk, ps);
      __builtin_amdgcn_sched_barrier(0);
    }
    mfma_to_valu_gap();  // snext is read (and, on the diagonal, masked) from here on
    // ---- check ---------------------------------------------------------------------------------
    const bool trig = first || !(ps[0] <= kTrig) || !(ps[1] <= kTrig);  // (NaN also lands here)
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(trig) != 0, 0)) {
      first = false;
      raise_reference(tile_max(scur[0]), tile_max(scur[1]));
      if (need_rescale) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          l_run[nb] *= alpha[nb];
#pragma unroll
          for (int i = 0; i < DB; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              // read and write-back are pinned to accumulation registers one element at a time; left
              // to itself the compiler drags all 128 accumulators through the general registers at
              // once, which evicts the query fragments from them for the whole loop
              float xv, y;
              asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(xv) : "a"(oacc[i][nb][r]));
              y = xv * alpha[nb];
              asm volatile("" : "+a"(y));
              oacc[i][nb][r] = y;
            }
            __builtin_amdgcn_sched_barrier(0);  // one accumulator block at a time
          }
          m_run[nb] = m_new[nb];
        }
      }
      ps[0] = 0.f, ps[1] = 0.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) {  // the whole tile again, against the new reference
        stage1(scur, j, j);
        stage2(j);
        stage3(j, j, pk, ps);
      }
    }
    l_run[0] += ps[0], l_run[1] += ps[1];
    if (__builtin_expect(is_edge((t + 1) * BN), 0)) mask_tile(snext, (t + 1) * BN);  // rare
    psn[0] = 0.f, psn[1] = 0.f;
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase B -------------------------------------------------------------------------------
    // (the softmax pipeline of tile t+1 fills and drains under the matrix ops: nothing of it runs
    // between the phases, where the matrix pipe would sit idle)
#pragma unroll
    for (int i = 0; i < 8; ++i) {  // i = 4 * (16-key step) + d block
      if (i + 3 < 8) ring[(i + 3 + KS) & 3] = read_v(i + 3);
      const int ks2 = i >> 2, db = i & 3;
      const u32x4 b0 = {pk[0][ks2 * 4], pk[0][ks2 * 4 + 1], pk[0][ks2 * 4 + 2], pk[0][ks2 * 4 + 3]};
      const u32x4 b1 = {pk[1][ks2 * 4], pk[1][ks2 * 4 + 1], pk[1][ks2 * 4 + 2], pk[1][ks2 * 4 + 3]};
      oacc[db][0] = Mma<T>::run(ring[(i + KS) & 3], b0, oacc[db][0]);
      stage1(snext, early_pair(i), i);
      if (i >= 1) stage2(i - 1);
      if (i == 0) store_k(par, par);  // tile t+2
      if (i == 2) store_v_half(par ^ 1, par ^ 1, 0);  // tile t+1
      if (i == 6) load_k(par, t + 4);
      oacc[db][1] = Mma<T>::run(ring[(i + KS) & 3], b1, oacc[db][1]);
      if (i >= 2) stage3(early_pair(i - 2), i - 2, pkn, psn);
      if (i == 4) store_v_half(par ^ 1, par ^ 1, 1);
      if (i == 7) load_v(par ^ 1, t + 3);
      __builtin_amdgcn_sched_barrier(0);
    }
    stage2(7);
    stage3(early_pair(6), 6, pkn, psn);
    stage3(early_pair(7), 7, pkn, psn);
    __syncthreads();
  };
  // a wavefront whose rows lie above the causal diagonal of the remaining tiles only feeds LDS
  auto idle_step = [&](int t, auto parity) {
    constexpr int par = decltype(parity)::value;
    store_k(par, par);
    store_v_half(par ^ 1, par ^ 1, 0);
    store_v_half(par ^ 1, par ^ 1, 1);
    load_k(par, t + 4);
    load_v(par ^ 1, t + 3);
    __syncthreads();
  };

  int t = 0;
  for (; t + 1 < nt_w; t += 2) {
    iteration(t, std::integral_constant<int, 0>{}, s_a, s_b, pk_a, pk_b, ps_a, ps_b);
    iteration(t + 1, std::integral_constant<int, 1>{}, s_b, s_a, pk_b, pk_a, ps_b, ps_a);
  }
  if (t < nt_w) {  // odd count: t is even here
    iteration(t, std::integral_constant<int, 0>{}, s_a, s_b, pk_a, pk_b, ps_a, ps_b);
    ++t;
  }
  for (; t < nt; ++t) {
    if (t & 1) idle_step(t, std::integral_constant<int, 1>{});
    else idle_step(t, std::integral_constant<int, 0>{});
  }

  // ---- epilogue ------------------------------------------------------------------------------------
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

int launch_fwd_mfma_w64(const FwdM& g, int dtype, hipStream_t s) {
  const int64_t blocks = (int64_t)g.B * g.Hq * g.n_qt;
  dim3 grid((unsigned)blocks), block(256);
  if (dtype == MI355_SDPA_BF16) hipLaunchKernelGGL((fwd_w64_kernel<bf16_t>), grid, block, 0, s, g);
  else hipLaunchKernelGGL((fwd_w64_kernel<f16_t>), grid, block, 0, s, g);
  return check_launch("fwd_w64_kernel");
}

}  // namespace mi355
