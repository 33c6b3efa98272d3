// Decode-step attention over an fp8 (OCP e4m3) K/V cache for gfx950: split-KV flash decoding
// on the 16x16x32 fp8 MFMA, streaming K and V straight from HBM into registers (no LDS on
// the hot path).  Defined as torch_neuronx/_sdpa_math.py:51-95 applied to the dequantised
// cache with a key-padding bias; the reference itself has no fp8 attention path.
//
// Work split: the live keys of all (batch, kv head) pairs, in steps of 32 keys, form one long
// list which is cut into equal contiguous ranges, one per wavefront; the wavefront serves all
// R = Lq * Hq/Hkv query rows that share a kv head, so every K/V byte is read from HBM exactly
// once, and padding past kv_lens[b] is never read.  A wavefront walks its range 32 keys at a
// time with a running max / sum / output, writes one partial result per (batch, kv head) it
// touched, and a second small kernel merges the partials of a sequence.
//
// Precision without dequantising the cache: the query row is scaled by a power of two and split
// into e4m3 terms (q = q0 + q1 + ..., four significant bits each).  Up to four terms occupy
// separate columns of the 16-wide MFMA N dimension, which would otherwise idle, and are summed after
// the product; when the query rows of a kv head leave no room for that many (more than 4 rows: two
// terms per matrix op, more than 8: one), the remaining terms go through the matrix ops a second
// (third, fourth) time into the same accumulators - the pipe is a fraction busy in this kernel.  A
// bf16 query (8 significant bits) is exact in two terms and gets two or three, a float16 query (11)
// gets three or four, a float32 query four (16 bits).  The probabilities are split the same way
// before P*V.
//
// Head dims 64, 128 and 256 are instances of one kernel; the description is for 128.
// Per 32 keys a lane loads two 16-byte pieces of each of two keys (A operand of S^T = K Q^T; the
// contraction order is permuted identically for Q) and eight 8-byte pieces of V, one from each
// of eight keys, which are byte-transposed in registers into the A operand of O^T = V^T P^T
// (head dim 64: one piece per key and 4-byte pieces of V; 256: four and 16-byte pieces).
// Every load is non-temporal (the cache is read once) and a V instruction covers four whole
// 128-byte rows: with plain loads the stream reads 5.8 TB/s whatever the shape, with
// non-temporal ones 5.8 TB/s when a row is fetched in two instructions and 6.5 TB/s when in one
// (measured with a memory-only model of this kernel's work split).
#include <algorithm>
#include <atomic>
#include <type_traits>

#include "common.h"

// Scratch of the entry point that allocates nothing (mi355_sdpa_decode_fp8kv_static): partial
// results and step counts of one decode call.  Every GPU the library runs on holds its own copy
// until the process ends.  In host code this name is only a handle for hipGetSymbolAddress; the
// device address it yields, kept per device, is what kernels and copies are given.
static __device__ __align__(256) unsigned char scratch[MI355_SDPA_DECODE_STATIC_SCRATCH_BYTES];

namespace mi355 {
namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
// wavefronts per SIMD the decode kernel is built for (at head dims up to 128 three or four spill; at 256
// the two K/V tiles in flight and the output accumulators alone take 190 registers: one)
constexpr int dec_occ(int D) { return D > 128 ? 1 : 2; }
constexpr int kMaxSimds = 1024;  // bound on the streaming kernel's grid: wavefronts per SIMD it is built for x this; sizes the workspace
constexpr float kPScale = 256.f;  // probabilities are stored as e4m3 of 256*p

struct DecP {
  const void* q;
  const uint8_t *k, *v;
  const float *k_scale, *v_scale;
  const int32_t* kv_lens;
  void* out;
  float* lse;
  float* ws_o;        // (slots,R,D) partial outputs; slot = b*Hkv + hk + wavefront index
  float* ws_ml;       // (slots,R,2)   partial (max, sum)
  int32_t* ws_steps;  // (B+1) exclusive prefix of the 32-key step counts per batch, then the total
  int64_t q_sb, q_sh, q_sl;
  int64_t k_sb, k_sh, k_sl;
  int64_t v_sb, v_sh, v_sl;
  int64_t o_sb, o_sh, o_sl;
  int B, Hq, Hkv, Lq, S, R;
  int n_waves;  // wavefronts of the streaming kernel
  int t_min;    // least number of steps per wavefront
  float scale;
};

__device__ __forceinline__ uint32_t fp8x2(float a, float b) {
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}
__device__ __forceinline__ f32x2 fp8x2_to_f32(uint32_t w) {
  return __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
}

// The split x = t0 + t1 + t2 into e4m3 terms for a pair of values; each lane keeps one term, picked
// with the lane's masks (0xffff for its own term, 0 elsewhere; all 0 for a dead column).  Written
// without branches: every lane computes all terms, which costs less than divergent control flow.
// Term number PARTS * pass + j goes to the lanes of column group j in pass `pass`.
struct PartMask { uint32_t m[4]; };
template <int PARTS, int PASSES>
__device__ __forceinline__ void split_pair(float a, float b, const PartMask& pm, uint32_t (&w)[PASSES]) {
#pragma unroll
  for (int ps = 0; ps < PASSES; ++ps) {
    w[ps] = 0u;
#pragma unroll
    for (int j = 0; j < PARTS; ++j) {
      const uint32_t t = fp8x2(a, b);
      w[ps] |= t & pm.m[j];
      if (ps * PARTS + j + 1 < PARTS * PASSES) {
        const f32x2 d = fp8x2_to_f32(t);
        a -= d[0], b -= d[1];
      }
    }
  }
}

// x + (x rotated right by N lanes inside each row of 16 lanes): one VALU op with a DPP modifier
template <int N>
__device__ __forceinline__ float add_row_ror(float x) {
  const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 | N, 0xf, 0xf, false);
  return x + __builtin_bit_cast(float, r);
}
// sum over the split-term columns n, n+RS, ... of a 16-lane row (all lanes get the total)
template <int PARTS>
__device__ __forceinline__ float sum_parts(float x) {
  if (PARTS == 1) return x;
  if (PARTS >= 3) x = add_row_ror<4>(x);  // (three terms: the fourth column group is dead and adds zeros)
  return add_row_ror<8>(x);
}

__device__ __forceinline__ long as_long(uint32_t lo, uint32_t hi) {
  return (long)(((uint64_t)hi << 32) | lo);
}

typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
// Head dims 64, 128 and 256: a K row is D/64 pieces of 64 bytes, of which lane group g takes 16 each
// (two contraction steps of 32 per piece); a V row is 16 pieces of D/16 bytes, one per lane n.
template <int D>
struct KVRegs {
  u32x4 k[2][D / 64];     // [16-key block][piece pc]: d = 64 pc + 16g .. +15 of the lane's key
  uint32_t v[8][D / 64];  // [key slot s]: d = (D/16) n .. +D/16-1 of key 4s + g, as dwords
};

// Steps per wavefront for a work list of `total` steps: equal shares, but not so small that the
// partial results outweigh the keys read.
__device__ __forceinline__ int steps_per_wave(int total, int n_waves, int t_min) {
  return max(t_min, (total + n_waves - 1) / n_waves);
}

// One workgroup = one wavefront, launched once per wavefront slot of the chip.  The work list is
// never materialised: step number G = (steps of batches < b) * Hkv + hk * steps(b) + s, so the
// steps of one (batch, kv head) are contiguous; wavefront w owns [w*T, (w+1)*T).  A wavefront
// prefix-sums the step counts of 64 batches at a time across its lanes and finds the batch of a
// step with a ballot.  An item is the part of one (batch, kv head) inside the wavefront's range.
// While an item streams, the query rows of the next one are already in flight (they wait in
// registers), and its first K/V tile is requested before the epilogue of the current one, so the
// memory pipe of a wavefront never drains between items.
template <typename TQ, int D, int PARTS, int PASSES>
__global__ __launch_bounds__(64, dec_occ(D)) void decode_kernel(DecP p) {
  constexpr int RS = PARTS >= 3 ? 4 : PARTS == 2 ? 8 : 16;  // column stride between split terms
  constexpr int NPC = D / 64;               // 64-byte pieces of a K row = dwords of a lane's V piece
  constexpr int KST = D / 32;               // contraction steps of S^T = K Q^T
  constexpr int PB = D / 16;                // bytes of a lane's V piece = output rows per lane n
  constexpr int LPP = (int)sizeof(TQ);      // 16-byte loads per 16 query elements (one piece of the lane)
  constexpr int QV = NPC * LPP;             // 16-byte loads of the lane's D/4 query elements
  const int lane = threadIdx.x;
  const int n = lane & 15, g = lane >> 4;
  const int part = n / RS, r = n % RS;
  const int rep = p.Hq / p.Hkv;
  const bool col_live = r < p.R && part < PARTS;
  const PartMask pm = {{col_live && part == 0 ? 0xffffu : 0u, col_live && part == 1 ? 0xffffu : 0u,
                        col_live && part == 2 ? 0xffffu : 0u, col_live && part == 3 ? 0xffffu : 0u}};
  const int rr = min(r, p.R - 1);
  const int hq_off = rr % rep, lq = rr / rep;

  // ---- the work list ------------------------------------------------------------------------------
  // Lane i of a block of 64 batches holds the batch's length, its step count and the inclusive
  // prefix of the counts.  Wavefront 0 also leaves the prefix sums for the merge kernel.
  auto block_counts = [&](int b0, int& len, int& cnt, int& incl) {
    const int bb = b0 + lane;
    len = 0;
    if (bb < p.B) len = p.kv_lens ? min(p.S, max(0, p.kv_lens[bb])) : p.S;
    cnt = (len + 31) >> 5;
    incl = cnt;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
  };
  const bool scribe = blockIdx.x == 0;
  int len0, cnt0, incl0;  // block 0 stays in registers: batches <= 64 never reload
  block_counts(0, len0, cnt0, incl0);
  if (scribe && lane < p.B) p.ws_steps[lane] = incl0 - cnt0;
  int seq_steps = __builtin_amdgcn_readlane(incl0, 63);
  for (int b0 = 64; b0 < p.B; b0 += 64) {
    int l, c, i;
    block_counts(b0, l, c, i);
    if (scribe && b0 + lane < p.B) p.ws_steps[b0 + lane] = seq_steps + i - c;
    seq_steps += __builtin_amdgcn_readlane(i, 63);
  }
  if (scribe && lane == 0) p.ws_steps[p.B] = seq_steps;
  const int total = seq_steps * p.Hkv;
  const int T = steps_per_wave(total, p.n_waves, p.t_min);
  const int g_first = blockIdx.x * T, g_end = min(total, g_first + T);
  if (g_first >= total) return;

  struct Item { int b, hk, begin, end, steps, slot; float kscale, vscale; };
  int cur_b0 = 0, cur_pref = 0;  // block cursor: items only move forward
  auto decode_item = [&](int G) {  // the item that starts at step G, g_first <= G < g_end
    Item it;
    int len = len0, cnt = cnt0, incl = incl0;
    if (cur_b0 != 0) block_counts(cur_b0, len, cnt, incl);
    while (G >= (cur_pref + __builtin_amdgcn_readlane(incl, 63)) * p.Hkv && cur_b0 + 64 < p.B) {
      cur_pref += __builtin_amdgcn_readlane(incl, 63);
      cur_b0 += 64;
      block_counts(cur_b0, len, cnt, incl);
    }
    // first batch whose steps end beyond G (a batch without steps never is the first)
    const uint64_t hit = __ballot((cur_pref + incl) * p.Hkv > G);
    const int ln = __builtin_ctzll(hit);
    const int nb = __shfl(cnt, ln, 64);                                  // steps of a kv head of this batch
    const int rem = G - (cur_pref + __shfl(incl - cnt, ln, 64)) * p.Hkv;  // steps into the batch
    const int hk = rem / nb, s0 = rem - hk * nb;
    const int ns = max(1, min(nb - s0, g_end - G));  // (never below 1: the walk always advances)
    it.b = __builtin_amdgcn_readfirstlane(cur_b0 + ln);
    it.hk = __builtin_amdgcn_readfirstlane(hk);
    it.steps = __builtin_amdgcn_readfirstlane(ns);
    it.begin = __builtin_amdgcn_readfirstlane(s0 * 32);
    it.end = __builtin_amdgcn_readfirstlane(min(__shfl(len, ln, 64), (s0 + ns) * 32));
    it.slot = it.b * p.Hkv + it.hk + blockIdx.x;
    // fetched here, ahead of the item's query and tiles, so that their use waits on nothing younger
    it.kscale = p.k_scale[it.b * p.Hkv + it.hk];
    it.vscale = p.v_scale[it.b * p.Hkv + it.hk];
    return it;
  };

  typedef __attribute__((ext_vector_type(4))) uint32_t qraw_t;
  qraw_t qraw[QV];  // the 32 query elements of this lane for the item fetched last, as loaded
  auto fetch_q = [&](const Item& it) {
    const TQ* qr = (const TQ*)p.q + it.b * p.q_sb + (it.hk * rep + hq_off) * p.q_sh + lq * p.q_sl + 16 * g;
#pragma unroll
    for (int i = 0; i < QV; ++i)
      qraw[i] = *(const qraw_t*)((const char*)(qr + 64 * (i / LPP)) + 16 * (i % LPP));
  };

  KVRegs<D> ra, rb;
  // Which key is which: the score tile of a 16-key block leaves the matrix op with rows 4g .. 4g+3
  // in lane group g, and the second product wants lane group g to hold the probabilities of the keys
  // whose V pieces it loaded, 4s + g for s = 0 .. 7.  So row m of block blk is key 16 blk + 4 (m % 4)
  // + m / 4: accumulator register i of block blk in lane group g is key 16 blk + 4 i + g, slot s = 4 blk + i.
  auto load = [&](KVRegs<D>& R_, const Item& it, int step) {
    const uint8_t* kp = p.k + it.b * p.k_sb + it.hk * p.k_sh;
    const uint8_t* vp = p.v + it.b * p.v_sb + it.hk * p.v_sh;
    const int base = it.begin + step * 32, last = it.end - 1;
    const int ksl = (int)p.k_sl, vsl = (int)p.v_sl;  // host checked: a (batch, head) slab spans < 2^31 bytes
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      const int row = min(base + blk * 16 + 4 * (n & 3) + (n >> 2), last);
      const uint8_t* kr = kp + (uint32_t)(row * ksl + 16 * g);
#pragma unroll
      for (int pc = 0; pc < NPC; ++pc) R_.k[blk][pc] = __builtin_nontemporal_load((const u32x4*)(kr + 64 * pc));
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int row = min(base + 4 * s + g, last);
      const uint8_t* vr = vp + (uint32_t)(row * vsl + PB * n);
      if constexpr (NPC == 1) {
        R_.v[s][0] = __builtin_nontemporal_load((const uint32_t*)vr);
      } else if constexpr (NPC == 2) {
        const u32x2 w = __builtin_nontemporal_load((const u32x2*)vr);
        R_.v[s][0] = w[0], R_.v[s][1] = w[1];
      } else {
        const u32x4 w = __builtin_nontemporal_load((const u32x4*)vr);
        R_.v[s][0] = w[0], R_.v[s][1] = w[1], R_.v[s][2] = w[2], R_.v[s][3] = w[3];
      }
    }
  };

  // Query fragment of the item fetched last: B operand of S^T = K Q^T.
  // The lane owns d = 64 pc + 16g .. +15 of row r for every piece pc, as for K; MFMA steps 2 pc and
  // 2 pc + 1 consume piece pc.
  // Returns the factor that turns a raw fp8 dot product into a log2-domain logit.
  auto convert_q = [&](const Item& it, long (&qb)[PASSES][KST]) -> float {
    float qv[D / 4];
    {
      typedef __attribute__((ext_vector_type(16 / sizeof(TQ)))) TQ qvec_t;
      constexpr int PER = 16 / sizeof(TQ);
#pragma unroll
      for (int i = 0; i < QV; ++i) {
        const qvec_t v = __builtin_bit_cast(qvec_t, qraw[i]);
#pragma unroll
        for (int e = 0; e < PER; ++e) qv[i * PER + e] = (float)v[e];
      }
    }
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < D / 4; ++i) amax = fmaxf(amax, fabsf(qv[i]));
    amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
    // power-of-two pre-scale so the row peaks in [120, 240]: well inside e4m3 and exact
    const float f = amax > 0.f ? __builtin_amdgcn_exp2f(floorf(__builtin_amdgcn_logf(240.f / amax))) : 1.f;
#pragma unroll
    for (int ks = 0; ks < KST; ++ks) {
      uint32_t w[4][PASSES];
#pragma unroll
      for (int jq = 0; jq < 4; ++jq)
        split_pair<PARTS, PASSES>(qv[ks * 8 + 2 * jq] * f, qv[ks * 8 + 2 * jq + 1] * f, pm, w[jq]);
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) qb[ps][ks] = as_long(w[0][ps] | (w[1][ps] << 16), w[2][ps] | (w[3][ps] << 16));
    }
    return p.scale * it.kscale / f * kLog2e;
  };

  int G = g_first;
  Item cur = decode_item(G);
  fetch_q(cur);
  load(ra, cur, 0);
  long qb[PASSES][KST];
  float c_row = convert_q(cur, qb);

  while (true) {
    // the next item: its query rows travel while this one streams
    const int g_next = G + cur.steps;
    const bool more = g_next < g_end;
    Item nxt = cur;
    if (more) {
      nxt = decode_item(g_next);
      fetch_q(nxt);
    } else {
      nxt.begin = cur.end - 1;  // no next item: the unconditional tile request below re-reads one cached row
    }

    f32x4 oacc[PB];
#pragma unroll
    for (int i = 0; i < PB; ++i) oacc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    const int w_end = cur.end;

    auto compute = [&](const KVRegs<D>& R_, int step) {
      const int base = cur.begin + step * 32;
      // S^T = K Q^T : rows = 16 keys of a block, columns = (split term, query row)
      f32x4 sacc[2];
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        sacc[blk] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KST; ++ks) {
          const u32x4 kk = R_.k[blk][ks >> 1];
          const long a = as_long(kk[(ks & 1) * 2], kk[(ks & 1) * 2 + 1]);
#pragma unroll
          for (int ps = 0; ps < PASSES; ++ps) sacc[blk] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a, qb[ps][ks], sacc[blk], 0, 0, 0);
        }
      }
      float t[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float x = sum_parts<PARTS>(sacc[i >> 2][i & 3]);
        const int key = base + (i >> 2) * 16 + 4 * (i & 3) + g;
        t[i] = key < w_end ? x * c_row : -INFINITY;
      }
      float tmax = t[0];
#pragma unroll
      for (int i = 1; i < 8; ++i) tmax = fmaxf(tmax, t[i]);
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(m_run, tmax);  // finite: every step holds at least one live key
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      m_run = m_new;
      float pv[8], psum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        pv[i] = __builtin_amdgcn_exp2f(t[i] - m_new);
        psum += pv[i];
      }
      l_run = l_run * alpha + psum;
#pragma unroll
      for (int i = 0; i < PB; ++i) oacc[i] *= alpha;
      // P^T (B operand): key slot s of this lane is key 4 s + g, the order V is loaded in
      uint32_t pw[4][PASSES];
#pragma unroll
      for (int jq = 0; jq < 4; ++jq)
        split_pair<PARTS, PASSES>(pv[2 * jq] * kPScale, pv[2 * jq + 1] * kPScale, pm, pw[jq]);
      long pb[PASSES];
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) pb[ps] = as_long(pw[0][ps] | (pw[1][ps] << 16), pw[2][ps] | (pw[3][ps] << 16));
      // O^T += V^T P^T : the lane holds bytes d = PB n + e (e = 0 .. PB-1) of its eight keys; matrix op e
      // takes byte e of every key (rows d = PB n + e), an 8 x PB byte transpose done as 4 x 4 ones
#pragma unroll
      for (int hf = 0; hf < NPC; ++hf) {  // e = 4 hf .. 4 hf + 3: dword hf of every piece
        uint32_t o_lo[4], o_hi[4];      // [e % 4]: key slots 0 .. 3 / 4 .. 7
#pragma unroll
        for (int q4 = 0; q4 < 2; ++q4) {
          const uint32_t w0 = R_.v[q4 * 4 + 0][hf], w1 = R_.v[q4 * 4 + 1][hf];
          const uint32_t w2 = R_.v[q4 * 4 + 2][hf], w3 = R_.v[q4 * 4 + 3][hf];
          const uint32_t t0 = __builtin_amdgcn_perm(w1, w0, 0x05010400);
          const uint32_t t1 = __builtin_amdgcn_perm(w1, w0, 0x07030602);
          const uint32_t t2 = __builtin_amdgcn_perm(w3, w2, 0x05010400);
          const uint32_t t3 = __builtin_amdgcn_perm(w3, w2, 0x07030602);
          uint32_t* o = q4 ? o_hi : o_lo;
          o[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100);
          o[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302);
          o[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100);
          o[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302);
        }
#pragma unroll
        for (int jq = 0; jq < 4; ++jq)
#pragma unroll
          for (int ps = 0; ps < PASSES; ++ps)
            oacc[hf * 4 + jq] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(
                as_long(o_lo[jq], o_hi[jq]), pb[ps], oacc[hf * 4 + jq], 0, 0, 0);
      }
    };

    const int steps = cur.steps;  // >= 1: an item is never empty
    // Loads are issued unconditionally (rows past the item's end clamp to its last key, a cache
    // hit) so that the count of loads in flight at every wait is the same on all paths.
    int s = 0;
    do {  // (a do-while: the compiler then knows that a tile was requested after the next query)
      load(rb, cur, s + 1);
      __builtin_amdgcn_sched_barrier(0);  // keep every tile's loads ahead of the work they overlap
      compute(ra, s);
      __builtin_amdgcn_sched_barrier(0);
      const bool stay = s + 2 < steps;  // else: the next item's first tile, in flight during the epilogue
      load(ra, stay ? cur : nxt, stay ? s + 2 : 0);
      __builtin_amdgcn_sched_barrier(0);
      if (s + 1 < steps) compute(rb, s + 1);
      s += 2;
    } while (s < steps);
    // all tiles of this item are consumed; what is in flight is the next item's first tile, and
    // its query rows landed long ago: build its fragment now, ahead of the stores below
    long qb_next[PASSES][KST];
    float c_next = 0.f;
    if (more) c_next = convert_q(nxt, qb_next);

    // ---- merge the split terms and emit this item's partial result -------------------------------
#pragma unroll
    for (int i = 0; i < PB; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) oacc[i][e] = sum_parts<PARTS>(oacc[i][e]);
    float l_tot = l_run + __shfl_xor(l_run, 16, 64);
    l_tot += __shfl_xor(l_tot, 32, 64);
    if (n < p.R) {  // split term 0 lanes of live rows
      const float vscale = cur.vscale * (1.f / kPScale);
      const int64_t slot = (int64_t)cur.slot * p.R + n;
      if (g == 0) p.ws_ml[slot * 2] = m_run, p.ws_ml[slot * 2 + 1] = l_tot;
      // (register a of matrix op e is row d = PB (4g + a) + e of O^T)
      float* dst = p.ws_o + slot * D + 4 * PB * g;
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int e4 = 0; e4 < NPC; ++e4)
          *(f32x4*)(dst + PB * a + 4 * e4) = f32x4{oacc[4 * e4][a], oacc[4 * e4 + 1][a], oacc[4 * e4 + 2][a], oacc[4 * e4 + 3][a]} * vscale;
    }
    if (!more) break;
    G = g_next;
    cur = nxt;
    c_row = c_next;
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
      for (int ks = 0; ks < KST; ++ks) qb[ps][ks] = qb_next[ps][ks];
  }
}

// Merge the partials of one (batch, kv head, query row); D threads = D output columns.
// The wavefronts that touched this (batch, kv head) follow from the step numbering alone, and
// their partials sit in consecutive slots.
template <typename TQ, int D>
__global__ __launch_bounds__(D) void decode_merge_kernel(DecP p) {
  constexpr int NW = D / 64;  // wavefronts of the workgroup
  __shared__ float s_red[2][4];
  __shared__ float w_s[kMaxSimds * 2];  // weights of the partials (at most one per wavefront of the streaming kernel)
  const int row = blockIdx.x % p.R;
  const int hk = (blockIdx.x / p.R) % p.Hkv;
  const int b = blockIdx.x / (p.R * p.Hkv);
  const int d = threadIdx.x;
  const int pref = p.ws_steps[b], nb = p.ws_steps[b + 1] - pref;
  const int T = steps_per_wave(p.ws_steps[p.B] * p.Hkv, p.n_waves, p.t_min);
  const int g0 = pref * p.Hkv + hk * nb;
  const int w0 = g0 / T;
  const int npart = nb > 0 ? (g0 + nb - 1) / T - w0 + 1 : 0;
  const int64_t slot0 = (int64_t)(b * p.Hkv + hk + w0) * p.R + row;  // partial c sits at slot0 + c*R
  float M = -INFINITY, L = 0.f, O = 0.f;
  constexpr int kFew = 8;
  if (npart <= kFew) {
    // few partials: fetch every (max, sum) pair and output value at once, then combine; each
    // thread repeats the scalar part, which costs less than a second round trip to memory
    float m[kFew], l[kFew], o[kFew];
#pragma unroll
    for (int c = 0; c < kFew; ++c) {
      const int64_t s = slot0 + (int64_t)min(c, max(npart - 1, 0)) * p.R;
      const bool live = c < npart;
      m[c] = live ? p.ws_ml[s * 2] : -INFINITY;
      l[c] = live ? p.ws_ml[s * 2 + 1] : 0.f;
      o[c] = live ? p.ws_o[s * D + d] : 0.f;
    }
#pragma unroll
    for (int c = 0; c < kFew; ++c) M = fmaxf(M, m[c]);
#pragma unroll
    for (int c = 0; c < kFew; ++c) {
      const float w = c < npart ? __builtin_amdgcn_exp2f(m[c] - M) : 0.f;
      L = fmaf(l[c], w, L);
      O = fmaf(o[c], w, O);
    }
  } else {
    // many partials (a long sequence in a small batch: up to one per wavefront of the chip): their
    // (max, sum) pairs a thread each, the weights left in LDS, and the partial outputs requested eight
    // at a time - read one after the other, 256 partials were 256 trips to the L2 in a row, and a
    // single sequence of 32768 keys spent two thirds of its decode step here
    for (int c = d; c < npart; c += D) M = fmaxf(M, p.ws_ml[(slot0 + (int64_t)c * p.R) * 2]);
    M = wave_max(M);
    if ((d & 63) == 0) s_red[0][d >> 6] = M;
    __syncthreads();
    M = s_red[0][0];
#pragma unroll
    for (int w = 1; w < NW; ++w) M = fmaxf(M, s_red[0][w]);
    for (int c = d; c < npart; c += D) {
      const int64_t s = slot0 + (int64_t)c * p.R;
      const float w = __builtin_amdgcn_exp2f(p.ws_ml[s * 2] - M);
      w_s[c] = w;
      L += p.ws_ml[s * 2 + 1] * w;
    }
    L = wave_sum(L);
    if ((d & 63) == 0) s_red[1][d >> 6] = L;
    __syncthreads();
    L = s_red[1][0];
#pragma unroll
    for (int w = 1; w < NW; ++w) L += s_red[1][w];
    const float* po = p.ws_o + slot0 * D + d;
    const int64_t stride = (int64_t)p.R * D;
    for (int c0 = 0; c0 < npart; c0 += 8) {
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = c0 + j < npart ? po[(c0 + j) * stride] : 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) O = fmaf(o[j], c0 + j < npart ? w_s[c0 + j] : 0.f, O);
    }
  }
  const int rep = p.Hq / p.Hkv;
  const int h = hk * rep + row % rep, lq = row / rep;
  TQ* o = (TQ*)p.out + b * p.o_sb + h * p.o_sh + lq * p.o_sl;
  o[d] = (TQ)(L > 0.f ? O / L : 0.f);
  if (p.lse && d == 0)
    p.lse[((int64_t)b * p.Hq + h) * p.Lq + lq] = L > 0.f ? (M + __builtin_amdgcn_logf(L)) * kLn2 : -INFINITY;
}

constexpr int kMinSteps = 4;     // 128 keys: below this the partial results rival the keys in bytes

int wave_slots(int head_dim) {  // wavefronts of the decode kernel the chip holds at once
  static int simds = 0;
  if (!simds) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0)
      simds = cus * 4;
    else
      simds = 256 * 4;
  }
  return std::min(simds, kMaxSimds) * dec_occ(head_dim);
}

// least steps per wavefront: num_splits > 0 asks for at most about that many pieces per sequence
int min_steps_for(const mi355_sdpa_decode_params& p) {
  const int64_t seq_steps = (p.k.size[2] + 31) / 32;
  int t = kMinSteps;
  if (p.num_splits > 0) t = (int)std::max<int64_t>(t, (seq_steps + p.num_splits - 1) / p.num_splits);
  return t;
}

// Terms per query element (and per probability): enough for the query's significant bits at four bits
// a term - bf16 two (three where the columns are free anyway), float16 three or four, float32 four -
// laid out as PARTS column groups per matrix op times PASSES trips through the matrix ops, by the
// number of query rows R that share the 16 columns.
template <typename TQ, int D>
int launch_td(const DecP& g, hipStream_t s) {
  constexpr bool BF = std::is_same<TQ, bf16_t>::value, F32 = sizeof(TQ) == 4;
#define DECODE(PARTS, PASSES) hipLaunchKernelGGL((decode_kernel<TQ, D, PARTS, PASSES>), dim3(g.n_waves), dim3(64), 0, s, g)
  if (g.R <= 4) {
    if constexpr (F32) DECODE(4, 1);
    else DECODE(3, 1);
  } else if (g.R <= 8) {
    if constexpr (BF) DECODE(2, 1);
    else DECODE(2, 2);
  } else {
    if constexpr (BF) DECODE(1, 2);
    else if constexpr (F32 && D <= 128) DECODE(1, 4);
    else DECODE(1, 3);  // (float32 at head dim 256: three terms, 12 bits - a fourth pass spills)
  }
#undef DECODE
  int rc = check_launch("decode_kernel");
  if (rc) return rc;
  hipLaunchKernelGGL((decode_merge_kernel<TQ, D>), dim3(g.B * g.Hkv * g.R), dim3(D), 0, s, g);
  return check_launch("decode_merge_kernel");
}
template <typename TQ>
int launch_t(const DecP& g, int head_dim, hipStream_t s) {
  return head_dim == 64 ? launch_td<TQ, 64>(g, s) : head_dim == 128 ? launch_td<TQ, 128>(g, s) : launch_td<TQ, 256>(g, s);
}

// (the same on every device: the size query and the call need not run with the same device current)
int64_t partial_slots(const mi355_sdpa_decode_params& p) {
  return p.q.size[0] * p.k.size[1] + kMaxSimds * dec_occ((int)p.q.size[3]);
}

}  // namespace

int decode_pick_splits(const mi355_sdpa_decode_params& p) {
  const int64_t seq_steps = (p.k.size[2] + 31) / 32;
  const int t = min_steps_for(p);
  return (int)((seq_steps + t - 1) / t);
}

// partial outputs, partial (max, sum) pairs, then the per-batch step prefix sums
size_t decode_workspace(const mi355_sdpa_decode_params& p) {
  const int64_t rep = p.k.size[1] ? p.q.size[1] / p.k.size[1] : 0;
  const int64_t R = rep * p.q.size[2];
  const int64_t D = p.q.size[3];
  return (size_t)(partial_slots(p) * R * (D + 2)) * sizeof(float) + (size_t)(p.q.size[0] + 1) * sizeof(int32_t);
}

// Device address of `scratch` on the current device, looked up once per device.
int decode_static_scratch(void** out) {
  constexpr int kMaxDevices = 64;
  static std::atomic<void*> addr[kMaxDevices];
  int dev = -1;
  const hipError_t e0 = hipGetDevice(&dev);
  if (e0 != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return set_error("SDPA decode: no usable current device (%s)", hipGetErrorString(e0)), MI355_SDPA_ERR_LAUNCH;
  void* ptr = addr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return set_error("SDPA decode: static scratch has no address on device %d (%s)", dev, hipGetErrorString(e)),
             MI355_SDPA_ERR_LAUNCH;
    addr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return MI355_SDPA_OK;
}

int launch_decode_fp8kv(const mi355_sdpa_decode_params& p, hipStream_t s) {
  DecP g;
  g.B = (int)p.q.size[0], g.Hq = (int)p.q.size[1], g.Lq = (int)p.q.size[2];
  g.Hkv = (int)p.k.size[1], g.S = (int)p.k.size[2];
  const int rep = g.Hq / g.Hkv;
  g.R = rep * g.Lq;
  const int D = (int)p.q.size[3];
  if ((D != 64 && D != 128 && D != 256) || p.v.size[3] != D || p.k.size[3] != D)
    return set_error("SDPA decode: head dim must be 64, 128 or 256 (the same for q, k and v), got %lld/%lld/%lld", (long long)p.q.size[3],
                     (long long)p.k.size[3], (long long)p.v.size[3]), MI355_SDPA_ERR_UNSUPPORTED;
  if (g.R < 1 || g.R > 16)
    return set_error("SDPA decode: Lq * Hq/Hkv must be in [1, 16], got %d", g.R), MI355_SDPA_ERR_UNSUPPORTED;
  if (p.q.stride[3] != 1 || p.k.stride[3] != 1 || p.v.stride[3] != 1 || p.out.stride[3] != 1)
    return set_error("SDPA decode: head dim must be unit-stride"), MI355_SDPA_ERR_UNSUPPORTED;
  if (((uintptr_t)p.k.data & 15) || ((uintptr_t)p.v.data & 15) || (p.k.stride[2] & 15) || (p.v.stride[2] & 15) ||
      (p.k.stride[1] & 15) || (p.v.stride[1] & 15) || (p.k.stride[0] & 15) || (p.v.stride[0] & 15))
    return set_error("SDPA decode: K/V rows must be 16-byte aligned"), MI355_SDPA_ERR_UNSUPPORTED;
  if (g.B == 0 || g.S == 0) return set_error("SDPA decode: empty batch or cache"), MI355_SDPA_ERR_UNSUPPORTED;
  g.q = p.q.data, g.k = (const uint8_t*)p.k.data, g.v = (const uint8_t*)p.v.data;
  g.k_scale = p.k_scale, g.v_scale = p.v_scale, g.kv_lens = p.kv_lens, g.out = p.out.data, g.lse = p.lse;
  g.q_sb = p.q.stride[0], g.q_sh = p.q.stride[1], g.q_sl = p.q.stride[2];
  g.k_sb = p.k.stride[0], g.k_sh = p.k.stride[1], g.k_sl = p.k.stride[2];
  g.v_sb = p.v.stride[0], g.v_sh = p.v.stride[1], g.v_sl = p.v.stride[2];
  g.o_sb = p.out.stride[0], g.o_sh = p.out.stride[1], g.o_sl = p.out.stride[2];
  const int64_t max_steps = (int64_t)g.B * g.Hkv * ((g.S + 31) / 32);
  if (max_steps >= (1ll << 31) || (int64_t)(g.S - 1) * p.k.stride[2] + D >= (1ll << 31) ||
      (int64_t)(g.S - 1) * p.v.stride[2] + D >= (1ll << 31))
    return set_error("SDPA decode: cache too large for 32-bit step and row offsets"), MI355_SDPA_ERR_UNSUPPORTED;
  g.t_min = min_steps_for(p);
  // (one or a few long sequences do better with one wavefront per SIMD and longer pieces than with two
  // and half the keys each: every (batch, kv head) is then cut into a hundred pieces and more, and what a
  // wavefront costs beyond its keys, and the partials to merge, weigh more than the second wavefront
  // hides.  8 kv heads, B=1: S=32768 35 -> 26 us, S=131072 64 -> 54; with more sequences, or more keys
  // in all, the other way round)
  const int slots_now = ((int64_t)g.B * g.Hkv <= 32 && max_steps <= 40 * 1024) ? std::min(wave_slots(D), kMaxSimds) : wave_slots(D);
  g.n_waves = (int)std::min<int64_t>(slots_now, std::max<int64_t>(1, (max_steps + g.t_min - 1) / g.t_min));
  const int64_t qes = p.q_dtype == MI355_SDPA_F32 ? 4 : 2;
  if (((uintptr_t)p.q.data & 15) || (p.q.stride[0] * qes) % 16 || (p.q.stride[1] * qes) % 16 || (p.q.stride[2] * qes) % 16)
    return set_error("SDPA decode: query rows must be 16-byte aligned"), MI355_SDPA_ERR_UNSUPPORTED;
  g.scale = p.scale;
  const int64_t slots = partial_slots(p) * g.R;
  g.ws_o = (float*)p.workspace;
  g.ws_ml = g.ws_o + slots * D;
  g.ws_steps = (int32_t*)(g.ws_ml + slots * 2);
  switch (p.q_dtype) {
    case MI355_SDPA_BF16: return launch_t<bf16_t>(g, D, s);
    case MI355_SDPA_F16: return launch_t<f16_t>(g, D, s);
    case MI355_SDPA_F32: return launch_t<float>(g, D, s);
  }
  return set_error("SDPA decode: query dtype must be float32, float16, or bfloat16"), MI355_SDPA_ERR_INVALID;
}

}  // namespace mi355
