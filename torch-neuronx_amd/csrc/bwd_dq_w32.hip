// Flash-attention backward, dQ, for gfx950, head dim 64 or 128, bf16/f16.
//
// One workgroup = 8 wavefronts of 32 query rows each (256 rows of one (batch, query head)), one
// workgroup per compute unit, two wavefronts per SIMD with 256 registers each; it walks the keys
// in tiles of 32:
//
//   S^T = K Q^T, dP^T = V dO^T      (A = K / V rows from LDS, B = Q / dO fragments in registers)
//   P^T = exp2(c S^T - lse), dS^T = P^T (dP^T - delta)
//   dQ^T += K^T dS^T                (A = K^T from the transposing LDS read, B = dS^T packed
//                                    straight from the accumulators)
//
// The scores of tile t + 1 are issued before the vector work of tile t, so that a wavefront's
// own matrix ops cover part of it; the rest is covered by the other wavefront of the SIMD (a
// wavefront issues at most one instruction every four cycles, so one wavefront per SIMD cannot
// keep the matrix and the vector pipe busy together).
//
// K and V tiles sit in LDS row-major and XOR swizzled (see tile_swz).  Math follows
// torch_neuronx/_sdpa_math.py:98-176: float32 accumulation, rows with lse = -inf give zero
// gradients, scale multiplies dQ once at the end.
#include <type_traits>

#include "bwd_mfma.h"

namespace mi355 {
namespace {

constexpr int BM = 256, BN = 32;
constexpr int AHEAD = 2;  // LDS operands are requested this many matrix ops ahead (3 and 4 measure the same)

// MASK = 1: per-batch key counts, and head dims below D (multiples of 8), the missing tail of every
// row counting as zeros.  MASK = 2: on top, a bias / bool keep-mask (a lane reads its own row of
// it) and the gradient of the bias.  MASK = 4: MASK = 1 plus the score functors and document ids
// of score_mod.h, applied to the score tile (and their derivative to dP - delta) in a block of its
// own ahead of the tile's vector work.
template <typename T, int D, int MASK>
__device__ __forceinline__ void bwd_dq_w32_body(const BwdM& p, const MaskArgs ma) {
  constexpr int KS = D / 16, DB = D / 32, CH = D / 8;
  constexpr int TILE = BN * D;
  constexpr int TCH = BN * CH;        // 16-byte chunks per tile
  constexpr bool SPLIT = 512 > TCH;   // more threads than chunks: one half stages K, the other V
  static_assert(AHEAD <= 2 * DB, "ring");
  constexpr int NBUF = 4;  // tile t lives in buffer t % 4
  // (the variant with a bias takes the launch's dynamic LDS: behind the tiles it keeps the list of the
  // key tiles it walks when the call brings a skip table, and a kernel may declare 64 KB at most)
  // MASK = 3 is dropout, with a bias or without: the (B, Hq, L, S) keep-mask is fetched like a bool bias into
  // LDS of its own, leaves the scores alone and multiplies dP, together with 1 / (1 - p)
  // (torch_neuronx/_sdpa_math.py:36-48, :154-158)
  constexpr bool BIASED = MASK == 2 || MASK == 3, DROP = MASK == 3;
  constexpr bool DYN = BIASED;
  __shared__ __attribute__((aligned(16))) uint16_t k_static[DYN ? 8 : NBUF * TILE];
  __shared__ __attribute__((aligned(16))) uint16_t v_static[DYN ? 8 : NBUF * TILE];
  extern __shared__ __attribute__((aligned(16))) uint16_t dyn_lds[];
  uint16_t (*const k_t)[TILE] = (uint16_t (*)[TILE])(DYN ? dyn_lds : k_static);
  uint16_t (*const v_t)[TILE] = (uint16_t (*)[TILE])(DYN ? dyn_lds + NBUF * TILE : v_static);
  uint16_t* const tile_list = dyn_lds + 2 * NBUF * TILE;  // [1024] and the count

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
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 31, half = lane >> 5;
  const int q0 = qt * BM, qw0 = q0 + wave * 32;
  const int qrow = qw0 + col, qc = min(qrow, p.L - 1);

  const int dr = MASK ? p.d_real : D;  // elements per row that exist
  // this lane's query row as B operand of the score products
  u32x4 qf[KS], dof[KS];
  float lse2, dl;
  {
    const uint16_t* qr = (const uint16_t*)p.q + b * p.q_sb + h * p.q_sh + (int64_t)qc * p.q_sl + half * 8;
    const uint16_t* gr = (const uint16_t*)p.go + b * p.go_sb + h * p.go_sh + (int64_t)qc * p.go_sl + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (!MASK || half * 8 + ks * 16 < dr) qf[ks] = *(const u32x4*)(qr + ks * 16), dof[ks] = *(const u32x4*)(gr + ks * 16);
      else qf[ks] = dof[ks] = u32x4{0u, 0u, 0u, 0u};
    }
    // (the fragments are awaited here, once: left pending, their first use inside the tile loop
    // becomes a wait for every outstanding load there, the tile loads in flight included)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[ks]), "+v"(dof[ks]));
    const int64_t idx = ((int64_t)b * p.Hq + h) * p.L + qc;
    const float l = p.lse[idx];
    // +inf turns exp2(x - lse) into 0 for rows past L and for rows without a live key
    lse2 = (qrow < p.L && l != -INFINITY) ? l * kLog2eF : INFINITY;
    if (p.make_delta) {
      // delta = rowsum(dO * O) (torch_neuronx/_sdpa_math.py:160-163): dO is in registers already
      const uint16_t* orow = (const uint16_t*)p.out + b * p.o_sb + h * p.o_sh + (int64_t)qc * p.o_sl + half * 8;
      float dsum = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        if (!MASK || half * 8 + ks * 16 < dr) dsum += dot8<T>(dof[ks], *(const u32x4*)(orow + ks * 16));
      dsum += __shfl_xor(dsum, 32, 64);
      dl = dsum;
      if (qrow < p.L && half == 0) p.delta[idx] = dsum, p.lse2[idx] = l != -INFINITY ? l * kLog2eF : INFINITY;
    } else {
      dl = p.delta[idx];
    }
  }

  uint16_t* gb_row = nullptr;  // this lane's row of the bias gradient, at its first key of a tile
  if constexpr (BIASED) {
    if (p.gbias && qrow < p.L)
      gb_row = (uint16_t*)p.gbias + b * p.gbias_sb + h * p.gbias_sh + (int64_t)qrow * p.gbias_sl + half * 4;
  }
  auto zero_gbias = [&](int t_from) {  // tiles this wavefront does not visit
    if constexpr (BIASED) {
      if (gb_row) {
        for (int t = t_from; t * BN < p.S; ++t)
#pragma unroll
          for (int g = 0; g < 4; ++g)
            if (t * BN + g * 8 + half * 4 < p.S) *(u32x2*)(gb_row + t * BN + g * 8) = u32x2{0u, 0u};
      }
    }
  };
  int S = p.S;  // keys of this batch that take part
  if constexpr (MASK) {
    if (ma.kv_lens) S = min(S, max(ma.kv_lens[b], 0));
  }
  // (split keys, variant with key counts only: this workgroup's part and its rows in the workspace)
  const bool parted = MASK == 1 && p.dq_split_tiles != 0;
  const int split = parted ? (int)blockIdx.y : 0;
  float* const part_row = parted ? p.part_dq + (((int64_t)split * p.B * p.Hq + (int64_t)b * p.Hq + h) * p.L + qc) * dr : nullptr;
  auto zero_row = [&]() {  // no live key: zero gradient
    zero_gbias(0);
    if (parted) {  // (every part writes its rows: the merge adds them all)
      if (qrow < p.L) {
#pragma unroll
        for (int i = 0; i < D / 8; ++i)
          if (half * (D / 2) + i * 4 < dr) *(f32x4*)(part_row + half * (D / 2) + i * 4) = f32x4{0.f, 0.f, 0.f, 0.f};
      }
      return;
    }
    if (qrow < p.L) {
      uint16_t* gq = (uint16_t*)p.gq + b * p.gq_sb + h * p.gq_sh + (int64_t)qrow * p.gq_sl;
#pragma unroll
      for (int i = 0; i < D / 16; ++i)
        if (half * (D / 2) + i * 8 < dr) *(u32x4*)(gq + half * (D / 2) + i * 8) = u32x4{0u, 0u, 0u, 0u};
    }
  };
  if constexpr (MASK) {
    if (S == 0) {
      zero_row();
      return;
    }
  }
  // The key tiles this workgroup walks.  Without a window: 0 .. nt-1.  With one, the tiles below the
  // lowest window of its rows are dropped whole, except the leading ones that hold sink keys: stream
  // position u is key tile u + (u >= n_lead ? skip : 0).
  constexpr bool FUNC = MASK == 1 || MASK == 4;
  constexpr bool SMOD = MASK == 4;  // score functors, document ids
  int nt = (S + BN - 1) / BN;
  if (ma.causal) nt = min(nt, (min(q0 + BM, p.L) - 1) / BN + 1);
  int n_lead = 0, skip = 0;
  // (document ids sorted along the sequence: the keys that this wavefront's rows can see, and whether
  // those rows all belong to one document)
  int doc_run_w[2] = {0, 0x7fffffff};
  bool doc_one_w = false;
  if constexpr (FUNC) {
    int t_lo = ma.window > 0 ? max(q0 - ma.window + 1, 0) / BN : 0;
    if constexpr (SMOD) {
      // document ids sorted along the sequence: only the run of keys whose id lies between the ids of
      // this workgroup's first and last row can hold a kept score; the same for this wavefront's own
      // rows, inside whose run a tile needs no comparison when the rows belong to one document
      if (p.sm.doc_sorted) {
        const int32_t* dqr = p.sm.doc_q + (int64_t)b * p.L;
        const int32_t* dkr = p.sm.doc_k + (int64_t)b * p.S;
        const int first = doc_first_samples(dkr, S, lane);  // (requested ahead of the ids below: one trip for both)
        const int d_lo = dqr[min(q0, p.L - 1)], d_hi = dqr[min(q0 + BM, p.L) - 1];
        const int w_lo = dqr[min(qw0, p.L - 1)], w_hi = dqr[min(qw0 + 32, p.L) - 1];
        int run[2];
        doc_runs(dkr, S, d_lo, d_hi, w_lo, w_hi, run, doc_run_w, lane, first);
        doc_one_w = w_lo == w_hi;
        nt = run[1] > run[0] ? min(nt, (run[1] + BN - 1) / BN) : 0;
        t_lo = max(t_lo, run[0] / BN);
      }
    }
    if (parted) t_lo = split * p.dq_split_tiles;  // (no window in such a call: the part's first tile)
    if (t_lo > 0) {
      n_lead = min(min(ma.window > 0 ? (ma.sink_keys + BN - 1) / BN : 0, t_lo), nt);
      skip = min(t_lo, nt) - n_lead;
      nt -= skip;
    }
    if (parted) {
      nt = min(nt, p.dq_split_tiles);
      if (nt <= 0) {  // (a part behind the keys of this batch, or above the causal diagonal of these rows)
        zero_row();
        return;
      }
    }
    if constexpr (SMOD) {
      if (nt <= 0) {  // (the document ids leave this workgroup's rows without a key)
        zero_row();
        return;
      }
    }
  }
  // With a skip table (variant with a bias, no bias gradient): the tiles in which the mask keeps at
  // least one score of this workgroup's rows.  The first wavefront ORs the bitmaps of the
  // workgroup's 64-row blocks and expands the set bits into a list in LDS, 64 tiles per step.
  bool listed = false;
  if constexpr (MASK == 2) {
    if (p.live_tiles && !ma.causal && !p.gbias) {
      if (wave == 0) {
        const int nrb = (p.L + 63) / 64, rb0 = q0 / 64;
        const uint32_t* map = p.live_tiles + ((int64_t)((p.bias_sb ? b : 0) * p.live_hm + (p.bias_sh ? h : 0)) * nrb + rb0) * p.live_words;
        uint32_t w = 0u;
        if (lane < p.live_words) {
#pragma unroll
          for (int r = 0; r < BM / 64; ++r)
            if (rb0 + r < nrb) w |= map[r * p.live_words + lane];
        }
        int cnt = 0;
        for (int j0 = 0; j0 < nt; j0 += 64) {
          const uint32_t ww = __shfl(w, (j0 >> 5) + (lane >> 5), 64);
          const bool live = j0 + lane < nt && ((ww >> (lane & 31)) & 1u);
          const uint64_t m = __builtin_amdgcn_ballot_w64(live);
          if (live) tile_list[cnt + __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u))] = (uint16_t)(j0 + lane);
          cnt += __builtin_popcountll(m);
        }
        if (lane == 0) *(int*)(tile_list + 1024) = cnt;
      }
      __syncthreads();
      const int n_live = __builtin_amdgcn_readfirstlane(*(const int*)(tile_list + 1024));
      listed = n_live < nt;  // (every tile live: the list is the identity)
      nt = n_live;
    }
  }
  auto tile_of = [&](int u) {
    if constexpr (MASK == 2) return listed ? __builtin_amdgcn_readfirstlane((int)tile_list[u]) : u;
    else return FUNC ? u + (u >= n_lead ? skip : 0) : u;
  };
  const int nt_w = ma.causal ? min(nt, (qw0 + 31) / BN + 1 - skip) : nt;  // tiles with work for this wavefront
  // first tile that needs masking: the one that reaches this wavefront's first row on the causal
  // diagonal (qw0 is a multiple of BN), or a ragged last tile; with a window also every tile that
  // reaches below the window of the wavefront's last row and is not made of sink keys alone
  const int t_edge = min(ma.causal ? qw0 / BN : 0x7fffffff, (S % BN) ? S / BN : 0x7fffffff);
  const int lim = ma.causal ? min(qrow, S - 1) : S - 1;
  const int lo_w = (FUNC && ma.window > 0) ? qrow - ma.window + 1 : (int)0x80000000;
  const int n_sink = FUNC ? ma.sink_keys : 0;
  auto edge_tile = [&](int u) {
    const int ta = tile_of(u);
    bool e = ta >= t_edge;
    if constexpr (FUNC) {
      if (ma.window > 0) e |= ta * BN < qw0 + 31 - ma.window + 1 && ta * BN + BN > n_sink;
    }
    return e;
  };

  // ---- staging: K and V tiles go from global memory straight into LDS ---------------------------
  // (buffer loads with the LDS bit: no trip through registers, no LDS store instructions).  Such a
  // load writes 64 x 16 contiguous bytes, one chunk per lane in lane order, at an LDS address that is
  // uniform for the wavefront: 1 KB = 1024 / (2 D) whole tile rows.  The swizzle is therefore
  // applied on the global side: the lane that owns LDS chunk position c of row r fetches the
  // row's chunk c ^ tile_swz(r).  The resources end with the last key row of this (batch, head),
  // and the whole offset travels in the vector offset, the part the hardware checks against that
  // bound: rows of a ragged last tile beyond it, and chunks past the end of a narrow row, read as
  // zeros.  The loads are inline assembly (the compiler's own form makes every later LDS read
  // wait for all outstanding loads); a tile is requested three iterations before its first use and
  // awaited by hand, with a count that leaves the youngest tile's loads in flight, before the
  // barrier that publishes it.
  const uint16_t* kp = (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh;
  const uint16_t* vp = (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh;
  const int64_t k_bytes = ((int64_t)(S - 1) * p.k_sl + dr) * 2, v_bytes = ((int64_t)(S - 1) * p.v_sl + dr) * 2;
  auto descriptor = [&](const void* base, int64_t bytes) {  // raw buffer resource, in scalar registers
    const uint64_t a = (uint64_t)base;
    return u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a),
                 (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu)),
                 (uint32_t)__builtin_amdgcn_readfirstlane((int)bytes), 0x00020000u};
  };
  const u32x4 k_rsrc = descriptor(kp, k_bytes), v_rsrc = descriptor(vp, v_bytes);
  const bool do_k = !SPLIT || wave < TCH / 64, do_v = !SPLIT || wave >= TCH / 64;  // (uniform per wavefront)
  constexpr int NDMA = SPLIT ? 1 : 2;  // loads per wavefront and tile
  const int s_idx = (SPLIT && tid >= TCH) ? tid - TCH : tid;
  const int s_row = s_idx / CH, s_ch = (s_idx % CH) ^ tile_swz<D>(s_row);
  uint32_t k_off = (uint32_t)((s_row * p.k_sl + s_ch * 8) * 2), v_off = (uint32_t)((s_row * p.v_sl + s_ch * 8) * 2);
  if (MASK && s_ch * 8 >= dr) k_off = v_off = 0x7ffffff0u;  // past the end of a narrow row
  const uint32_t k_tile_bytes = (uint32_t)(BN * p.k_sl * 2), v_tile_bytes = (uint32_t)(BN * p.v_sl * 2);
  typedef __attribute__((address_space(3))) unsigned char* lds_bytes;
  // LDS byte address of this wavefront's 1 KB of a tile, for tile buffer 0
  const uint32_t lds_k = (uint32_t)(uintptr_t)(lds_bytes)&k_t[0][0] + (uint32_t)((SPLIT ? wave % (TCH / 64) : wave) * 1024);
  const uint32_t lds_v = (uint32_t)(uintptr_t)(lds_bytes)&v_t[0][0] + (uint32_t)((SPLIT ? wave % (TCH / 64) : wave) * 1024);
  auto tile_load = [&](const u32x4& rsrc, uint32_t voffset, uint32_t lds_addr) {
    // (m0 holds the LDS address of such a load, one wait state after it is written; it is declared
    // clobbered, so the compiler keeps no value of its own in m0 across the statement)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :: "s"(__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(voffset), "s"(rsrc) : "memory", "m0");
  };
  auto load_tile = [&](int t) {  // tile t (the last one again past the end) into buffer t % 4
    const uint32_t tt = (uint32_t)tile_of(min(t, nt - 1));
    const uint32_t boff = (uint32_t)((t & (NBUF - 1)) * TILE * 2);
    if (do_k) tile_load(k_rsrc, k_off + tt * k_tile_bytes, lds_k + boff);
    if (do_v) tile_load(v_rsrc, v_off + tt * v_tile_bytes, lds_v + boff);
  };
  auto wait_all_tiles = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
  auto wait_older_tiles = [&]() {  // all but the tile requested last
    if constexpr (NDMA == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
  };

  // element offsets inside a tile (the swizzle is not additive in the d block / contraction step:
  // one offset register per combination)
  const int tr_jj = lane & 15, tr_g = lane >> 4;
  int tr_off[2][DB];  // [second read of a pair][d block], without the 16-key step
#pragma unroll
  for (int sec = 0; sec < 2; ++sec)
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int row = 8 * sec + (tr_g >> 1) * 4 + (tr_jj >> 2);
      const int d = db * 32 + 16 * (tr_g & 1) + 4 * (tr_jj & 3);
      tr_off[sec][db] = row * D + (((d >> 3) ^ tile_swz<D>(row)) << 3) + (d & 7);
    }
  int row_off[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) row_off[ks] = col * D + (((2 * ks + half) ^ tile_swz<D>(col)) << 3);
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  // Transposing read: within 16 lanes, lane 4 k + m supplies the address of four consecutive d of
  // key k (d quad m), and lane i receives element i % 4 of the pieces of lanes i / 4, 4 + i / 4,
  // 8 + i / 4, 12 + i / 4: four keys at d = i.  A lane of the 32x32x16 A operand (d row lane % 32,
  // key half lane / 32) takes two such reads: keys 4 half .. +3 and 8 + 4 half .. +3 of a 16-key
  // step, the order in which the score accumulators hold them.
  auto tr_read = [&](const uint16_t* ptr) {
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(ptr));
    return __builtin_bit_cast(u32x2, v);
  };
  // operand i = DB * (16-key step) + d block of K^T
  auto read_cols = [&](const uint16_t* tile, int i) {
    const u32x2 lo = tr_read(tile + tr_off[0][i % DB] + (i / DB) * 16 * D);
    const u32x2 hi = tr_read(tile + tr_off[1][i % DB] + (i / DB) * 16 * D);
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
  };

  f32x16 dqacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) zero(dqacc[i]);
  const float c = p.scale * kLog2eF;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // Score functors and document ids (MASK = 4): the raw score tile s becomes mod(scale * s) / scale
  // and dP becomes delta + (dP - delta) * mod'(scale * s), so that the common code behind them forms
  // P from the modified score and dS = P (dP - delta) mod'.  Lane = query row, element r = key
  // 8 (r / 4) + 4 half + r % 4 of the tile; one block per functor behind a uniform test.
  const float sm_inv_scale = SMOD ? 1.f / p.scale : 0.f;
  const float sm_slope = (SMOD && p.sm.alibi) ? p.sm.alibi[h] * sm_inv_scale : 0.f;
  const float* const sm_kb = (SMOD && p.sm.key_bias) ? p.sm.key_bias + (int64_t)h * p.S : nullptr;
  const float* const sm_kw = (SMOD && p.sm.key_weight) ? p.sm.key_weight + (int64_t)h * p.S : nullptr;
  const int32_t* const sm_dk = (SMOD && p.sm.doc_q && p.sm.doc_k) ? p.sm.doc_k + (int64_t)b * p.S : nullptr;
  // (this row's id is read again where a tile is compared element by element, rather than kept in a
  // register across the loop: such tiles are the few that straddle a document boundary)
  auto my_doc = [&]() { return sm_dk ? p.sm.doc_q[(int64_t)b * p.L + qc] : 0; };
  // (which functors are on, as one scalar: the common cases - no functor at work in this tile, ALiBi
  // alone - then cost one or two taken branches per tile instead of one per functor)
  const int sm_on = SMOD ? __builtin_amdgcn_readfirstlane((sm_kw ? 1 : 0) | (sm_kb ? 2 : 0) | (p.sm.alibi ? 4 : 0) | (p.sm.softcap > 0.f ? 8 : 0)) : 0;
  auto apply_smod = [&](f32x16& sv, f32x16& dpv, int ta) {
    if constexpr (SMOD) {
      const int kvb = ta * BN + half * 4;
      // (sorted ids: a tile inside the key run of this wavefront's one document keeps everything,
      // a tile outside the run of its rows' documents keeps nothing - no load either way)
      const bool doc_whole = doc_one_w && ta * BN >= doc_run_w[0] && ta * BN + BN <= doc_run_w[1];
      if (sm_on == 0 && (sm_dk == nullptr || doc_whole)) return;
      if (sm_on == 4 && (sm_dk == nullptr || doc_whole)) {
        const float base = (float)(kvb - qrow);
#pragma unroll
        for (int r = 0; r < 16; ++r) sv[r] = fmaf(sm_slope, base + (float)((r >> 2) * 8 + (r & 3)), sv[r]);
        return;
      }
      // this lane's 16 values of a vector per key (a tile that ends within the keys reads them at
      // constant offsets from one address; a ragged last tile clamps every index)
      auto load_keys = [&](const auto* row, auto (&val)[16]) {
        if (ta * BN + BN <= p.S) {
          const auto* at = row + kvb;
#pragma unroll
          for (int r = 0; r < 16; ++r) val[r] = at[(r >> 2) * 8 + (r & 3)];
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) val[r] = row[min(kvb + (r >> 2) * 8 + (r & 3), p.S - 1)];
        }
      };
      if (sm_kw) {
        float w[16];
        load_keys(sm_kw, w);
#pragma unroll
        for (int r = 0; r < 16; ++r) sv[r] *= w[r], dpv[r] = fmaf(dpv[r] - dl, w[r], dl);
      }
      if (sm_kb) {
        float kb[16];
        load_keys(sm_kb, kb);
#pragma unroll
        for (int r = 0; r < 16; ++r) sv[r] = fmaf(kb[r], sm_inv_scale, sv[r]);
      }
      if (p.sm.alibi) {
        const float base = (float)(kvb - qrow);
#pragma unroll
        for (int r = 0; r < 16; ++r) sv[r] = fmaf(sm_slope, base + (float)((r >> 2) * 8 + (r & 3)), sv[r]);
      }
      if (p.sm.softcap > 0.f) {
        const float cap_s = p.sm.softcap * sm_inv_scale, icap_s = p.scale / p.sm.softcap;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float th = tanh_fast(sv[r] * icap_s);
          sv[r] = cap_s * th, dpv[r] = fmaf(dpv[r] - dl, fmaf(-th, th, 1.f), dl);
        }
      }
      if (sm_dk) {
        const bool none = p.sm.doc_sorted && (ta * BN >= doc_run_w[1] || ta * BN + BN <= doc_run_w[0]);
        if (none) {
#pragma unroll
          for (int r = 0; r < 16; ++r) sv[r] = -INFINITY;
        } else if (!doc_whole) {
          int id[16];
          load_keys(sm_dk, id);
          const int mine = my_doc();
#pragma unroll
          for (int r = 0; r < 16; ++r) sv[r] = id[r] != mine ? -INFINITY : sv[r];
        }
      }
    }
  };

  // S^T and dP^T of the tile in buffer `buf`: operand i = 2 * contraction step + (0: K rows, 1: V rows)
  auto scores = [&](int buf, f32x16& sacc, f32x16& dpacc) {
    u32x4 ring[8];
    auto rd = [&](int i) { return *(const u32x4*)(((i & 1) ? v_t[buf] : k_t[buf]) + row_off[i >> 1]); };
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) ring[i] = rd(i);
#pragma unroll
    for (int i = 0; i < 2 * KS; ++i) {
      if (i + AHEAD < 2 * KS) ring[(i + AHEAD) & 7] = rd(i + AHEAD);
      if (i & 1) dpacc = Mma<T>::run(ring[i & 7], dof[i >> 1], i == 1 ? zero16 : dpacc);
      else sacc = Mma<T>::run(ring[i & 7], qf[i >> 1], i == 0 ? zero16 : sacc);
    }
  };
  // Bias of a score tile (MASK >= 2): this lane's 16 keys of its query row (row stride 0: a bias per
  // key), as 4 groups of 4 consecutive keys.  It travels like the K / V tiles: from global memory
  // straight into LDS, 16 bytes per lane and instruction whatever the element size, into 4 KB that
  // belong to the wavefront -
  //   float32     4 loads: load g, lane (row, half) -> keys 8 g + 4 half .. +3, read back by the same lane
  //   16 bits     2 loads: load i, lane (row, half) -> keys 16 i + 8 half .. +7; group g of lane (row, half)
  //               is the half-th 8 bytes of what lane (row, g % 2) fetched in load g / 2
  //   bool        1 load:  lane (row, half) -> keys 16 half .. +15; group g is dword 2 (g % 2) + half of
  //               what lane (row, g / 2) fetched
  // - with loads written as assembly and awaited by count.  (Fetched into registers with the
  // compiler's own loads, the wait that it puts in front of their first use covers every load in
  // flight, the tiles requested three iterations ahead included: the kernel then waits out a trip to
  // memory per tile.)  One buffer: the bias of tile t + 1 is requested right after that of tile t
  // has been read back, and is awaited when tile t + 1 needs it, by then the oldest loads in flight.
  // The resource starts at this wavefront's first row of the (batch, head) plane and ends with its
  // last one: keys past S read the next row or, past the last row, zeros (they are masked anyway).
  uint32_t braw[16];
  const int bkind = BIASED ? __builtin_amdgcn_readfirstlane(ma.bias_kind) : 0;
  const int besz = bkind == 1 ? 4 : bkind == 4 ? 1 : 2;
  const int b_rows = min(32, p.L - qw0);
  const u32x4 b_rsrc = descriptor((const char*)p.bias + (bkind ? (b * p.bias_sb + h * p.bias_sh + (int64_t)qw0 * p.bias_sl) * besz : 0),
                                  (bkind && b_rows > 0) ? ((int64_t)(b_rows - 1) * p.bias_sl + p.S) * besz : 0);
  const uint32_t b_voff = BIASED ? (uint32_t)((min(col, max(b_rows - 1, 0)) * p.bias_sl + half * (bkind == 1 ? 4 : bkind == 4 ? 16 : 8)) * besz) : 0u;
  const int b_loads = bkind == 1 ? 4 : bkind == 4 ? 1 : 2;
  const unsigned char* const bias_w = (const unsigned char*)(tile_list + 1040) + (BIASED ? wave * 4096 : 0);
  const uint32_t lds_b = (uint32_t)(uintptr_t)(lds_bytes)bias_w;
  // the keep bytes of a dropout call: one load, lane (row, half) -> keys 16 half .. +15, 1 KB per wavefront behind the bias tiles
  const u32x4 kp_rsrc = descriptor((const char*)p.keep + (DROP ? (((int64_t)b * p.Hq + h) * p.L + qw0) * p.keep_ld : 0),
                                   (DROP && b_rows > 0) ? (int64_t)b_rows * p.keep_ld : 0);  // (whole rows: a dword that reaches past the records reads as zero)
  const uint32_t kp_voff = DROP ? (uint32_t)(min(col, max(b_rows - 1, 0)) * p.keep_ld + half * 16) : 0u;
  const unsigned char* const keep_w = (const unsigned char*)(tile_list + 1040) + (DROP ? 8 * 4096 + wave * 1024 : 0);
  const uint32_t lds_kp = (uint32_t)(uintptr_t)(lds_bytes)keep_w;
  uint32_t kraw[4];
  auto load_bias = [&](int t) {
    if constexpr (BIASED) {
      if (bkind || DROP) {
        // (the reads of the tile before are behind this wavefront before its buffer is rewritten)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      }
      if constexpr (DROP) tile_load(kp_rsrc, kp_voff + (uint32_t)(t * BN), lds_kp);
      if (bkind) {
        const uint32_t g0 = b_voff + (uint32_t)((listed ? tile_of(min(t, max(nt - 1, 0))) : t) * BN * besz);
        tile_load(b_rsrc, g0, lds_b);
        if (b_loads > 1) tile_load(b_rsrc, g0 + 32, lds_b + 1024);
        if (b_loads > 2) {
          tile_load(b_rsrc, g0 + 64, lds_b + 2048);
          tile_load(b_rsrc, g0 + 96, lds_b + 3072);
        }
      }
    }
  };
  // the bias of the tile at hand, from LDS into braw (the only younger loads are those of the tile
  // requested at the end of the previous iteration)
  auto fetch_bias = [&]() {
    if constexpr (BIASED) {
      if constexpr (NDMA == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
      if constexpr (DROP) {
#pragma unroll
        for (int g = 0; g < 4; ++g) kraw[g] = *(const uint32_t*)(keep_w + (col + 32 * (g >> 1)) * 16 + (g & 1) * 8 + half * 4);
      }
      if (bkind == 1) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const u32x4 w = *(const u32x4*)(bias_w + g * 1024 + lane * 16);
          braw[4 * g] = w[0], braw[4 * g + 1] = w[1], braw[4 * g + 2] = w[2], braw[4 * g + 3] = w[3];
        }
      } else if (bkind == 4) {
#pragma unroll
        for (int g = 0; g < 4; ++g) braw[g] = *(const uint32_t*)(bias_w + (col + 32 * (g >> 1)) * 16 + (g & 1) * 8 + half * 4);
      } else if (bkind) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const u32x2 w = *(const u32x2*)(bias_w + (g >> 1) * 1024 + (col + 32 * (g & 1)) * 16 + half * 8);
          braw[2 * g] = w[0], braw[2 * g + 1] = w[1];
        }
      }
    }
  };
  // bias of the 16 accumulator registers in the log2 domain (the element type is tested once,
  // outside the loop: inside, every element would carry the branch)
  auto bias_log2 = [&](float (&bl)[16]) {
    typedef __attribute__((ext_vector_type(2))) _Float16 h2;
    auto each = [&](auto conv) {
#pragma unroll
      for (int r = 0; r < 16; ++r) bl[r] = conv(r);
    };
    if (bkind == 1) each([&](int r) { return __builtin_bit_cast(float, braw[r]) * kLog2eF; });
    else if (bkind == 4) each([&](int r) { return ((braw[r >> 2] >> (8 * (r & 3))) & 0xffu) ? 0.f : -INFINITY; });
    else if (bkind == 3)
      each([&](int r) { return __builtin_bit_cast(float, (r & 1) ? (braw[r >> 1] & 0xffff0000u) : (braw[r >> 1] << 16)) * kLog2eF; });
    else if (bkind == 2) each([&](int r) { return (float)__builtin_bit_cast(h2, braw[r >> 1])[r & 1] * kLog2eF; });
    else each([](int) { return 0.f; });
  };
  // dS^T of tile t, packed as the B operand of dQ^T += K^T dS^T
  auto softmax = [&](int u, const f32x16& sacc, const f32x16& dpacc, uint32_t (&pS)[8]) {
    const int t = tile_of(u);  // (stream position -> key tile)
    const bool edge = SMOD ? edge_tile(u) : t >= t_edge;
    float bl[16];
    if constexpr (BIASED) bias_log2(bl);
    // (the test for a tile that needs masking stays outside the unrolled loop: inside, the compiler
    // turns it into selects that every element of every tile pays for)
    auto elements = [&](auto edge_c) {
      constexpr bool EDGE = decltype(edge_c)::value;
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        float ds[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          float pr;
          if constexpr (BIASED) pr = __builtin_amdgcn_exp2f(fmaf(sacc[r + e], c, bl[r + e]) - lse2);
          else pr = __builtin_amdgcn_exp2f(fmaf(sacc[r + e], c, -lse2));
          if constexpr (EDGE) {
            const int kv = t * BN + ((r + e) >> 2) * 8 + half * 4 + ((r + e) & 3);
            // (bitwise on purpose: with || and && every element gets a cascade of branches)
            const bool dead = SMOD ? (kv > lim) | ((kv < lo_w) & (kv >= n_sink)) : kv > lim;
            pr = dead ? 0.f : pr;
          }
          if constexpr (DROP) {
            const float keep = (float)((kraw[(r + e) >> 2] >> (8 * ((r + e) & 3))) & 0xffu);
            ds[e] = pr * fmaf(dpacc[r + e] * keep, p.keep_scale, -dl);
          } else {
            ds[e] = pr * (dpacc[r + e] - dl);
          }
        }
        pS[r >> 1] = Mma<T>::pack(ds[0], ds[1]);
      }
    };
    if (__builtin_expect(edge, 0)) elements(std::true_type{});
    else elements(std::false_type{});
    if constexpr (BIASED) {
      // grad_bias = grad_logits (torch_neuronx/_sdpa_math.py:163,169): the packed pairs are its
      // elements in the input dtype already; four consecutive keys per store
      if (gb_row) {
#pragma unroll
        for (int g = 0; g < 4; ++g)
          if (t * BN + g * 8 + half * 4 < p.S) *(u32x2*)(gb_row + t * BN + g * 8) = u32x2{pS[2 * g], pS[2 * g + 1]};
      }
    }
  };
  auto accumulate = [&](int buf, const uint32_t (&pS)[8]) {
    u32x4 ring[8];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) ring[i] = read_cols(k_t[buf], i);
#pragma unroll
    for (int i = 0; i < 2 * DB; ++i) {
      if (i + AHEAD < 2 * DB) ring[(i + AHEAD) & 7] = read_cols(k_t[buf], i + AHEAD);
      const int r0 = (i / DB) * 4;
      const u32x4 bS = {pS[r0], pS[r0 + 1], pS[r0 + 2], pS[r0 + 3]};
      dqacc[i % DB] = Mma<T>::run(ring[i & 7], bS, dqacc[i % DB]);
    }
  };

  // Iteration t: tile t + 3 is requested, scores of tile t + 1, vector work of tile t, dQ of tile t.
  // Buffers: tile t in t % 4 (the buffer of tile t + 3 is that of tile t - 1, whose last readers
  // passed the barrier that ended iteration t - 1).
  load_bias(0);
  load_tile(0);
  load_tile(1);
  wait_all_tiles();
  __syncthreads();
  load_tile(2);
  f32x16 s_a, dp_a, s_b, dp_b;
  if (!BIASED && !SMOD && nt_w > 0) scores(0, s_a, dp_a);
  auto iteration = [&](int t, auto tile_mod, f32x16& scur, f32x16& dpcur, f32x16& snext, f32x16& dpnext) {
    // (t % 4 is a compile-time constant, four copies of the iteration: the buffer of a tile then is
    // an immediate offset of the LDS reads, not an addition on the vector unit per read)
    constexpr int buf = decltype(tile_mod)::value, bn = (buf + 1) & (NBUF - 1);
    if (t < nt_w) {
      // (the variant with a bias has no registers to spare for a second score tile: it computes the
      // scores of tile t here, and relies on the other wavefront of the SIMD alone for overlap.  The
      // dropout variant would have them, but gains nothing from the pipelined form: it runs at the
      // cost of reading its mask, a byte per score, from memory.)
      if constexpr (BIASED) {
        scores(buf, scur, dpcur);
        uint32_t pS[8];
        fetch_bias();
        load_bias(t + 1);
        softmax(t, scur, dpcur, pS);
        accumulate(buf, pS);
      } else if constexpr (SMOD) {
        // (the functor variant keeps one score tile, like the variant with a bias: a second one does
        // not fit next to the functors' operands at head dim 128)
        scores(buf, scur, dpcur);
        apply_smod(scur, dpcur, tile_of(t));
        uint32_t pS[8];
        softmax(t, scur, dpcur, pS);
        accumulate(buf, pS);
      } else {
        // Software pipelined by hand (a wavefront issues in order, and left alone the compiler emits
        // the matrix ops in solid runs with all of the vector work between them): the scores of tile
        // t + 1 are one matrix op per slot, and each slot forms one element of dS of tile t; the
        // operands of dQ follow in the same register ring.  A tile that crosses the causal diagonal
        // or the end of the keys gets the scores of its masked positions set to -inf first, in a
        // block of its own (tested per element, the test becomes selects that every tile pays for).
        // (For a wavefront's last tile the scores of the tile after it are computed and dropped.)
        if (__builtin_expect(edge_tile(t), 0)) {
          const int kv0 = tile_of(t) * BN;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int kv = kv0 + (r >> 2) * 8 + half * 4 + (r & 3);
            // (bitwise on purpose: with || and && every element gets a cascade of branches)
            const bool dead = FUNC ? (kv > lim) | ((kv < lo_w) & (kv >= n_sink)) : kv > lim;
            scur[r] = dead ? -INFINITY : scur[r];
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        uint32_t pS[8];
        u32x4 ring[8];
        const uint16_t* kt = k_t[buf];
        auto rd = [&](int i) { return *(const u32x4*)(((i & 1) ? v_t[bn] : k_t[bn]) + row_off[i >> 1]); };
#pragma unroll
        for (int i = 0; i < AHEAD; ++i) ring[i] = rd(i);
        __builtin_amdgcn_sched_barrier(0);
        float ds_even = 0.f;
        // (scores and dS are on the critical path, the dQ accumulation is not: the wavefront that is
        // in its score slots goes first when both of a SIMD want to issue; measured 1.4 %)
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int i = 0; i < 2 * KS; ++i) {
          const int n = i + AHEAD;
          ring[n & 7] = n < 2 * KS ? rd(n) : read_cols(kt, n - 2 * KS);
          if (i & 1) dpnext = Mma<T>::run(ring[i & 7], dof[i >> 1], i == 1 ? zero16 : dpnext);
          else snext = Mma<T>::run(ring[i & 7], qf[i >> 1], i == 0 ? zero16 : snext);
          // elements of dS: 16 over the 2 * KS slots
#pragma unroll
          for (int r = i * 16 / (2 * KS); r < (i + 1) * 16 / (2 * KS); ++r) {
            const float pr = __builtin_amdgcn_exp2f(fmaf(scur[r], c, -lse2));
            const float d = pr * (dpcur[r] - dl);
            if (r & 1) pS[r >> 1] = Mma<T>::pack(ds_even, d);
            else ds_even = d;
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_setprio(0);
#pragma unroll
        for (int j = 0; j < 2 * DB; ++j) {
          if (j + AHEAD < 2 * DB) ring[(j + AHEAD) & 7] = read_cols(kt, j + AHEAD);
          const int r0 = (j / DB) * 4;
          const u32x4 bS = {pS[r0], pS[r0 + 1], pS[r0 + 2], pS[r0 + 3]};
          dqacc[j % DB] = Mma<T>::run(ring[j & 7], bS, dqacc[j % DB]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    load_tile(t + 3);
    // Tile t + 2, read from the next iteration on, has to be whole.  (With a bias the tile read next
    // is t + 1, and a wavefront with work has seen it land when it awaited this iteration's bias, a
    // younger load: it leaves the bias of the next tile and the tile requested above in flight.  A
    // wavefront without work awaits no bias and waits here.)
    if (!BIASED || t >= nt_w) wait_older_tiles();
    __syncthreads();
  };
  for (int t = 0;;) {
    if (t >= nt) break;
    iteration(t, std::integral_constant<int, 0>{}, s_a, dp_a, s_b, dp_b);
    if (++t >= nt) break;
    iteration(t, std::integral_constant<int, 1>{}, s_b, dp_b, s_a, dp_a);
    if (++t >= nt) break;
    iteration(t, std::integral_constant<int, 2>{}, s_a, dp_a, s_b, dp_b);
    if (++t >= nt) break;
    iteration(t, std::integral_constant<int, 3>{}, s_b, dp_b, s_a, dp_a);
    ++t;
  }
  zero_gbias(nt_w);

  if (parted) {
    if (qrow < p.L) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int d = db * 32 + g * 8 + half * 4;
          if (d < dr)
            *(f32x4*)(part_row + d) = f32x4{dqacc[db][g * 4] * p.scale, dqacc[db][g * 4 + 1] * p.scale, dqacc[db][g * 4 + 2] * p.scale,
                                            dqacc[db][g * 4 + 3] * p.scale};
        }
    }
    return;
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
        if (!MASK || db * 32 + g * 8 + half * 4 < dr) *(u32x2*)(gq + db * 32 + g * 8 + half * 4) = w;
      }
  }
}

// The kernel of a variant.  A call whose bias comes with a verdict about it (see MaskArgs) is launched
// twice: as the variant with a bias (MASK = 2), and as the variant with key counts marked PATTERN; the
// verdict lets one of them run.
template <typename T, int D, int MASK, bool PATTERN = false>
__global__ __launch_bounds__(512, 1) void bwd_dq_w32_kernel(BwdM p) {
  static_assert(!PATTERN || MASK == 1, "the pattern kernel is the variant with key counts");
  MaskArgs ma = mask_args_of(p);
  if constexpr (MASK == 2 || PATTERN) {
    if (verdict_pattern(p, ma) != PATTERN) return;
  } else if constexpr (MASK == 3) {
    verdict_pattern(p, ma);  // (dropout: one variant takes a bias or none, so the verdict is applied in place)
  }
  bwd_dq_w32_body<T, D, MASK>(p, ma);
}

// dQ of a call whose keys were split: the sum of the parts' float32 rows, rounded once.  One 64-thread
// block per query row, four columns per thread.
template <typename T>
__global__ __launch_bounds__(64) void bwd_dq_merge_kernel(BwdM p) {
  const int64_t row = blockIdx.x;  // (b * Hq + h) * L + l
  const int l = (int)(row % p.L), h = (int)((row / p.L) % p.Hq), b = (int)(row / ((int64_t)p.L * p.Hq));
  const int64_t rows = (int64_t)p.B * p.Hq * p.L;
  const int c = threadIdx.x * 4;
  if (c >= p.d_real) return;
  const float* src = p.part_dq + row * p.d_real + c;
  f32x4 a = {0.f, 0.f, 0.f, 0.f};
  for (int i = 0; i < p.dq_n_split; ++i) a += *(const f32x4*)(src + i * rows * p.d_real);
  u32x2 w;
  w[0] = Mma<T>::pack(a[0], a[1]);
  w[1] = Mma<T>::pack(a[2], a[3]);
  *(u32x2*)((uint16_t*)p.gq + b * p.gq_sb + h * p.gq_sh + (int64_t)l * p.gq_sl + c) = w;
}

}  // namespace

bool bwd_dq_w32_fits(const BwdM& g, int head_dim) {
  // 32-bit byte offsets from the start of a (batch, kv head) for K and V
  (void)head_dim;
  return (int64_t)(g.S + BN) * g.k_sl * 2 < (1ll << 31) && (int64_t)(g.S + BN) * g.v_sl * 2 < (1ll << 31) && g.k_sl >= 0 && g.v_sl >= 0;
}

int launch_bwd_dq_w32(const BwdM& g, int dtype, int head_dim, hipStream_t s) {
  const int64_t blocks = (int64_t)g.B * g.Hq * ((g.L + BM - 1) / BM);
  const dim3 grid((unsigned)blocks, (unsigned)(g.dq_split_tiles ? g.dq_n_split : 1)), block(512);
  const bool bf = dtype == MI355_SDPA_BF16;
  if (g.sm.any && (g.keep_scale != 0.f || g.bias_kind || g.gbias)) {
    set_error("SDPA: score functors in bwd_dq_w32_kernel need a call without bias and dropout");
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  if (g.keep_scale != 0.f && (!g.keep || g.live_tiles)) {
    set_error("SDPA: dropout in bwd_dq_w32_kernel needs a keep-mask and no tile table");
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  const int mask = g.sm.any ? 4 : g.keep_scale != 0.f ? 3 : (g.bias_kind || g.gbias) ? 2 : (g.kv_lens || g.d_real != head_dim || g.window > 0 || g.dq_split_tiles) ? 1 : 0;
  if (g.dq_split_tiles && (mask != 1 || g.window > 0 || !g.part_dq)) {
    set_error("SDPA: split keys in bwd_dq_w32_kernel need a call without bias, dropout, functors and window, and a workspace");
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  // (the tiles, the tile list of a call with a skip table, 4 KB of bias tile per wavefront)
  const int dyn = (mask == 2 || mask == 3) ? 2 * 4 * BN * head_dim * 2 + 2080 + 8 * 4096 + (mask == 3 ? 8 * 1024 : 0) : 0;
  if (mask == 2 || mask == 3) {
    const void* fn2 = head_dim == 128 ? (bf ? (const void*)bwd_dq_w32_kernel<bf16_t, 128, 2> : (const void*)bwd_dq_w32_kernel<f16_t, 128, 2>)
                                      : (bf ? (const void*)bwd_dq_w32_kernel<bf16_t, 64, 2> : (const void*)bwd_dq_w32_kernel<f16_t, 64, 2>);
    const void* fn3 = head_dim == 128 ? (bf ? (const void*)bwd_dq_w32_kernel<bf16_t, 128, 3> : (const void*)bwd_dq_w32_kernel<f16_t, 128, 3>)
                                      : (bf ? (const void*)bwd_dq_w32_kernel<bf16_t, 64, 3> : (const void*)bwd_dq_w32_kernel<f16_t, 64, 3>);
    const void* fn = mask == 3 ? fn3 : fn2;
    static LdsOnce once[8];  // (one per instance with dynamic LDS)
    const hipError_t attr = reserve_lds(once[(head_dim == 128 ? 4 : 0) + (bf ? 2 : 0) + (mask == 3 ? 1 : 0)], fn, dyn);
    if (attr != hipSuccess) {
      set_error("SDPA: cannot reserve %d bytes of LDS for bwd_dq_w32_kernel: %s", dyn, hipGetErrorString(attr));
      return MI355_SDPA_ERR_LAUNCH;
    }
  }
#define LAUNCH(TT, DD, MM) hipLaunchKernelGGL((bwd_dq_w32_kernel<TT, DD, MM>), grid, block, ((MM) == 2 || (MM) == 3) ? dyn : 0, s, g)
#define LAUNCH_M(TT, DD)                                                     \
  do {                                                                       \
    if (mask == 2 && g.verdict) /* (see bwd_dq_w32_kernel) */                \
      hipLaunchKernelGGL((bwd_dq_w32_kernel<TT, DD, 1, true>), grid, block, 0, s, g); \
    if (mask == 4) LAUNCH(TT, DD, 4);                                        \
    else if (mask == 3) LAUNCH(TT, DD, 3);                                   \
    else if (mask == 2) LAUNCH(TT, DD, 2);                                   \
    else if (mask == 1) LAUNCH(TT, DD, 1);                                   \
    else LAUNCH(TT, DD, 0);                                                  \
  } while (0)
#define LAUNCH_D(DD)                                                         \
  do {                                                                       \
    if (bf) LAUNCH_M(bf16_t, DD); else LAUNCH_M(f16_t, DD);                  \
  } while (0)
  if (head_dim == 128) LAUNCH_D(128);
  else LAUNCH_D(64);
#undef LAUNCH_D
#undef LAUNCH_M
#undef LAUNCH
  const int rc = check_launch("bwd_dq_w32_kernel");
  if (rc != MI355_SDPA_OK || !g.dq_split_tiles) return rc;
  const dim3 rows((unsigned)((int64_t)g.B * g.Hq * g.L));
  if (bf) hipLaunchKernelGGL((bwd_dq_merge_kernel<bf16_t>), rows, dim3(64), 0, s, g);
  else hipLaunchKernelGGL((bwd_dq_merge_kernel<f16_t>), rows, dim3(64), 0, s, g);
  return check_launch("bwd_dq_merge_kernel");
}

}  // namespace mi355
