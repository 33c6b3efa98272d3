// Flash-attention forward for gfx950, head dim 64, 128 or 256 (narrower rows: see MASK), bf16/f16.
//
// One workgroup = WAVES wavefronts of 32 query rows each, all of one (batch, query head):
// WAVES = 8 (256 rows, one workgroup per compute unit) for long sequences, WAVES = 4 (128 rows,
// two workgroups per compute unit) for short or few ones.  Either way a SIMD hosts two
// wavefronts with 256 registers each (head dim 256: one wavefront with 512).
//
// Why two wavefronts per SIMD: a wavefront issues at most one instruction every four cycles,
// whatever the instruction.  A 32x32x16 matrix op keeps the matrix pipe busy for 32 cycles, the
// softmax of the scores it produces costs about 20 cycles on the vector unit (v_exp_f32 is half
// rate), and around those sit LDS reads, waits and scalar bookkeeping.  A single wavefront per
// SIMD (64 query rows, so that every LDS fragment feeds two matrix ops) runs out of issue slots
// long before either pipe is full; with two, one wavefront's vector and LDS instructions issue
// under the other's matrix op.  LDS bandwidth does not bind (a compute unit reads about
// 256 B/clk with ds_read_b128; this kernel asks for a third of that).  What the kernel runs
// into instead is the power limit: with random operands a pure stream of these matrix ops
// sustains about 1.7 PFLOP/s on MI355X (2.3 with zeros), and every LDS read, global load and
// vector op costs some of that.
//
// Inside a wavefront the key loop is software pipelined by hand, because a wavefront issues in
// order: the softmax of a 32-key tile is split in two halves that ride on the matrix ops of two
// different phases, and LDS operands are fetched AHEAD matrix ops ahead through a register
// ring.  The loop carries no row maximum: see kTrig.  K and V tiles go from global memory
// straight into LDS, three tiles ahead of their use; so does a bias, one tile ahead.
// Products are computed transposed (S^T = K Q^T, O^T = V^T P^T) as in fwd_mfma.hip, so the
// softmax statistics are per-lane scalars and P goes from accumulator to B operand in registers.
//
// Numerics: torch_neuronx/_sdpa_math.py:51-95 (float32 accumulation and softmax, probabilities
// rounded to the input dtype for P*V only, dead rows give zeros and lse = -inf).
#include <type_traits>

#include "fwd_mfma.h"

namespace mi355 {
namespace {

constexpr int BN = 32;
constexpr int AHEAD = 4;  // LDS operands are requested this many matrix ops ahead
constexpr float kLazy = 8.f;  // log2 headroom before the accumulator is rescaled

// MASK = 1 adds per-batch key counts (kv_lens) and head dims below D (multiples of 8): the missing
// tail of every Q / K / V row counts as zeros, which changes neither the scores nor the live part
// of the output.  MASK = 2 adds an additive bias or boolean keep-mask on top, folded into the
// score tile right after the matrix ops that produce it.  The bias travels like the tiles: from
// global memory straight into LDS (lane-private slots), with loads written as assembly and
// awaited by count, so that nothing in the loop waits on a count the compiler chose.
// MASK = 3 is dropout: the (B, Hq, L, S) keep-mask travels like a boolean bias, but it leaves the
// scores, the row sums and the lse alone and zeroes the dropped probabilities where they are packed
// for the second product; 1 / (1 - p) is applied with the final normalisation
// (torch_neuronx/_sdpa_math.py:36-48: the mask multiplies the normalised probabilities).
// MASK = 4 is MASK = 1 plus the score functors and document ids of score_mod.h:
// they rewrite the raw score tile in a block of its own right after the matrix ops that produce it,
// where the bias of MASK = 2 is folded in, so the softmax behind them is the common code.
template <typename T, int D, int WAVES, int MASK>
__device__ __forceinline__ void fwd_w32_body(const FwdM& p, const MaskArgs ma) {
  constexpr int BM = 32 * WAVES, NT = 64 * WAVES;
  constexpr int KS = D / 16;      // matrix ops of S^T = K Q^T per tile (phase A)
  constexpr int DB = D / 32;      // 32-row blocks of O^T
  constexpr int NPV = 2 * DB;     // matrix ops of O^T += V^T P^T per tile (phase B)
  constexpr int CH = D / 8;       // 16-byte chunks per row
  constexpr int TCH = BN * CH;    // ... per tile
  static_assert(AHEAD <= KS && AHEAD <= NPV && (KS + NPV) % 8 == 0, "ring layout");
  // (head dim 256 and the variant with a bias need more than the 64 KB of LDS a kernel may declare:
  // they take the launch's dynamic LDS instead; head dim 256 runs one wavefront per SIMD with the
  // 512-register budget)
  constexpr bool BIASED = MASK == 2 || MASK == 3, DROP = MASK == 3;  // a bias tile in LDS; ... and the tile of a dropout keep-mask beside it
  constexpr bool DYN = D > 128 || BIASED;
  // Tiles go from global memory straight into LDS (see the staging section): four unpadded,
  // swizzled buffers per operand, tile t in buffer t % 4.
  // mask functors (window, sink keys, sink logit): in the masked variant without a bias
  constexpr bool FUNC = MASK == 1 || MASK == 4;
  constexpr bool SMOD = MASK == 4;  // score functors, document ids
  constexpr int NBUF = 4, TILE = BN * D;
  __shared__ __attribute__((aligned(16))) uint16_t k_static[DYN ? 8 : NBUF * TILE];
  __shared__ __attribute__((aligned(16))) uint16_t v_static[DYN ? 8 : NBUF * TILE];
  extern __shared__ __attribute__((aligned(16))) uint16_t dyn_lds[];
  uint16_t* const k_dma = DYN ? dyn_lds : k_static;
  uint16_t* const v_dma = DYN ? dyn_lds + NBUF * TILE : v_static;
  // bias tiles (MASK = 2): per wavefront two buffers of four 1 KB groups, every lane its own 16 bytes of each
  uint16_t* const bias_lds = dyn_lds + 2 * NBUF * TILE;
  // ... and, with a tile skip table, the list of the key tiles this workgroup walks (1024 entries and the count)
  uint16_t* const tile_list = bias_lds + WAVES * 2048;
  // (dropout, which never comes with a table, has a wavefront's 1 KB of keep bytes there)
  const unsigned char* const keep_lds = (const unsigned char*)(bias_lds + WAVES * 2048);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: keeps per-wavefront tests on the scalar unit
  int b, h, qt;
  int wrow = wave * 32;  // this wavefront's first row within the workgroup's rows
  int split = 0;  // (grouped calls with split keys: which part of them)
  if (MASK != 3 && p.grouped) {  // (see FwdM::grouped)
    const int rep = p.Hq / p.Hkv, hpw = p.grouped, chunks = rep / hpw;  // heads per workgroup, workgroups per kv head
    const int bhc = blockIdx.x / p.n_split;
    split = blockIdx.x % p.n_split;
    const int bhk = bhc / chunks;
    b = bhk / p.Hkv, h = (bhk % p.Hkv) * rep + (bhc % chunks) * hpw + wave % hpw, qt = 0;
    wrow = (wave / hpw) * 32;
  } else {
    decode_block(p, b, h, qt);
  }
  const int hk = h / (p.Hq / p.Hkv);
  const int col = lane & 31, half = lane >> 5;
  const int q0 = qt * BM;
  const int qw0 = q0 + wrow;
  const int qrow = qw0 + col;
  const int qw_last = qw0 + 31;

  const int dr = MASK ? p.d_real : D;    // elements per row of Q and K that exist
  const int drv = MASK ? p.dv_real : D;  // ... of V and the output
  // keys of this batch that take part
  int S = p.S;
  if constexpr (MASK) {
    if (ma.kv_lens) S = min(S, max(ma.kv_lens[b], 0));
    if constexpr (BIASED) {
      // A keep-mask per key (no row stride: padding masks): the keys behind the last one it keeps are
      // never visited, as with a key count.  Every wavefront scans the row itself (S bytes, four
      // per lane and step; rows are whole dwords) and they all arrive at the same count.
      if (ma.bias_kind == 4 && p.bias_sl == 0 && S > 0) {
        const uint8_t* mrow = (const uint8_t*)p.bias + b * p.bias_sb + h * p.bias_sh;
        int last = -1;
        for (int j = lane * 4; j < S; j += 256) {
          const uint32_t w = *(const uint32_t*)(mrow + j);
          if (w) last = j + ((31 - __builtin_clz(w)) >> 3);
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) last = max(last, __shfl_xor(last, off, 64));
        S = min(S, __builtin_amdgcn_readfirstlane(last) + 1);
      }
    }
  }
  // The key tiles this workgroup walks.  Without a window: 0 .. nt-1.  With one, the tiles below the
  // lowest window of its rows are dropped whole, except the leading ones that hold sink keys: stream
  // position u is key tile u + (u >= n_lead ? skip : 0).
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
      // Document ids that are sorted along the sequence: the keys whose id lies between the ids of
      // this workgroup's first and last row are one run of doc_k; the tiles outside it hold no kept
      // score and are not walked.  The same for this wavefront's own rows: inside its run a tile
      // needs no comparison at all when the rows belong to one document.  Four searches, fused.
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
    if (t_lo > 0) {
      n_lead = min(min(ma.window > 0 ? (ma.sink_keys + BN - 1) / BN : 0, t_lo), nt);
      skip = min(t_lo, nt) - n_lead;
      nt -= skip;
    }
  }
  // ALiBi under a causal mask: the bias grows towards the diagonal, by up to 39 bits of the exponent
  // per tile for the steepest head, so walking the keys upwards the reference of the lazy softmax is
  // overtaken tile after tile and the rare slow path (true maximum, rescaled accumulators, the tile's
  // probabilities once more) becomes the common one: 110 of 388 us at B=2, 32 heads, S=4096.  Such
  // calls walk their tiles from the diagonal down instead: the first tiles set the reference, and
  // what follows only falls.  Every wavefront then walks all of the workgroup's tiles (the ones above
  // its own diagonal come first and are masked whole: rows without a live key yet, see the check).
  // (a head whose slope is not positive keeps the upward walk: its bias falls towards the diagonal)
  const bool backwards = SMOD && ma.causal && p.sm.alibi != nullptr && ma.window == 0 && n_lead == 0 && skip == 0 &&
                         !(p.sm.doc_q && p.sm.doc_k) && p.sm.alibi[h] > 0.f;
  constexpr bool SPLITS = MASK == 1 || (MASK == 2 && D <= 128);  // the variants that can split their keys
  if constexpr (SPLITS) {
    if (p.split_tiles) {  // this workgroup's share of the key tiles (no window, no skip table then)
      skip = split * p.split_tiles;
      nt = max(min(nt - skip, p.split_tiles), 0);
    }
  }
  // With a tile skip table (variant with a bias): the tiles in which the mask keeps at least one score
  // of this workgroup's rows, in ascending order.  The first wavefront ORs the bitmaps of the
  // workgroup's 64-row blocks and expands the set bits into a list in LDS, 64 tiles per step.
  bool listed = false;
  if constexpr (MASK == 2) {
    if (p.live_tiles && !ma.causal) {
      listed = true;
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
  // the sink logits of this (batch, head) as one: the logarithm of the sum of their exponentials
  auto sink_lse = [&]() {
    const float* zs = p.sink_logit + ((int64_t)b * p.Hq + h) * p.n_sinks;
    float zm = -INFINITY, zl = 0.f;
    for (int n = 0; n < p.n_sinks; ++n) zm = fmaxf(zm, zs[n]);
    if (zm == -INFINITY) return -INFINITY;
    for (int n = 0; n < p.n_sinks; ++n) zl += __expf(zs[n] - zm);
    return zm + __builtin_logf(zl);
  };
  auto tile_of = [&](int u) {
    if constexpr (MASK == 2) return listed ? __builtin_amdgcn_readfirstlane((int)tile_list[u]) : u + skip;
    // (the pipeline also forms, and drops, the scores of the stream position behind a wavefront's last
    // one: walking down that would be tile -1, whose per-key vectors lie in front of their arrays)
    else if constexpr (SMOD) return backwards ? max(nt - 1 - u, 0) : u + (u >= n_lead ? skip : 0);
    else return FUNC ? u + (u >= n_lead ? skip : 0) : SPLITS ? u + skip : u;  // (head dim 256: split keys, no window)
  };
  if constexpr (MASK) {
    if (nt <= 0) {  // no live key: zeros and lse = -inf (torch_neuronx/_sdpa_math.py:85-87), or the sink logit alone
      if constexpr (SPLITS) {
        if (p.split_tiles) {  // (split keys: a part without keys carries no weight in the merge)
          if (qrow < p.L && half == 0) p.part_lse[(((int64_t)b * p.Hq + h) * p.n_split + split) * p.L + qrow] = -INFINITY;
          return;
        }
      }
      if (qrow < p.L) {
        uint16_t* orow = (uint16_t*)p.out + b * p.o_sb + h * p.o_sh + (int64_t)qrow * p.o_sl;
#pragma unroll
        for (int i = 0; i < D / 16; ++i)
          if (half * (D / 2) + i * 8 < drv) *(u32x4*)(orow + half * (D / 2) + i * 8) = u32x4{0u, 0u, 0u, 0u};
        if (p.lse && half == 0)
          p.lse[((int64_t)b * p.Hq + h) * p.L + qrow] = (FUNC && p.sink_logit) ? sink_lse() : -INFINITY;
      }
      return;
    }
  }

  const uint16_t* qp = (const uint16_t*)p.q + b * p.q_sb + h * p.q_sh;
  const uint16_t* kp = (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh;
  const uint16_t* vp = (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh;

  u32x4 qf[KS];
  {
    const uint16_t* qr = qp + (int64_t)min(qrow, p.L - 1) * p.q_sl + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (!MASK || half * 8 + ks * 16 < dr) qf[ks] = *(const u32x4*)(qr + ks * 16);
      else qf[ks] = u32x4{0u, 0u, 0u, 0u};
    }
    // (awaited in the prologue, once, behind the request for the first tiles, so that the two trips
    // to memory overlap: left pending, their first use inside the tile loop would become a wait for
    // every outstanding load there, the tile loads in flight included)
  }
  auto await_q = [&]() {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[ks]));
    // (one wavefront per SIMD owns both halves of the register file: the Q fragments live in the
    // accumulation half, where the matrix ops read them directly; left to the allocator they are
    // parked there anyway and copied back, four moves ahead of every op that uses one)
    if constexpr (D > 128) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(qf[ks]));
    }
  };

  const int nt_w = (ma.causal && !backwards) ? min(nt, qw_last / BN + 1 - skip) : nt;

  // K and V are read through buffer resources that end with the last key row of this (batch, head);
  // the whole offset travels in the vector offset, the part the hardware checks against that bound:
  // rows of a ragged last tile beyond it read as zeros (their scores are masked, and a zero V row
  // keeps 0 * V finite).
  const int k_bytes = (int)(((int64_t)(S - 1) * p.k_sl + dr) * 2), v_bytes = (int)(((int64_t)(S - 1) * p.v_sl + drv) * 2);
  const int k_tile_bytes = (int)(BN * p.k_sl * 2), v_tile_bytes = (int)(BN * p.v_sl * 2);
  // ---- staging: K and V tiles go from global memory straight into LDS ------------------------------
  // (buffer loads with the LDS bit: no trip through registers, no LDS store instructions).  Such a
  // load writes 64 x 16 contiguous bytes, one chunk per lane in lane order, at an LDS address that is
  // uniform for the wavefront, so the tiles are unpadded and bank conflicts are avoided by a
  // swizzle applied on the global side: the lane that owns LDS chunk position c of row r fetches
  // the row's chunk c ^ tile_swz(r).  Rows of a ragged last tile lie beyond the resource's bound
  // and read as zeros.  The loads are inline assembly (the compiler's own form makes every later
  // LDS read wait for all outstanding loads) and are awaited by hand.  Tiles travel in pairs,
  // pair j = K tile j+1 and V tile j, the two that the barrier of iteration j-1 publishes; pair
  // j is requested right after the barrier of iteration j-4, when the last reads of the buffers
  // it overwrites are behind every wavefront, so a pair has three iterations to land.
  constexpr int KL = TCH / 64;             // wavefront loads per tile
  constexpr bool DSPLIT = KL < WAVES;      // fewer than wavefronts: half of them stage K, half V
  constexpr int NL = DSPLIT ? 1 : KL / WAVES;  // loads per wavefront and tile
  constexpr int PL = DSPLIT ? 1 : 2 * NL;      // ... and pair
  static_assert(DSPLIT ? 2 * KL == WAVES : KL % WAVES == 0, "staging layout");
  auto descriptor = [&](const void* base, int bytes) {  // raw buffer resource, in scalar registers
    const uint64_t a = (uint64_t)base;
    return u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a),
                 (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu)),
                 (uint32_t)__builtin_amdgcn_readfirstlane(bytes), 0x00020000u};
  };
  const u32x4 kd_rsrc = descriptor(kp, k_bytes), vd_rsrc = descriptor(vp, v_bytes);
  const int d_wave = DSPLIT ? wave % KL : wave;  // this wavefront's first 1 KB slice of a tile
  const bool dma_k = !DSPLIT || wave < KL, dma_v = !DSPLIT || wave >= KL;  // (uniform per wavefront)
  uint32_t kd_off[NL], vd_off[NL];
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int ch = (d_wave + i * WAVES) * 64 + lane, row = ch / CH, gch = (ch % CH) ^ tile_swz<D>(row);
    kd_off[i] = (uint32_t)((row * p.k_sl + gch * 8) * 2);
    vd_off[i] = (uint32_t)((row * p.v_sl + gch * 8) * 2);
    if constexpr (MASK) {  // chunks past the end of a narrow row: an offset beyond any resource reads as zeros
      if (gch * 8 >= dr) kd_off[i] = 0x7ffffff0u;
      if (gch * 8 >= drv) vd_off[i] = 0x7ffffff0u;
    }
  }
  typedef __attribute__((address_space(3))) unsigned char* lds_bytes;
  const uint32_t lds_kd = (uint32_t)(uintptr_t)(lds_bytes)k_dma + (uint32_t)(d_wave * 1024);
  const uint32_t lds_vd = (uint32_t)(uintptr_t)(lds_bytes)v_dma + (uint32_t)(d_wave * 1024);
  auto tile_load = [&](const u32x4& rsrc, uint32_t voffset, uint32_t lds_addr) {
    // (m0 holds the LDS address of such a load, one wait state after it is written; it is declared
    // clobbered, so the compiler keeps no value of its own in m0 across the statement)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :: "s"(__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(voffset), "s"(rsrc) : "memory", "m0");
  };
  auto request_k = [&](int t) {  // K tile t (the last one again past the end) into buffer t % 4
    const uint32_t g = (uint32_t)(tile_of(min(t, nt - 1)) * k_tile_bytes), l = lds_kd + (uint32_t)((t & (NBUF - 1)) * TILE * 2);
    if (dma_k) {
#pragma unroll
      for (int i = 0; i < NL; ++i) tile_load(kd_rsrc, kd_off[i] + g, l + i * WAVES * 1024);
    }
  };
  auto request_v = [&](int t) {
    const uint32_t g = (uint32_t)(tile_of(min(t, nt - 1)) * v_tile_bytes), l = lds_vd + (uint32_t)((t & (NBUF - 1)) * TILE * 2);
    if (dma_v) {
#pragma unroll
      for (int i = 0; i < NL; ++i) tile_load(vd_rsrc, vd_off[i] + g, l + i * WAVES * 1024);
    }
  };
  auto request_pair = [&](int j) { request_k(j + 1), request_v(j); };
  auto wait_all_tiles = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
  auto wait_youngest_pair_only = [&]() {  // everything but the pair requested last has landed
    if constexpr (PL == 1) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
    else if constexpr (PL == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    else if constexpr (PL == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  };
  auto wait_oldest_pair = [&]() {  // of three in flight
    static_assert(PL == 1 || PL == 2 || PL == 4 || PL == 8, "wait count");
    if constexpr (PL == 1) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    else if constexpr (PL == 2) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else if constexpr (PL == 4) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  };
  // element offsets of the LDS reads inside a swizzled tile.  The swizzle is not additive in the d
  // block / contraction step within a 256-byte window of a row (one offset register per
  // combination there); the second window of a 512-byte row is the first plus 256 bytes, which
  // travels in the instruction's immediate offset.
  constexpr int KSW = KS < 8 ? KS : 8, DBW = DB < 4 ? DB : 4;
  int row_off_w[KSW], tr_off_w[2][DBW];  // K row reads; V transposing reads [second read of a pair][d block]
#pragma unroll
  for (int ks = 0; ks < KSW; ++ks) row_off_w[ks] = col * D + (((2 * ks + half) ^ tile_swz<D>(col)) << 3);
#pragma unroll
  for (int sec = 0; sec < 2; ++sec)
#pragma unroll
    for (int db = 0; db < DBW; ++db) {
      const int row = 8 * sec + ((lane >> 5) & 1) * 4 + ((lane & 15) >> 2);
      const int d = db * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
      tr_off_w[sec][db] = row * D + (((d >> 3) ^ tile_swz<D>(row)) << 3) + (d & 7);
    }
  auto row_off_of = [&](int ks) { return row_off_w[ks % KSW] + (ks / KSW) * 128; };
  auto tr_off_of = [&](int sec, int db) { return tr_off_w[sec][db % DBW] + (db / DBW) * 128; };

  // Transposing read: within 16 lanes, lane 4 k + m supplies the address of four consecutive d of
  // key k (d quad m), and lane i receives element i % 4 of the pieces of lanes i / 4, 4 + i / 4,
  // 8 + i / 4, 12 + i / 4: four keys at d = 4 (i / 4) + i % 4 = i.  A lane of the 32x32x16 A
  // operand (d row lane % 32, key half lane / 32) takes two such reads: keys 4 half .. +3 and
  // 8 + 4 half .. +3 of a 16-key step, the order in which the S^T accumulator holds them.
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  auto tr_read = [&](const uint16_t* ptr) {
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(ptr));
    return __builtin_bit_cast(u32x2, v);
  };

  f32x16 oacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) zero(oacc[i]);
  float m_run = -INFINITY, l_run = 0.f;
  const float c = p.scale * kLog2eF;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int lim = ma.causal ? min(qrow, S - 1) : S - 1;
  // (window: keys below lo_w are dropped unless they are sink keys)
  const int lo_w = (FUNC && ma.window > 0) ? qrow - ma.window + 1 : (int)0x80000000;
  const int n_sink = FUNC ? ma.sink_keys : 0;

  auto mask_tile = [&](f32x16& s, int kv0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int kv = kv0 + (r >> 2) * 8 + half * 4 + (r & 3);
      // (bitwise on purpose: with || and && every element gets a cascade of branches)
      const bool dead = FUNC ? (kv > lim) | ((kv < lo_w) & (kv >= n_sink)) : kv > lim;
      s[r] = dead ? -INFINITY : s[r];
    }
  };
  // Bias of the score tile: lane = query row, 4 groups of 4 consecutive keys.  The resource starts
  // at this wavefront's first row of the (batch, head) plane and ends with its last one, so keys
  // past S read as zero (they are masked anyway).  Folded into the RAW scores, s += bias / scale,
  // so that everything downstream (reference tracking, lse) is the unbiased code.
  // A wavefront's 32 x 32 tile lands in its own 4 KB of LDS through the same kind of load as the
  // K / V tiles, 16 bytes per lane and instruction whatever the element size:
  //   float32     4 loads: load g, lane (row, half) -> keys 8 g + 4 half .. +3, read back by the same lane
  //   16 bits     2 loads: load i, lane (row, half) -> keys 16 i + 8 half .. +7; group g of lane (row, half)
  //               is the half-th 8 bytes of what lane (row, g % 2) fetched in load g / 2
  //   bool        1 load:  lane (row, half) -> keys 16 half .. +15; group g is dword 2 (g % 2) + half of
  //               what lane (row, g / 2) fetched
  // One buffer: the tile after next is requested right after this one has been read, and has a
  // whole iteration to land.  It is awaited by count: when the bias of tile t+1 is needed, the only
  // younger loads are those of the pair requested at the end of the previous iteration.
  uint32_t braw[4];
  float inv_scale = 0.f;
  const int bkind = BIASED ? __builtin_amdgcn_readfirstlane(ma.bias_kind) : 0;  // 0 none, 1 float32, 2 float16, 3 bfloat16, 4 bool
  const int b_esz = bkind == 1 ? 4 : bkind == 4 ? 1 : 2;
  const int b_rows = min(32, p.L - qw0);
  const u32x4 b_rsrc = descriptor((const char*)p.bias + (bkind ? (b * p.bias_sb + h * p.bias_sh + (int64_t)qw0 * p.bias_sl) * b_esz : 0),
                                  (bkind && b_rows > 0) ? (int)(((b_rows - 1) * p.bias_sl + p.S) * b_esz) : 0);
  const uint32_t b_voff = (uint32_t)((min(col, max(b_rows - 1, 0)) * p.bias_sl + half * (bkind == 1 ? 4 : bkind == 4 ? 16 : 8)) * b_esz);
  const int b_loads = bkind == 1 ? 4 : bkind == 4 ? 1 : 2;
  const unsigned char* const bias_w = (const unsigned char*)bias_lds + (BIASED ? wave * 4096 : 0);
  const uint32_t lds_b = (uint32_t)(uintptr_t)(lds_bytes)bias_w;
  if (bkind) inv_scale = 1.f / p.scale;
  // Dropout: the keep bytes of the tile, (B, Hq, L, S) contiguous, travel the way a bool bias does -
  // one load, lane (row, half) -> keys 16 half .. +15 - into 1 KB of the wavefront's own, beside the bias.
  const u32x4 kp_rsrc = descriptor((const char*)p.keep + (DROP ? (((int64_t)b * p.Hq + h) * p.L + qw0) * p.keep_ld : 0),
                                   (DROP && b_rows > 0) ? (int)((int64_t)b_rows * p.keep_ld) : 0);  // (whole rows: a dword that reaches past the records reads as zero)
  const uint32_t kp_voff = DROP ? (uint32_t)(min(col, max(b_rows - 1, 0)) * p.keep_ld + half * 16) : 0u;
  const unsigned char* const keep_w = keep_lds + (DROP ? wave * 1024 : 0);
  const uint32_t lds_kp = (uint32_t)(uintptr_t)(lds_bytes)keep_w;
  uint32_t kraw[4];
  auto load_bias = [&](int t) {
    if constexpr (BIASED) {
      if (bkind || DROP) {
        // (the reads of the tile before are behind this wavefront before its buffer is rewritten)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      }
      if (bkind) {
        const uint32_t g0 = b_voff + (uint32_t)((listed ? tile_of(min(t, nt - 1)) : t + skip) * BN * b_esz);
        tile_load(b_rsrc, g0, lds_b);
        if (b_loads > 1) tile_load(b_rsrc, g0 + 32, lds_b + 1024);
        if (b_loads > 2) {
          tile_load(b_rsrc, g0 + 64, lds_b + 2048);
          tile_load(b_rsrc, g0 + 96, lds_b + 3072);
        }
      }
      if constexpr (DROP) tile_load(kp_rsrc, kp_voff + (uint32_t)((t + skip) * BN), lds_kp);
    }
  };
  // (awaited: in the loop.  This wait also covers the pair that the iteration's barrier publishes.)
  auto apply_bias = [&](f32x16& sv, bool awaited) {
    if constexpr (BIASED) {
      if (awaited) wait_youngest_pair_only();
      if constexpr (DROP) {  // the tile's keep bytes, used where its probabilities are packed
#pragma unroll
        for (int g = 0; g < 4; ++g) kraw[g] = *(const uint32_t*)(keep_w + (col + 32 * (g >> 1)) * 16 + (g & 1) * 8 + half * 4);
      }
      if (bkind == 1) {
        // (head dim 256 has no registers to spare: one group at a time there)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const u32x4 w = *(const u32x4*)(bias_w + g * 1024 + lane * 16);
          // (vector elements are copied out first: a bit cast applied to the element itself reads element 0)
          const uint32_t u[4] = {w[0], w[1], w[2], w[3]};
#pragma unroll
          for (int r = 0; r < 4; ++r) sv[4 * g + r] = fmaf(__builtin_bit_cast(float, u[r]), inv_scale, sv[4 * g + r]);
          if constexpr (D > 128) __builtin_amdgcn_sched_barrier(0);
        }
      } else if (bkind == 4) {
#pragma unroll
        for (int g = 0; g < 4; ++g) braw[g] = *(const uint32_t*)(bias_w + (col + 32 * (g >> 1)) * 16 + (g & 1) * 8 + half * 4);
        // (a tile that the mask keeps whole - most tiles of a padding or window mask - costs four
        // compares instead of three instructions per score)
        const bool whole = braw[0] == 0x01010101u && braw[1] == 0x01010101u && braw[2] == 0x01010101u && braw[3] == 0x01010101u;
        if (__builtin_amdgcn_ballot_w64(!whole) != 0) {
          const bool none = (braw[0] | braw[1] | braw[2] | braw[3]) == 0u;  // ... and one that it drops whole, 16 moves
          if (__builtin_amdgcn_ballot_w64(!none) == 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sv[r] = -INFINITY;
          } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) sv[r] = ((braw[r >> 2] >> (8 * (r & 3))) & 0xffu) ? sv[r] : -INFINITY;
          }
        }
      } else if (bkind) {
        typedef __attribute__((ext_vector_type(2))) _Float16 h2;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const u32x2 w = *(const u32x2*)(bias_w + (g >> 1) * 1024 + (col + 32 * (g & 1)) * 16 + half * 8);
          const uint32_t u[2] = {w[0], w[1]};
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const uint32_t wide = (r & 1) ? (u[r >> 1] & 0xffff0000u) : (u[r >> 1] << 16);
            const float f = bkind == 2 ? (float)__builtin_bit_cast(h2, u[r >> 1])[r & 1] : __builtin_bit_cast(float, wide);
            sv[4 * g + r] = fmaf(f, inv_scale, sv[4 * g + r]);
          }
          if constexpr (D > 128) __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };

  // Score functors and document ids (MASK = 4): the raw score tile s (lane = query row, element r =
  // key 8 (r / 4) + 4 half + r % 4 of the tile) becomes mod(scale * s) / scale, so that everything
  // behind it - reference tracking, exp2 with the scale folded in, lse - is the common code.  Each
  // functor is a block of its own behind a uniform test.  The captured vectors are read with plain
  // loads (the wait in front of their use also covers the tile loads in flight: the price of a
  // functor that needs a vector per key); a document mask over sorted ids tests a whole tile with two
  // loads and compares element by element only in the tiles that straddle a document boundary.
  const float sm_inv_scale = SMOD ? 1.f / p.scale : 0.f;
  const float sm_slope = (SMOD && p.sm.alibi) ? p.sm.alibi[h] * sm_inv_scale : 0.f;
  const float* const sm_kb = (SMOD && p.sm.key_bias) ? p.sm.key_bias + (int64_t)h * p.S : nullptr;
  const float* const sm_kw = (SMOD && p.sm.key_weight) ? p.sm.key_weight + (int64_t)h * p.S : nullptr;
  const int32_t* const sm_dk = (SMOD && p.sm.doc_q && p.sm.doc_k) ? p.sm.doc_k + (int64_t)b * p.S : nullptr;
  // (this row's id is read again where a tile is compared element by element, rather than kept in a
  // register across the loop: such tiles are the few that straddle a document boundary)
  auto my_doc = [&]() { return sm_dk ? p.sm.doc_q[(int64_t)b * p.L + min(qrow, p.L - 1)] : 0; };
  // (which functors are on, as one scalar: the common cases - no functor at work in this tile, ALiBi
  // alone - then cost one or two taken branches per tile instead of one per functor)
  const int sm_on = SMOD ? __builtin_amdgcn_readfirstlane((sm_kw ? 1 : 0) | (sm_kb ? 2 : 0) | (p.sm.alibi ? 4 : 0) | (p.sm.softcap > 0.f ? 8 : 0)) : 0;
  auto apply_smod = [&](f32x16& sv, int ta) {
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
        for (int r = 0; r < 16; ++r) sv[r] *= w[r];
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
        for (int r = 0; r < 16; ++r) sv[r] = cap_s * tanh_fast(sv[r] * icap_s);
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

  // first tile that needs masking: the one that reaches this wavefront's first row on the causal
  // diagonal (qw0 is a multiple of BN), or a ragged last tile
  const int t_edge = min(ma.causal ? qw0 / BN : 0x7fffffff, (S % BN) ? S / BN : 0x7fffffff);
  // ... or, with a window, a tile that reaches below the window of this wavefront's last row and
  // is not made of sink keys alone.  (Stream position -> does the tile need masking.)
  auto edge = [&](int u) {
    const int ta = tile_of(u);
    bool e = ta >= t_edge;
    if constexpr (FUNC) {
      if (ma.window > 0) e |= ta * BN < qw_last - ma.window + 1 && ta * BN + BN > n_sink;
    }
    return e;
  };

  float m_new = -INFINITY, mc = 0.f, alpha = 1.f;
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
  // probability outgrew 2^kLazy-ish headroom: then, and only
  // then, the slow path finds the true tile maximum, raises the reference of every row that beat
  // it by more than kLazy in the exponent, rescales those rows' accumulators and redoes the
  // tile's probabilities.  Exact arithmetic: numerator and row sum always carry the same
  // reference, and lse = reference * scale + ln(sum).
  constexpr float kTrig = 8192.f;  // 16 probabilities of at most 2^kLazy stay below this
  auto raise_reference = [&](float t0) {
    const float tm = fmaxf(t0, __shfl_xor(t0, 32, 64));
    const bool up = (tm - m_run) * c > kLazy;  // false for NaN (-inf minus -inf)
    m_new = up ? tm : m_run;
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);
    mc = m_use * c;
    need_rescale = __builtin_amdgcn_ballot_w64(up) != 0;
  };

  // Softmax of one register pair, in three stages so that consecutive pairs can be staggered by
  // hand (the chain read S -> fma -> exp2 -> add/pack is strictly dependent and a wavefront
  // issues in order).  Pair j of 8: accumulator registers 2 j, 2 j + 1.
  float xs[2][2], pv[2][2];
  auto stage1 = [&](const f32x16& sv, int j) {
    xs[j & 1][0] = fmaf(sv[2 * j], c, -mc);
    xs[j & 1][1] = fmaf(sv[2 * j + 1], c, -mc);
  };
  auto stage2 = [&](int j) {
    pv[j & 1][0] = __builtin_amdgcn_exp2f(xs[j & 1][0]);
    pv[j & 1][1] = __builtin_amdgcn_exp2f(xs[j & 1][1]);
  };
  auto stage3 = [&](int j, uint32_t (&pk)[8], float& ps) {
    ps += pv[j & 1][0] + pv[j & 1][1];
    asm volatile("" : "+v"(ps));  // keeps the add in its slot (left alone it sinks below the loop body)
    if constexpr (DROP) {  // (the sum above keeps the dropped probabilities)
      const int r = 2 * j;
      const float k0 = (float)((kraw[r >> 2] >> (8 * (r & 3))) & 0xffu), k1 = (float)((kraw[r >> 2] >> (8 * (r & 3) + 8)) & 0xffu);
      pk[j] = Mma<T>::pack(pv[j & 1][0] * k0, pv[j & 1][1] * k1);
    } else {
      pk[j] = Mma<T>::pack(pv[j & 1][0], pv[j & 1][1]);
    }
  };
  // Pairs 0..3 hold the tile's first 16 keys (the first contraction step of P*V), pairs 4..7 the
  // last 16.  Four pairs are spread over the eight matrix ops of a phase:
  //   slot 2q: exp2 of pair q, scaling of pair q+1     slot 2q+1: sum and packing of pair q
  auto softmax_slot = [&](const f32x16& sv, int base, int slot, uint32_t (&pk)[8], float& ps) {
    const int q = slot >> 1;
    if ((slot & 1) == 0) {
      stage2(base + q);
      if (q + 1 < 4) stage1(sv, base + q + 1);
    } else {
      stage3(base + q, pk, ps);
    }
  };

  // ---- prologue ----------------------------------------------------------------------------------
  load_bias(0);
  request_k(0);
  request_pair(0);
  await_q();
  wait_all_tiles();
  __syncthreads();
  request_pair(1);
  request_pair(2);
  f32x16 s_a, s_b;
  uint32_t pk_a[8], pk_b[8];
  float ps_a = 0.f, ps_b = 0.f;
  {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const u32x4 a = *(const u32x4*)(k_dma + row_off_of(ks));
      s_a = Mma<T>::run(a, qf[ks], ks == 0 ? zero16 : s_a);
    }
    apply_bias(s_a, false);
    load_bias(1);
    apply_smod(s_a, tile_of(0));
    if (edge(0)) mask_tile(s_a, tile_of(0) * BN);
    raise_reference(tile_max(s_a));  // the first reference is the maximum of the first tile
    m_run = m_new;
#pragma unroll
    for (int j = 0; j < 4; ++j) {  // first half of tile 0
      stage1(s_a, j);
      stage2(j);
      stage3(j, pk_a, ps_a);
    }
  }
  __syncthreads();  // K buffer 0 is rewritten during the first iteration
  request_pair(3);
  // LDS operands travel through a four-entry register ring, three matrix ops ahead of their use;
  // the ring runs across iterations (the first three K fragments of a tile are requested at the
  // end of the previous iteration, right after the barrier that publishes the tile)
  u32x4 ring[8];
#pragma unroll
  for (int ks = 0; ks < AHEAD; ++ks)
    ring[ks] = *(const u32x4*)(k_dma + TILE + row_off_of(ks));

  // One pipelined iteration.  On entry scur holds S^T of tile t and pk / ps the probabilities of its
  // first 16 keys; snext receives S^T of tile t+1 and pkn / psn the first half of ITS probabilities.
  //   phase A   S^T(t+1) = K(t+1) Q^T on the matrix pipe  |  softmax of the last 16 keys of tile t
  //   check     sum of tile t against kTrig; rare slow path
  //   phase B   O^T += V^T(t) P^T(t) on the matrix pipe    |  softmax of the first 16 keys of tile
  //             t+1, request of tiles t+5 (K) and t+4 (V)
  auto iteration = [&](int t, auto tile_mod, f32x16& scur, f32x16& snext, uint32_t (&pk)[8], uint32_t (&pkn)[8],
                       float& ps, float& psn) {
    constexpr int tq = decltype(tile_mod)::value;  // t % 4, known at compile time
    // tiles t+1 (K, this iteration's scores), t+2 (K, published by this iteration's barrier), t (V)
    const uint16_t* kt = k_dma + ((tq + 1) & 3) * TILE;
    const uint16_t* kn = k_dma + ((tq + 2) & 3) * TILE;
    const uint16_t* vt = v_dma + tq * TILE;
    auto read_k = [&](int ks) { return *(const u32x4*)(kt + row_off_of(ks)); };
    auto read_kn = [&](int ks) { return *(const u32x4*)(kn + row_off_of(ks)); };
    auto read_v = [&](int i) {  // d block i % DB, 16-key step i / DB
      const u32x2 lo = tr_read(vt + tr_off_of(0, i % DB) + (i / DB) * 16 * D);
      const u32x2 hi = tr_read(vt + tr_off_of(1, i % DB) + (i / DB) * 16 * D);
      return u32x4{lo[0], lo[1], hi[0], hi[1]};
    };
    __builtin_amdgcn_sched_barrier(0);
    stage1(scur, 4);
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase A -------------------------------------------------------------------------------
    // (the scores are on the critical path - probabilities, then the second product wait for them -
    // while the second product only accumulates: the wavefront in phase A goes first when both of
    // a SIMD want to issue; measured 2 % on the whole kernel)
    if constexpr (!MASK) __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      // ring entry = (matrix op number within the tile, K ops first) mod 8
      if (ks + AHEAD < KS) ring[(ks + AHEAD) & 7] = read_k(ks + AHEAD);
      else ring[(ks + AHEAD) & 7] = read_v(ks + AHEAD - KS);
      snext = Mma<T>::run(ring[ks & 7], qf[ks], ks == 0 ? zero16 : snext);
#pragma unroll
      for (int hs = ks * 8 / KS; hs < (ks + 1) * 8 / KS; ++hs) softmax_slot(scur, 4, hs, pk, ps);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- check ---------------------------------------------------------------------------------
    // (NaN also lands here.)  A row whose keys so far were all masked has no reference yet
    // (m_run = -inf, probabilities formed against 0): it takes the slow path until a live key
    // sets one, or sums against 0 would be rescaled from -inf, or underflow, later.  Without a
    // mask key 0 is live for every row.
    bool trig = !(ps <= kTrig);
    if constexpr (MASK) trig |= m_run == -INFINITY;
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(trig) != 0, 0)) {
      raise_reference(tile_max(scur));
      if (need_rescale) {
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < DB; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
        m_run = m_new;
      }
      ps = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {  // the whole tile again, against the new reference
        stage1(scur, j);
        stage2(j);
        stage3(j, pk, ps);
      }
    }
    l_run += ps;
    psn = 0.f;
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase B -------------------------------------------------------------------------------
    if constexpr (!MASK) __builtin_amdgcn_s_setprio(0);
    // The first matrix op needs nothing of S^T(t+1): it is issued before anything reads that tile,
    // so the wait for the last op of phase A is spent on the matrix pipe.  The barrier sits two
    // slots before the end: by then every wavefront has stored its share of tiles t+2 (K) and
    // t+1 (V) and has issued its last read of V(t); behind it the first K fragments of the next
    // phase A are requested.  The eight half-steps of the softmax are spread over the slots, the
    // last one trailing the loop.
#pragma unroll
    for (int i = 0; i < NPV; ++i) {  // i = DB * (16-key step) + d block
      if (i == NPV - 2) {
        if constexpr (!BIASED) wait_oldest_pair();  // (with a bias: awaited together with the bias)
        __syncthreads();
      }
      if (i + AHEAD < NPV) ring[(KS + i + AHEAD) & 7] = read_v(i + AHEAD);
      if (i == NPV - 2) {
#pragma unroll
        for (int j = 0; j < (AHEAD + 1) / 2; ++j) ring[j] = read_kn(j);
      }
      if (i == NPV - 1) {
#pragma unroll
        for (int j = (AHEAD + 1) / 2; j < AHEAD; ++j) ring[j] = read_kn(j);
        request_pair(t + 4);
      }
      const int ks2 = i / DB, db = i % DB;
      const u32x4 b0 = {pk[ks2 * 4], pk[ks2 * 4 + 1], pk[ks2 * 4 + 2], pk[ks2 * 4 + 3]};
      oacc[db] = Mma<T>::run(ring[(KS + i) & 7], b0, oacc[db]);
      if (i == 0) {
        apply_bias(snext, true);
        load_bias(t + 2);
        apply_smod(snext, tile_of(t + 1));
        if (__builtin_expect(edge(t + 1), 0)) mask_tile(snext, tile_of(t + 1) * BN);  // rare
        stage1(snext, 0);
      }
      // half-steps 0 .. 6 spread over the slots (the last one trails the loop)
#pragma unroll
      for (int hs = (i == 0 ? 0 : max((i * 8) / NPV - 1, 0)); hs < max(((i + 1) * 8) / NPV - 1, 0); ++hs)
        softmax_slot(snext, 0, hs, pkn, psn);
      __builtin_amdgcn_sched_barrier(0);
    }
    softmax_slot(snext, 0, 7, pkn, psn);
  };
  // a wavefront whose rows lie above the causal diagonal of the remaining tiles only feeds LDS
  auto idle_step = [&](int t) {
    wait_oldest_pair();
    __syncthreads();
    request_pair(t + 4);
  };

  int t = 0;
  for (;;) {  // the buffer of a tile is a compile-time constant: four copies of the iteration
    if (t >= nt_w) break;
    iteration(t, std::integral_constant<int, 0>{}, s_a, s_b, pk_a, pk_b, ps_a, ps_b);
    if (++t >= nt_w) break;
    iteration(t, std::integral_constant<int, 1>{}, s_b, s_a, pk_b, pk_a, ps_b, ps_a);
    if (++t >= nt_w) break;
    iteration(t, std::integral_constant<int, 2>{}, s_a, s_b, pk_a, pk_b, ps_a, ps_b);
    if (++t >= nt_w) break;
    iteration(t, std::integral_constant<int, 3>{}, s_b, s_a, pk_b, pk_a, ps_b, ps_a);
    ++t;
  }
  for (; t < nt; ++t) idle_step(t);
  // (no load into LDS may be in flight when the workgroup's LDS is handed to the next one)
  wait_all_tiles();

  // ---- epilogue ------------------------------------------------------------------------------------
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  float lse_row = l_tot > 0.f ? m_run * p.scale + __builtin_logf(l_tot) : -INFINITY;
  if constexpr (DROP) inv *= p.keep_scale;
  if constexpr (FUNC) {
    // the sink logit joins the row's maximum and sum (flex_attention.py.jinja:1921-1923, :2134-2140)
    if (p.sink_logit) {
      const float z = sink_lse();
      if (z != -INFINITY) {
        const float mn = l_tot > 0.f ? m_run * p.scale : -INFINITY;  // the reference, natural-log domain
        const float mx = fmaxf(mn, z);
        const float f = l_tot > 0.f ? __expf(mn - mx) : 0.f;
        const float l2 = l_tot * f + __expf(z - mx);
        inv = f / l2;
        lse_row = mx + __builtin_logf(l2);
      }
    }
  }
  if constexpr (SPLITS) {
    if (p.split_tiles) {  // split keys: this part's normalised rows and their log-sum-exp, in float32, for the merge
      if (qrow < p.L) {
        const int64_t prow = (((int64_t)b * p.Hq + h) * p.n_split + split) * p.L + qrow;
        float* po = p.part_o + prow * drv;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int d = db * 32 + g * 8 + half * 4;
            if (d < drv)
              *(f32x4*)(po + d) = f32x4{oacc[db][g * 4] * inv, oacc[db][g * 4 + 1] * inv, oacc[db][g * 4 + 2] * inv, oacc[db][g * 4 + 3] * inv};
          }
        if (half == 0) p.part_lse[prow] = lse_row;
      }
      return;
    }
  }
  // A lane holds its query row in 8-byte pieces, 16 bytes apart: stored as they are, one
  // instruction writes 32 fragments of 16 bytes, and the stores of a workgroup's last tile,
  // which nothing overlaps, took 3 % of the kernel.  The tile goes through LDS instead (the
  // tile buffers are free now; 32 rows x D per wavefront, 16-byte chunks XOR-swizzled by row
  // against bank conflicts) and leaves as whole rows, 16 bytes per lane.
  __syncthreads();  // every wavefront is done with the K / V tiles
  uint16_t* ot = wave < WAVES / 2 ? k_dma + wave * 32 * D : v_dma + (wave - WAVES / 2) * 32 * D;
  constexpr int SW = CH < 16 ? CH - 1 : 15;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w;
      w[0] = Mma<T>::pack(oacc[db][g * 4 + 0] * inv, oacc[db][g * 4 + 1] * inv);
      w[1] = Mma<T>::pack(oacc[db][g * 4 + 2] * inv, oacc[db][g * 4 + 3] * inv);
      *(u32x2*)(ot + col * D + (((db * 4 + g) ^ (col & SW)) << 3) + half * 4) = w;
    }
  constexpr int RPI = 64 / CH;  // rows per store instruction
  const int rr = lane / CH, cc = lane % CH;
  uint16_t* obase = (uint16_t*)p.out + b * p.o_sb + h * p.o_sh + cc * 8;
#pragma unroll
  for (int i = 0; i < 32 / RPI; ++i) {
    const int r = i * RPI + rr;
    const u32x4 w = *(const u32x4*)(ot + r * D + ((cc ^ (r & SW)) << 3));
    if (qw0 + r < p.L && (!MASK || cc * 8 < drv)) *(u32x4*)(obase + (int64_t)(qw0 + r) * p.o_sl) = w;
  }
  if (qrow < p.L && p.lse && half == 0) p.lse[((int64_t)b * p.Hq + h) * p.L + qrow] = lse_row;
}

// The kernel of a variant.  A call whose bias comes with a verdict about it (see MaskArgs) is launched
// twice: as the variant with a bias (MASK = 2), and as the variant with key counts marked PATTERN.  The
// verdict lets one of them run: a bias that is the keep-everything or the causal pattern, with or
// without right padding, is never read - the PATTERN kernel generates it, at the speed of a call that
// was made with the causal flag - and any other bias leaves that kernel's workgroups nothing to do.
// (Two kernels rather than one that branches: both variants in one kernel need more scalar registers
// than there are, and the variant with a bias pays for its bias slot even when the slot is empty.)
template <typename T, int D, int WAVES, int MASK, bool PATTERN = false>
__global__ __launch_bounds__(64 * WAVES, D > 128 ? 1 : 8 / WAVES) void fwd_w32_kernel(FwdM p) {
  static_assert(!PATTERN || MASK == 1, "the pattern kernel is the variant with key counts");
  MaskArgs ma = mask_args_of(p);
  if constexpr (MASK == 2 || PATTERN) {
    if (verdict_pattern(p, ma) != PATTERN) return;
  } else if constexpr (MASK == 3) {
    verdict_pattern(p, ma);  // (dropout: one variant takes a bias or none, so the verdict is applied in place)
  }
  fwd_w32_body<T, D, WAVES, MASK>(p, ma);
}

// Merge of the parts of a call whose keys were split: out = sum_s w_s O_s with w_s = exp(lse_s - lse),
// lse = log sum_s exp(lse_s).  One workgroup per query row, one thread per output element.  The parts'
// lse are read side by side (a thread per part) and their weights left in LDS; the rows of the parts
// are then requested eight at a time: read one after the other, each of the two passes was a chain of
// trips to the L2, and a call with 64 parts spent as long here as in the attention kernel.
template <typename T>
__global__ __launch_bounds__(128) void fwd_split_merge_kernel(FwdM p) {
  constexpr int MAXP = 512;  // (fwd_w32_plan never makes more parts)
  __shared__ float w_s[MAXP];
  __shared__ float red_s[4];
  const int64_t row = blockIdx.x;  // (b * Hq + h) * L + l
  const int l = (int)(row % p.L);
  const int64_t bh = row / p.L;
  const int b = (int)(bh / p.Hq), h = (int)(bh % p.Hq);
  const float* pl = p.part_lse + bh * p.n_split * p.L + l;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float ls[MAXP / 128];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < MAXP / 128; ++i) {
    const int sp = tid + 128 * i;
    ls[i] = sp < p.n_split ? pl[(int64_t)sp * p.L] : -INFINITY;
    m = fmaxf(m, ls[i]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  if (lane == 0) red_s[wave] = m;
  __syncthreads();
  m = fmaxf(red_s[0], red_s[1]);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < MAXP / 128; ++i) {
    const int sp = tid + 128 * i;
    const float w = ls[i] == -INFINITY ? 0.f : __expf(ls[i] - m);  // (a part without keys: weight 0, its rows were never written)
    w_s[sp] = w;  // (every slot: the loop below multiplies the slots past the last part by a zero, which a stale NaN would survive)
    sum += w;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
  if (lane == 0) red_s[2 + wave] = sum;
  __syncthreads();
  sum = red_s[2] + red_s[3];
  float acc[2] = {0.f, 0.f};
  const int d = tid;  // columns d and d + 128 (head dims up to 256)
  const float* po = p.part_o + (bh * p.n_split * p.L + l) * p.dv_real;
  const int64_t part_stride = (int64_t)p.L * p.dv_real;
  for (int s0 = 0; s0 < p.n_split; s0 += 8) {
    float x[2][8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool on = s0 + j < p.n_split && w_s[min(s0 + j, MAXP - 1)] > 0.f;
#pragma unroll
      for (int i = 0; i < 2; ++i) x[i][j] = (on && d + 128 * i < p.dv_real) ? po[(s0 + j) * part_stride + d + 128 * i] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int i = 0; i < 2; ++i) acc[i] = fmaf(s0 + j < p.n_split ? w_s[min(s0 + j, MAXP - 1)] : 0.f, x[i][j], acc[i]);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
    if (d + 128 * i < p.dv_real) {
      T* o = (T*)p.out + b * p.o_sb + h * p.o_sh + (int64_t)l * p.o_sl + d + 128 * i;
      *(uint16_t*)o = (uint16_t)Mma<T>::pack(sum > 0.f ? acc[i] / sum : 0.f, 0.f);
    }
  if (d == 0 && p.lse) p.lse[row] = sum > 0.f ? m + __builtin_logf(sum) : -INFINITY;
}

// one instantiation; head dim 256 and the variant with a bias need more than the 64 KB of LDS a kernel may declare
template <typename T, int D, int WAVES, int MASK, bool PATTERN = false>
int launch_one(const FwdM& g, dim3 grid, hipStream_t s) {
  int bytes = 0;
  if constexpr (D > 128 || MASK == 2 || MASK == 3) {
    // (four buffers per operand, 4 KB of bias tile per wavefront, and the tile list of a call with a skip table)
    constexpr int kBase = 2 * 4 * BN * D * 2 + (MASK >= 2 ? WAVES * 4096 : 0) + (MASK == 3 ? WAVES * 1024 : 0);
    constexpr int kBytes = kBase + (MASK == 2 ? 2048 + 16 : 0);
    static LdsOnce once;
    const hipError_t attr = reserve_lds(once, (const void*)fwd_w32_kernel<T, D, WAVES, MASK, PATTERN>, kBytes);
    if (attr != hipSuccess) {
      set_error("SDPA: cannot reserve %d bytes of LDS for fwd_w32_kernel: %s", kBytes, hipGetErrorString(attr));
      return MI355_SDPA_ERR_LAUNCH;
    }
    bytes = (MASK == 2 && g.live_tiles) ? kBytes : kBase;
  }
  hipLaunchKernelGGL((fwd_w32_kernel<T, D, WAVES, MASK, PATTERN>), grid, dim3(64 * WAVES), bytes, s, g);
  return MI355_SDPA_OK;
}
template <typename T, int D, int WAVES>
int launch_mask(const FwdM& g, int mask, dim3 grid, hipStream_t s) {
  if (mask == 4) return launch_one<T, D, WAVES, 4>(g, grid, s);
  if (mask == 3) return launch_one<T, D, WAVES, 3>(g, grid, s);
  if (mask == 2) {
    if (g.verdict) {  // (see fwd_w32_kernel)
      if (int rc = launch_one<T, D, WAVES, 1, true>(g, grid, s)) return rc;
    }
    return launch_one<T, D, WAVES, 2>(g, grid, s);
  }
  if (mask == 1) return launch_one<T, D, WAVES, 1>(g, grid, s);
  return launch_one<T, D, WAVES, 0>(g, grid, s);
}
template <typename T>
int launch_dims(const FwdM& g, int head_dim, int waves, int mask, dim3 grid, hipStream_t s) {
  if (head_dim == 256) return launch_mask<T, 256, 4>(g, mask, grid, s);  // 128-row workgroups only
  if (head_dim == 128) return waves == 8 ? launch_mask<T, 128, 8>(g, mask, grid, s) : launch_mask<T, 128, 4>(g, mask, grid, s);
  return waves == 8 ? launch_mask<T, 64, 8>(g, mask, grid, s) : launch_mask<T, 64, 4>(g, mask, grid, s);
}

}  // namespace

// Grouped mode: every head of a kv group in one workgroup when their rows fit its wavefronts (four
// wavefronts where they do, eight otherwise; for up to 32 query rows also a share of the group's
// heads per workgroup) and there is no dropout mask and no bias that depends
// on the head (with one that does not, every wavefront of the workgroup arrives at the same key count
// when it trims a keep-mask per key, and so at the same number of tiles).  When that leaves most of
// the 256 compute units without a workgroup and the key loop is long, the keys are split: at least 8
// tiles per part, about two workgroups per compute unit.
void fwd_w32_plan(FwdM& g, int head_dim, int& waves) {
  if (g.d_real <= 0 || g.d_real > head_dim) g.d_real = head_dim;
  if (g.dv_real <= 0 || g.dv_real > head_dim) g.dv_real = g.d_real;
  if (head_dim == 256) waves = 4;
  const int rep = g.Hq / g.Hkv;
  g.grouped = 0, g.split_tiles = 0, g.n_split = 1;
  // (one head per kv head counts too: nothing is shared then, but such a call can split its keys)
  if ((g.bias_kind == 0 || g.bias_sh == 0) && g.keep_scale == 0.f && !g.live_tiles) {
    const int blocks32 = (g.L + 31) / 32;  // 32-row blocks per head
    if (4 % rep == 0 && blocks32 * rep <= 4) waves = 4, g.grouped = rep;
    else if (head_dim != 256 && 8 % rep == 0 && blocks32 * rep <= 8) waves = 8, g.grouped = rep;
    else if (blocks32 == 1) {
      // a decode step with more heads per kv head than wavefronts, or a number of them that does not
      // divide 8: 8, 4, 2 or 1 of them per workgroup, whichever is the most that divides it
      int d = head_dim != 256 ? 8 : 4;
      while (rep % d != 0) d >>= 1;
      waves = d == 8 ? 8 : 4, g.grouped = d;
    }
  }
  // (the variant with a bias splits at head dims up to 128 only)
  if (g.grouped && (head_dim <= 128 || g.bias_kind == 0) && !g.causal && g.window == 0 && !g.sink_logit && !g.sm.any) {
    const int64_t groups = (int64_t)g.B * g.Hkv * (g.Hq / g.Hkv / g.grouped);
    const int nt = (g.S + BN - 1) / BN;
    const int want = (int)std::min<int64_t>((512 + groups - 1) / groups, nt / 8);  // (at most 512 parts: fwd_split_merge_kernel's limit)
    if (groups < 256 && want >= 2) {
      g.split_tiles = (nt + want - 1) / want;
      g.n_split = (nt + g.split_tiles - 1) / g.split_tiles;
    }
  }
  g.n_qt = g.grouped ? 1 : (g.L + 32 * waves - 1) / (32 * waves);
  if (g.grouped) g.verdict = nullptr;  // (few rows: the mask is taken as it is)
}

size_t fwd_w32_workspace(const FwdM& g0, int head_dim, int waves) {
  FwdM g = g0;
  fwd_w32_plan(g, head_dim, waves);
  if (!g.split_tiles) return 0;
  return (size_t)g.B * g.Hq * g.n_split * g.L * (g.dv_real + 1) * sizeof(float);
}

int launch_fwd_mfma_w32(const FwdM& g0, int dtype, int head_dim, int waves, hipStream_t s) {
  FwdM g = g0;
  fwd_w32_plan(g, head_dim, waves);
  if (g.split_tiles) {  // (the caller's workspace: too small or absent, and the call runs unsplit)
    const size_t rows = (size_t)g.B * g.Hq * g.n_split * g.L;
    if (g.part_o && g.n_split <= 512 && g.part_bytes >= rows * (g.dv_real + 1) * sizeof(float)) g.part_lse = g.part_o + rows * g.dv_real;
    else g.split_tiles = 0, g.n_split = 1;
  }
  const int64_t blocks = g.grouped ? (int64_t)g.B * (g.Hq / g.grouped) * g.n_split : (int64_t)g.B * g.Hq * g.n_qt;
  if (blocks == 0) return MI355_SDPA_OK;
  if (blocks > 0x7fffffff) {
    set_error("SDPA: too many query tiles (%lld)", (long long)blocks);
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  const dim3 grid((unsigned)blocks);
  // kernel variant: 3 with a keep-mask (and a bias or none), 2 with a bias, 1 with key counts or rows narrower than the kernel's head dim
  if (g.keep_scale != 0.f && (!g.keep || g.live_tiles)) {
    set_error("SDPA: dropout in fwd_w32_kernel needs a keep-mask and no tile table");
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  if (g.sm.any && (g.bias_kind != 0 || g.keep_scale != 0.f)) {
    set_error("SDPA: score functors in fwd_w32_kernel go with no bias and no dropout");
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  const int mask = g.sm.any ? 4 : g.keep_scale != 0.f ? 3 : g.bias_kind != 0 ? 2 : (g.kv_lens != nullptr || g.d_real != head_dim || g.dv_real != head_dim || g.window > 0 || g.sink_logit || g.split_tiles) ? 1 : 0;
  int rc = dtype == MI355_SDPA_BF16 ? launch_dims<bf16_t>(g, head_dim, waves, mask, grid, s)
                                          : launch_dims<f16_t>(g, head_dim, waves, mask, grid, s);
  if (rc != MI355_SDPA_OK) return rc;
  rc = check_launch("fwd_w32_kernel");
  if (rc != MI355_SDPA_OK || !g.split_tiles) return rc;
  const dim3 rows((unsigned)((int64_t)g.B * g.Hq * g.L));
  if (dtype == MI355_SDPA_BF16) hipLaunchKernelGGL((fwd_split_merge_kernel<bf16_t>), rows, dim3(128), 0, s, g);
  else hipLaunchKernelGGL((fwd_split_merge_kernel<f16_t>), rows, dim3(128), 0, s, g);
  return check_launch("fwd_split_merge_kernel");
}

}  // namespace mi355
