// Flash-attention backward, dK and dV, for gfx950, head dim 64 or 128, bf16/f16.
//
// One workgroup = 8 wavefronts = 128 keys of one (batch, kv head); it loops over the query
// heads of the group (the GQA sum of decompositions.py:2595-2598 happens in registers) and over
// 64-row query tiles.  The four matrix products of a tile are split between TWO wavefronts per
// 32-key block, which sit on the same SIMD:
//
//   role A   S = Q K^T            P = exp2(c S - lse)            dV^T += dO^T P
//   role B   dS = P (dP - delta)  dK^T += Q^T dS                 dP = dO V^T of the next tile
//
// so that each wavefront holds one accumulator (64 registers) and one operand (K or V
// fragments, 32 registers) and fits in 256 registers: with two wavefronts per SIMD the vector
// work of one issues under the matrix ops of the other (a wavefront issues at most one
// instruction every four cycles, so a single wavefront per SIMD cannot keep both pipes busy).
// Role B needs P from role A: A leaves it in LDS (packed to the input dtype, as it is fed to the
// matrix pipe), and B finishes a tile ONE ITERATION BEHIND A, so the only synchronisation is the
// one barrier per tile that the staging needs anyway; B's vector work then runs under A's first
// matrix ops and A's under B's.  Three tile buffers are live: the one being staged, A's and B's.
//
// Q and dO tiles sit in LDS row-major as they sit in memory; the transposed operands (dO^T, Q^T)
// come out of the transposing LDS read ds_read_b64_tr_b16, so nothing is transposed on the
// vector unit.  Math follows torch_neuronx/_sdpa_math.py:98-176: float32 accumulation, rows
// with lse = -inf give zero gradients, scale multiplies dK once at the end.
#include <type_traits>

#include "bwd_mfma.h"

namespace mi355 {
namespace {

constexpr int BQ = 64, BK = 128;
template <int D>
constexpr int smem_bytes() {  // three Q and three dO tiles, two P hand-over buffers, lse / delta rows
  return 2 * 3 * BQ * D * 2 + 2 * 4 * 64 * 16 * 4 + 2 * 3 * BQ * 4;
}

// MASK >= 1 also serves head dims below D (multiples of 8): the missing tail of every row counts
// as zeros.
// MASK = 1: per-batch key counts and a bias / bool keep-mask that depends on the key only (a lane
// is a key: one register);  MASK = 2: a bias / keep-mask with a row per query as well (one element
// per score, fetched by role A ahead of the tile's matrix ops);  MASK = 4: MASK = 1 plus the score
// functors and document ids of score_mod.h: role A rewrites its score tile in a block of its own
// and hands P times the derivative of the functors to role B, which forms dS from it.
template <typename T, int D, int MASK>
__device__ __forceinline__ void bwd_dkdv_w32_body(const BwdM& p, const MaskArgs ma) {
  constexpr int KS = D / 16, DB = D / 32, CH = D / 8;
  constexpr int TILE = BQ * D;           // tiles are XOR swizzled, not padded: see tile_swz
  constexpr int NCH = BQ * CH / 512;     // 16-byte chunks of a tile per thread
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint16_t* const q_t = (uint16_t*)smem;          // [3][TILE]
  uint16_t* const do_t = q_t + 3 * TILE;          // [3][TILE]
  uint32_t* const pex = (uint32_t*)(do_t + 3 * TILE);  // [2][4 key blocks][64 lanes][16]
  float* const lse_s = (float*)(pex + 2 * 4 * 1024);   // [3][BQ]
  float* const dl_s = lse_s + 3 * BQ;                  // [3][BQ]
  int32_t* const doc_s = (int32_t*)(dl_s + 3 * BQ);     // [3][BQ] document ids of the tile's rows (MASK = 4)
  uint32_t* const live_s = (uint32_t*)(dl_s + 3 * BQ);  // [heads of the group][words]: query tiles with a kept score (skip table; MASK = 2)
  uint16_t* const items_s = (uint16_t*)(live_s + 256);  // [1024] live items, and their count behind them

  const int streams = p.B * p.Hkv;
  // Split items: a key block's heads go to parts_h workgroups, and their query tiles to parts / parts_h.
  // A (batch, kv head, share of the heads) keeps its place in the launch order modulo the number of
  // such streams - and with that its XCD, when that number is a multiple of 8 - over all key blocks
  // and tile shares: the workgroups that walk the same Q / dO tiles meet in one L2.
  int kt, st, ph = 0, pq = 0;
  if (p.parts > 1) {
    const int vstreams = streams * p.parts_h;
    const int v = blockIdx.x % vstreams, rest = blockIdx.x / vstreams;
    kt = rest % p.n_kt, pq = rest / p.n_kt;
    st = v / p.parts_h, ph = v % p.parts_h;
  } else {
    kt = blockIdx.x / streams;  // low key tiles see the most queries under a causal mask: first
    st = blockIdx.x % streams;
  }
  const int part = pq * p.parts_h + ph;  // its rows among the partial results
  const int b = st / p.Hkv, hk = st % p.Hkv;
  if constexpr (MASK == 4) {
    if (p.kt_order) kt = p.kt_order[b * p.n_kt + kt];  // (the batch's key blocks, heaviest first)
  }
  const int rep_all = p.Hq / p.Hkv;
  const int rep = p.parts > 1 ? rep_all / p.parts_h : rep_all;  // heads of the group that this workgroup walks
  const int h0 = ph * rep;                                       // the first of them
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int role = wave >> 2, kb = wave & 3;  // wavefronts w and w + 4 share a SIMD and a key block
  const int col = lane & 31, half = lane >> 5;
  const int k0 = kt * BK, kw0 = k0 + kb * 32;
  const int key = kw0 + col;

  const int dr = MASK ? p.d_real : D;  // elements per row that exist
  int S = p.S;  // keys of this batch that take part
  if constexpr (MASK) {
    if (ma.kv_lens) S = min(S, max(ma.kv_lens[b], 0));
  }
  // this lane's key as B operand: K fragments for S = Q K^T (role A), V fragments for dP = dO V^T (role B)
  u32x4 frag[KS];
  {
    const int kc = max(min(key, S - 1), 0);  // (a live row: rows past the batch's keys may hold anything)
    const uint16_t* r = role ? (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh + (int64_t)kc * p.v_sl
                             : (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh + (int64_t)kc * p.k_sl;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (!MASK || half * 8 + ks * 16 < dr) frag[ks] = *(const u32x4*)(r + half * 8 + ks * 16);
      else frag[ks] = u32x4{0u, 0u, 0u, 0u};
    }
    // (the fragments are awaited here, once: left pending, their first use inside the tile loop
    // becomes a wait for every outstanding load there, the tile loads of the next items included)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(frag[ks]));
  }

  // sliding window (masked variant without a per-score bias): rows past the window of the block's last
  // key see none of its keys, unless the block holds sink keys
  constexpr bool FUNC = MASK == 1 || MASK == 4;
  constexpr bool SMOD = MASK == 4;  // score functors, document ids
  // MASK = 3 is dropout, MASK = 5 dropout with a bias (an instance of its own: the bias and the keep
  // bytes of a tile together are more than the registers hold at head dim 128, and a call without a
  // bias need not pay for that): the (B, Hq, L, S) keep-mask is fetched like a bool bias, beside the
  // bias, by the wavefronts that form the probabilities.  They feed dV with the kept probabilities and hand all of them to the dK
  // wavefronts, the dropped ones with the sign bit set (a probability is never negative): dP is
  // multiplied by keep / (1 - p) there (torch_neuronx/_sdpa_math.py:36-48, :154-158).
  constexpr bool HASB = MASK == 2 || MASK == 5, DROP = MASK == 3 || MASK == 5;  // a bias per score; a keep-mask
  constexpr bool BIASED = HASB || DROP;
  const int W = FUNC ? ma.window : 0, n_sink = FUNC ? ma.sink_keys : 0;
  // the query rows that see this lane's key are first_q .. past_q - 1: from the key itself on under a
  // causal mask, none for a key past the batch's count, up to the end of the key's window unless it is a sink
  const int first_q = key >= S ? INT_MAX : ma.causal ? key : INT_MIN;
  const int past_q = (W > 0 && key >= n_sink) ? key + W : INT_MAX;
  const bool listed = MASK == 2 && p.live_t != nullptr;
  const int nqs = (p.L + BQ - 1) / BQ;
  int qs_begin = ma.causal ? min(k0 / BQ, nqs) : 0;
  int qs_end = (W > 0 && k0 >= n_sink) ? max(min(nqs, (k0 + BK + W - 2) / BQ + 1), qs_begin) : nqs;
  // document ids (MASK = 4): this lane's key id; with ids sorted along the sequence the rows whose id
  // lies between the ids of the block's first and last key are one run, found by two searches over
  // doc_q, and only the query tiles that touch it are walked
  const bool sm_doc = SMOD && p.sm.doc_q && p.sm.doc_k;
  // (every load of the searches' first round goes out before anything waits: one trip to memory)
  const bool sm_runs = SMOD && sm_doc && p.sm.doc_sorted && k0 < S;
  int sm_first = 0, sm_d_lo = 0, sm_d_hi = 0;
  if constexpr (SMOD) {
    if (sm_runs) {
      sm_first = doc_first_samples(p.sm.doc_q + (int64_t)b * p.L, p.L, lane);
      sm_d_lo = p.sm.doc_k[(int64_t)b * p.S + k0], sm_d_hi = p.sm.doc_k[(int64_t)b * p.S + min(k0 + BK, S) - 1];
    }
  }
  const int sm_dk = sm_doc ? p.sm.doc_k[(int64_t)b * p.S + max(min(key, S - 1), 0)] : 0;
  const int sm_dk_first = __builtin_amdgcn_readlane(sm_dk, 0), sm_dk_last = __builtin_amdgcn_readlane(sm_dk, 31);
  // (the rows that this wavefront's 32 keys can see: the run of doc_q with their ids)
  int doc_run_w[2] = {0, 0x7fffffff};
  if constexpr (SMOD) {
    if (sm_runs) {
      int run[2];
      doc_runs(p.sm.doc_q + (int64_t)b * p.L, p.L, sm_d_lo, sm_d_hi, sm_dk_first, sm_dk_last, run, doc_run_w, lane, sm_first);
      qs_begin = max(qs_begin, run[0] / BQ);
      qs_end = run[1] > run[0] ? max(min(qs_end, (run[1] + BQ - 1) / BQ), qs_begin) : qs_begin;
    }
  }
  const int per_head = qs_end - qs_begin;
  int n_items = (MASK && k0 >= S) ? 0 : rep * per_head;  // no live key in this tile: zeros
  // Items run query tile by query tile from the LAST tile down, the group's heads inside.  The
  // workgroups of a (batch, kv head) share an XCD, and those that start together - under a causal
  // mask they need different numbers of tiles, all ending with the last one - then ask for the same
  // Q / dO tile at about the same time: one of them brings it into the XCD's L2, the others find it
  // there.  (Head by head and upwards from each block's own first tile, the workgroups are at
  // different tiles all the time and each streams Q / dO from memory on its own: 1.7 GB of fetches
  // per call on a (2, 32/8, 4096, 128) problem, against 0.13 GB of Q and dO.)
  // (with a skip table: the items whose tile holds a kept score, listed in LDS before the first item)
  bool compact = false;
  int it0 = 0;  // first item of this workgroup's part
  auto item_id = [&](int it) {
    if constexpr (MASK == 2) return compact ? __builtin_amdgcn_readfirstlane((int)items_s[it + it0]) : it + it0;
    else return it + it0;
  };
  // (item / rep as a multiply-high by ceil(2^32 / rep), exact while item * rep < 2^32: these two are
  // evaluated many times per item, on the scalar unit, and a division there is twenty instructions)
  const uint32_t rep_inv = (uint32_t)((0x100000000ull + (uint32_t)rep - 1) / (uint32_t)rep);
  auto item_tile = [&](int it) { return rep == 1 ? item_id(it) : (int)__umulhi((uint32_t)item_id(it), rep_inv); };  // (2^32 does not fit)
  auto item_head = [&](int it) { return hk * rep_all + h0 + (item_id(it) - item_tile(it) * rep); };
  auto item_q0 = [&](int it) { return (qs_end - 1 - item_tile(it)) * BQ; };

  // ---- staging: every thread moves two 16-byte chunks of the Q tile and two of the dO tile ------
  // Buffer resources end with the last row of the batch (the tile offset travels in the vector
  // offset, which is the part the hardware checks against that bound): rows past L read as zeros
  // or as another head's rows, and are switched off through lse = +inf.
  const int64_t q_ext = ((int64_t)(p.Hq - 1) * p.q_sh + (int64_t)(p.L - 1) * p.q_sl + dr) * 2;
  const int64_t go_ext = ((int64_t)(p.Hq - 1) * p.go_sh + (int64_t)(p.L - 1) * p.go_sl + dr) * 2;
  auto descriptor = [&](const void* base, int64_t bytes) {  // raw buffer resource, in scalar registers
    const uint64_t a = (uint64_t)base;
    return u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a),
                 (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu)),
                 (uint32_t)__builtin_amdgcn_readfirstlane((int)bytes), 0x00020000u};
  };
  const u32x4 q_rsrc = descriptor((const uint16_t*)p.q + b * p.q_sb, q_ext);
  const u32x4 go_rsrc = descriptor((const uint16_t*)p.go + b * p.go_sb, go_ext);
  // row statistics of this batch (written by bwd_delta_kernel): (Hq, L) floats each
  const u32x4 lse_rsrc = descriptor(p.lse2 + (int64_t)b * p.Hq * p.L, (int64_t)p.Hq * p.L * 4);
  const u32x4 dl_rsrc = descriptor(p.delta + (int64_t)b * p.Hq * p.L, (int64_t)p.Hq * p.L * 4);
  const u32x4 doc_rsrc = descriptor(sm_doc ? p.sm.doc_q + (int64_t)b * p.L : nullptr, sm_doc ? (int64_t)p.L * 4 : 0);
  // The tiles go from global memory straight into LDS (buffer loads with the LDS bit: no trip
  // through registers, no LDS store instructions).  The loads are written as inline assembly: the
  // compiler's own form of them makes it wait for all outstanding loads before the next LDS read
  // of any address, which would expose the whole memory latency at the top of every iteration.
  // Their completion is awaited by hand, before the barrier that publishes the tile (wait_tiles).  Such a load writes 64 x 16 contiguous bytes, one
  // chunk per lane in lane order, at an LDS address that is uniform for the wavefront: 1 KB = 1024 / (2 D)
  // whole tile rows.  The swizzle is therefore applied on the global side: the lane that owns LDS
  // chunk position c of row r fetches the row's chunk c ^ tile_swz(r).
  const int s_row = tid / CH;                       // rows s_row + n * 512 / CH
  const int s_ch = (tid % CH) ^ tile_swz<D>(s_row);  // (row s_row + 32 has the swizzle of row s_row)
  uint32_t q_off[NCH], go_off[NCH];
#pragma unroll
  for (int n = 0; n < NCH; ++n) {
    q_off[n] = (uint32_t)(((s_row + (512 / CH) * n) * p.q_sl + s_ch * 8) * 2);
    go_off[n] = (uint32_t)(((s_row + (512 / CH) * n) * p.go_sl + s_ch * 8) * 2);
    if (MASK && s_ch * 8 >= dr) q_off[n] = go_off[n] = 0x7ffffff0u;  // past the end of a narrow row: reads as zeros
  }
  typedef __attribute__((address_space(3))) unsigned char* lds_bytes;
  // LDS byte addresses of this wavefront's 1 KB inside a pass of 512 chunks, for tile buffer 0
  const uint32_t lds_q = (uint32_t)(uintptr_t)(lds_bytes)q_t + wave * 1024;
  const uint32_t lds_do = (uint32_t)(uintptr_t)(lds_bytes)do_t + wave * 1024;
  auto tile_load = [&](const u32x4& rsrc, uint32_t voffset, uint32_t lds_addr) {
    // (m0 holds the LDS address of such a load, one wait state after it is written; it is declared
    // clobbered, so the compiler keeps no value of its own in m0 across the statement)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :: "s"(__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(voffset), "s"(rsrc) : "memory", "m0");
  };
  const uint32_t lds_lse = (uint32_t)(uintptr_t)(lds_bytes)lse_s, lds_dl = (uint32_t)(uintptr_t)(lds_bytes)dl_s;
  const uint32_t lds_doc = (uint32_t)(uintptr_t)(lds_bytes)doc_s;
  auto row_load = [&](const u32x4& rsrc, uint32_t voffset, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds"
                 :: "s"(__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(voffset), "s"(rsrc) : "memory", "m0");
  };
  auto wait_tiles = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
  auto load_item = [&](int it, int buf) {  // the tiles of item `it` into tile buffer `buf`
    const int h = item_head(it), q0 = item_q0(it);
    const uint32_t qb = (uint32_t)((h * p.q_sh + (int64_t)q0 * p.q_sl) * 2);
    const uint32_t gb = (uint32_t)((h * p.go_sh + (int64_t)q0 * p.go_sl) * 2);
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
      tile_load(q_rsrc, q_off[n] + qb, lds_q + (uint32_t)(buf * TILE * 2 + n * 8192));
      tile_load(go_rsrc, go_off[n] + gb, lds_do + (uint32_t)(buf * TILE * 2 + n * 8192));
    }
    if (wave == 0) {  // the 64 rows' statistics: one dword per lane, straight into LDS as well
      const uint32_t off = (uint32_t)((h * p.L + q0 + lane) * 4);
      row_load(lse_rsrc, off, lds_lse + (uint32_t)(buf * BQ * 4));
      row_load(dl_rsrc, off, lds_dl + (uint32_t)(buf * BQ * 4));
      if constexpr (SMOD) {
        if (sm_doc) row_load(doc_rsrc, (uint32_t)((q0 + lane) * 4), lds_doc + (uint32_t)(buf * BQ * 4));
      }
    }
  };
  // Rows past L of a head's last tile hold another head's rows and statistics (or zeros): they are
  // switched off through lse = +inf and delta = 0, written over what the loads brought once those
  // have landed (wait_tiles first).
  auto finish_item = [&](int it, int buf) {
    const int q0 = item_q0(it);
    if (q0 + BQ > p.L && tid < BQ && q0 + tid >= p.L) lse_s[buf * BQ + tid] = INFINITY, dl_s[buf * BQ + tid] = 0.f;
  };

  // Transposing read: within 16 lanes, lane 4 k + m supplies the address of four consecutive d of
  // row k (d quad m), and lane i receives element i % 4 of the pieces of lanes i / 4, 4 + i / 4,
  // 8 + i / 4, 12 + i / 4: four rows at d = i.  A lane of the 32x32x16 A operand (d row lane % 32,
  // row half lane / 32) takes two such reads: rows 4 half .. +3 and 8 + 4 half .. +3 of a 16-row
  // step, the order in which the score accumulators hold them.
  // The element offsets inside a tile depend on the swizzle of the row a lane reads, which is not
  // additive in the d block / contraction step: one offset register per combination.
  const int tr_jj = lane & 15, tr_g = lane >> 4;
  int tr_off[2][DB];  // [second read of a pair][d block], without the 16-row step (a multiple of 16 rows)
#pragma unroll
  for (int sec = 0; sec < 2; ++sec)
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int row = 8 * sec + (tr_g >> 1) * 4 + (tr_jj >> 2);  // within the 16-row step
      const int d = db * 32 + 16 * (tr_g & 1) + 4 * (tr_jj & 3);
      tr_off[sec][db] = row * D + (((d >> 3) ^ tile_swz<D>(row)) << 3) + (d & 7);
    }
  int row_off[KS];  // [contraction step], without the 32-row block
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) row_off[ks] = col * D + (((2 * ks + half) ^ tile_swz<D>(col)) << 3);
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  auto tr_read = [&](const uint16_t* ptr) {
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(ptr));
    return __builtin_bit_cast(u32x2, v);
  };
  // operand i = DB * (16-row step) + d block of the transposed tile
  auto read_cols = [&](const uint16_t* tile, int i) {
    const u32x2 lo = tr_read(tile + tr_off[0][i % DB] + (i / DB) * 16 * D);
    const u32x2 hi = tr_read(tile + tr_off[1][i % DB] + (i / DB) * 16 * D);
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
  };
  // operand i = KS * (32-row block) + contraction step of the row-major tile
  auto read_rows = [&](const uint16_t* tile, int i) {
    return *(const u32x4*)(tile + row_off[i % KS] + (i / KS) * 32 * D);
  };

  f32x16 acc[DB];  // dV^T (role A) or dK^T (role B): d rows x this lane's key
#pragma unroll
  for (int i = 0; i < DB; ++i) zero(acc[i]);
  const float c = p.scale * kLog2eF;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  constexpr int AHEAD = 4;

  // scores of the 64 x 32 tile: sc[mq] = rows(tile)[32 mq ..] * frag
  auto scores = [&](const uint16_t* tile, f32x16 (&sc)[2]) {
    u32x4 ring[8];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) ring[i] = read_rows(tile, i);
#pragma unroll
    for (int i = 0; i < 2 * KS; ++i) {
      if (i + AHEAD < 2 * KS) ring[(i + AHEAD) & 7] = read_rows(tile, i + AHEAD);
      sc[i / KS] = Mma<T>::run(ring[i & 7], frag[i % KS], (i % KS) == 0 ? zero16 : sc[i / KS]);
    }
  };
  // acc += cols(tile)^T * pk, pk = the 64 x 32 tile of P or dS packed from the accumulator layout
  auto accumulate = [&](const uint16_t* tile, const uint32_t (&pk)[2][8]) {
    u32x4 ring[8];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) ring[i] = read_cols(tile, i);
#pragma unroll
    for (int i = 0; i < 4 * DB; ++i) {
      if (i + AHEAD < 4 * DB) ring[(i + AHEAD) & 7] = read_cols(tile, i + AHEAD);
      const int ks4 = i / DB, db = i % DB, mq = ks4 >> 1, r0 = (ks4 & 1) * 4;
      const u32x4 bb = {pk[mq][r0], pk[mq][r0 + 1], pk[mq][r0 + 2], pk[mq][r0 + 3]};
      acc[db] = Mma<T>::run(ring[i & 7], bb, acc[db]);
    }
  };

  const int bkind = HASB ? __builtin_amdgcn_readfirstlane(ma.bias_kind) : 0;
  const int besz = __builtin_amdgcn_readfirstlane(bkind == 1 ? 4 : bkind == 4 ? 1 : 2);  // (in a scalar register: a descriptor built from a vector register is looked up lane by lane)
  const uint32_t b_rowbytes = HASB ? (uint32_t)(p.bias_sl * besz) : 0u;
  const uint32_t b_lane = HASB ? (uint32_t)((half * 4 * p.bias_sl + key) * besz) : 0u;
  const int b_records = HASB ? __builtin_amdgcn_readfirstlane((int)(((int64_t)(p.L - 1) * p.bias_sl + p.S) * besz)) : 0;
  // the fetched bias elements of a tile, turned into floats in the log2 domain in place (the
  // element type is tested once, outside the loops: inside, every element would carry the branch)
  auto bias_to_log2 = [&](uint32_t (&w)[2][16]) {
    auto each = [&](auto conv) {
#pragma unroll
      for (int mq = 0; mq < 2; ++mq)
#pragma unroll
        for (int r = 0; r < 16; ++r) w[mq][r] = __builtin_bit_cast(uint32_t, conv(w[mq][r]));
    };
    if (bkind == 1) each([](uint32_t x) { return __builtin_bit_cast(float, x) * kLog2eF; });
    else if (bkind == 4) each([](uint32_t x) { return x ? 0.f : -INFINITY; });
    else if (bkind == 3) each([](uint32_t x) { return __builtin_bit_cast(float, x << 16) * kLog2eF; });
    else each([](uint32_t x) { return (float)__builtin_bit_cast(_Float16, (uint16_t)x) * kLog2eF; });
  };
  // MASK = 2: the bias of this lane's key in each of a tile's 64 rows, in the order of the score
  // accumulators, requested ahead of the tile's first product.  (Requesting it a tile ahead
  // keeps 32 more registers live across the loop, which spills at head dim 128 and is slower.)
  // The resource ends with
  // the last row of the (batch, head): rows past L read as zeros (they are switched off through
  // lse = +inf), keys past S as a neighbouring element (their probabilities are replaced by zero).
  uint32_t braw[2][16];
  uint32_t kraw[DROP ? 2 : 1][16];  // (dropout) the keep bytes of the same scores
  auto load_bias_a = [&](int it) {
    if constexpr (BIASED) {
      const int q0 = item_q0(it);
      if (it >= n_items || (ma.causal && q0 + BQ - 1 < kw0) || kw0 >= S) return;
      if constexpr (DROP) {
        const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            uniform_ptr((const char*)p.keep + ((int64_t)b * p.Hq + item_head(it)) * p.L * p.keep_ld), 0,
            __builtin_amdgcn_readfirstlane((int)((int64_t)(p.L - 1) * p.keep_ld + p.S)), 0x00020000);
        const uint32_t kbase = (uint32_t)((q0 + half * 4) * p.keep_ld + key);
#pragma unroll
        for (int mq = 0; mq < 2; ++mq)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            kraw[mq][r] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b8(k_rsrc, kbase + (uint32_t)((mq * 32 + (r >> 2) * 8 + (r & 3)) * p.keep_ld), 0, 0);
      }
      if constexpr (!HASB) return;
      const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
          uniform_ptr((const char*)p.bias + (b * p.bias_sb + item_head(it) * p.bias_sh) * besz), 0, b_records, 0x00020000);
      const uint32_t base = b_lane + (uint32_t)q0 * b_rowbytes;
      auto each = [&](auto fetch) {
#pragma unroll
        for (int mq = 0; mq < 2; ++mq)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            braw[mq][r] = fetch(base + (uint32_t)(mq * 32 + (r >> 2) * 8 + (r & 3)) * b_rowbytes);
      };
      if (bkind == 1) each([&](uint32_t off) { return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(b_rsrc, off, 0, 0); });
      else if (bkind == 4) each([&](uint32_t off) { return (uint32_t)__builtin_amdgcn_raw_buffer_load_b8(b_rsrc, off, 0, 0); });
      else each([&](uint32_t off) { return (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(b_rsrc, off, 0, 0); });
    }
  };
  // One tile of role A, software pipelined by hand (a wavefront issues in order, and left alone
  // the compiler emits a tile's matrix ops in two solid runs with all of the vector work between
  // them, which leaves the overlap to the other wavefront of the SIMD alone):
  //   phase 1  scores of rows 0-31
  //   phase 2  scores of rows 32-63        | probabilities of rows 0-31
  //   phase 3  dV from rows 0-31           | probabilities of rows 32-63
  //   phase 4  dV from rows 32-63
  // Every matrix op is one slot: the LDS operand of the op AHEAD slots later is requested, the op
  // is issued, and 16 / KS probabilities are formed.  A tile that crosses the causal diagonal or
  // the end of the keys (edge) has the scores of its masked positions set to -inf between the
  // phases, in blocks of their own: tested per element inside the unrolled loops, the compiler
  // turns the test into selects that every element of every tile pays for.
  auto role_a_tile = [&](int it, int tb, int pb, bool edge) {
    constexpr int EPS = 16 / KS;  // probabilities per slot (2 or 4)
    constexpr int SPG = 4 / EPS;  // slots per group of four consecutive rows
    load_bias_a(it);
    float bl = 0.f;  // this key's bias in the log2 domain
    // score functors of this item (MASK = 4): the head's slope, this key's weight and bias
    const float sm_inv_scale = SMOD ? 1.f / p.scale : 0.f;
    const float cap_s = SMOD ? p.sm.softcap * sm_inv_scale : 0.f, icap_s = (SMOD && p.sm.softcap > 0.f) ? p.scale / p.sm.softcap : 0.f;
    float sm_slope = 0.f, sm_w = 1.f, sm_kb = 0.f;
    if constexpr (SMOD) {
      const int hh = item_head(it);
      if (p.sm.alibi) sm_slope = p.sm.alibi[hh] * sm_inv_scale;
      if (p.sm.key_weight) sm_w = p.sm.key_weight[(int64_t)hh * p.S + min(key, p.S - 1)];
      if (p.sm.key_bias) sm_kb = p.sm.key_bias[(int64_t)hh * p.S + min(key, p.S - 1)] * sm_inv_scale;
    }
    // (the functors' derivative differs from one: the dK wavefronts get P times it, see hand_over)
    const bool need_dfac = SMOD && (p.sm.key_weight != nullptr || p.sm.softcap > 0.f);
    if constexpr (MASK == 1) {
      if (ma.bias_kind)
        bl = bias_value(p.bias, b * p.bias_sb + item_head(it) * p.bias_sh + min(key, p.S - 1), ma.bias_kind) * kLog2eF;
    }
    const uint16_t* qt = q_t + tb * TILE;
    const uint16_t* dot = do_t + tb * TILE;
    const float* lrow = &lse_s[tb * BQ + half * 4];
    uint32_t* px = pex + (pb * 4 + kb) * 1024 + lane * 4;  // [4 groups of 4 words][lane][4]
    f32x16 sc[2];
    uint32_t pk[2][8];
    uint32_t pkx[DROP ? 2 : 1][8];  // (dropout) what the dK wavefronts get: every probability, the dropped ones negative
    f32x4 l4[2][4];
    u32x4 ring[8];
    auto load_l4 = [&](int mq, int r4) { l4[mq][r4] = *(const f32x4*)(lrow + mq * 32 + r4 * 8); };
    auto prob = [&](int mq, int r) {
      const float l = l4[mq][r >> 2][r & 3];
      float x;
      if constexpr (HASB) x = __builtin_amdgcn_exp2f(fmaf(sc[mq][r], c, __builtin_bit_cast(float, braw[mq][r])) - l);
      else if constexpr (MASK == 1) x = __builtin_amdgcn_exp2f(fmaf(sc[mq][r], c, bl) - l);
      else x = __builtin_amdgcn_exp2f(fmaf(sc[mq][r], c, -l));
      return x;
    };
    auto slot_probs = [&](int mq, int slot) {  // and the row statistics of the group after the next slot's
      if ((slot + 1) % SPG == 0 && (slot + 1) / SPG < 4) load_l4(mq, (slot + 1) / SPG);
#pragma unroll
      for (int k = 0; k < EPS; k += 2) {
        const int r = slot * EPS + k;
        const float p0 = prob(mq, r), p1 = prob(mq, r + 1);
        if constexpr (DROP) {
          const float s0 = kraw[mq][r] ? p0 : -p0, s1 = kraw[mq][r + 1] ? p1 : -p1;
          pkx[mq][r >> 1] = Mma<T>::pack(s0, s1);
          pk[mq][r >> 1] = Mma<T>::pack(fmaxf(s0, 0.f), fmaxf(s1, 0.f));
        } else {
          pk[mq][r >> 1] = Mma<T>::pack(p0, p1);
        }
      }
    };
    // score functors: the raw score tile s becomes mod(scale * s) / scale (lane = key, element r =
    // row 32 mq + 8 (r / 4) + 4 half + r % 4 of the tile), one block per functor behind a uniform test
    const int sm_on = SMOD ? __builtin_amdgcn_readfirstlane((p.sm.key_weight ? 1 : 0) | (p.sm.key_bias ? 2 : 0) | (p.sm.alibi ? 4 : 0) | (p.sm.softcap > 0.f ? 8 : 0)) : 0;
    auto smod_scores = [&](int mq) {
      if constexpr (SMOD) {
        if (sm_on == 0) return;  // (document ids alone: nothing to rewrite)
        if (p.sm.key_weight) {
#pragma unroll
          for (int r = 0; r < 16; ++r) sc[mq][r] *= sm_w;
        }
        if (p.sm.key_bias) {
#pragma unroll
          for (int r = 0; r < 16; ++r) sc[mq][r] += sm_kb;
        }
        if (p.sm.alibi) {
          const float base = (float)(key - item_q0(it) - mq * 32 - half * 4);
#pragma unroll
          for (int r = 0; r < 16; ++r) sc[mq][r] = fmaf(sm_slope, base - (float)((r >> 2) * 8 + (r & 3)), sc[mq][r]);
        }
        if (p.sm.softcap > 0.f) {
#pragma unroll
          for (int r = 0; r < 16; ++r) sc[mq][r] = cap_s * tanh_fast(sc[mq][r] * icap_s);
        }
      }
    };
    auto mask_scores = [&](int mq) {
      const int q0 = item_q0(it);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int qi = q0 + mq * 32 + (r >> 2) * 8 + half * 4 + (r & 3);
        // (one compare or two against per-lane bounds: spelled out as the conditions they stand for,
        // the test is compiled into a cascade of branches per element)
        bool dead = FUNC ? (qi < first_q) | (qi >= past_q) : qi < first_q;
        if constexpr (SMOD) {
          if (sm_doc) dead |= doc_s[tb * BQ + mq * 32 + (r >> 2) * 8 + half * 4 + (r & 3)] != sm_dk;
        }
        sc[mq][r] = dead ? -INFINITY : sc[mq][r];
      }
    };
    auto hand_over = [&](int mq) {
      if (SMOD && need_dfac) {
        // Score functors whose derivative differs from one: the dK wavefronts get P times that
        // derivative, formed here from the packed probabilities and the modified scores
        // (1 - tanh^2 = 1 - (s' / cap)^2, a masked score's -inf clamped to a derivative of 0, times
        // the key's weight) - outside the slots, which carry neither a branch nor a register for it.
        uint32_t w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float t0 = __builtin_amdgcn_fmed3f(sc[mq][2 * j] * icap_s, -1.f, 1.f), t1 = __builtin_amdgcn_fmed3f(sc[mq][2 * j + 1] * icap_s, -1.f, 1.f);
          w[j] = Mma<T>::pack(Mma<T>::unpack(pk[mq][j], 0) * (fmaf(-t0, t0, 1.f) * sm_w), Mma<T>::unpack(pk[mq][j], 1) * (fmaf(-t1, t1, 1.f) * sm_w));
        }
        *(u32x4*)(px + (2 * mq) * 256) = u32x4{w[0], w[1], w[2], w[3]};
        *(u32x4*)(px + (2 * mq + 1) * 256) = u32x4{w[4], w[5], w[6], w[7]};
      } else {
        const uint32_t(&w)[8] = DROP ? pkx[DROP ? mq : 0] : pk[mq];
        *(u32x4*)(px + (2 * mq) * 256) = u32x4{w[0], w[1], w[2], w[3]};
        *(u32x4*)(px + (2 * mq + 1) * 256) = u32x4{w[4], w[5], w[6], w[7]};
      }
    };
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) ring[i] = read_rows(qt, i);
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase 1
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      ring[(i + AHEAD) & 7] = read_rows(qt, i + AHEAD);
      sc[0] = Mma<T>::run(ring[i & 7], frag[i], i == 0 ? zero16 : sc[0]);
      if (i == KS - 1) load_l4(0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (HASB) bias_to_log2(braw);
    smod_scores(0);
    if (__builtin_expect(edge, 0)) mask_scores(0);
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase 2
#pragma unroll
    for (int i = KS; i < 2 * KS; ++i) {
      const int n = i + AHEAD;  // the operand after next: rows of Q, then columns of dO
      ring[n & 7] = n < 2 * KS ? read_rows(qt, n) : read_cols(dot, n - 2 * KS);
      sc[1] = Mma<T>::run(ring[i & 7], frag[i - KS], i == KS ? zero16 : sc[1]);
      slot_probs(0, i - KS);
      if (i == 2 * KS - 1) load_l4(1, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    hand_over(0);
    smod_scores(1);
    if (__builtin_expect(edge, 0)) mask_scores(1);
    __builtin_amdgcn_sched_barrier(0);
    // ---- phases 3 and 4: operand j = DB * (16-row step) + d block of dO^T
#pragma unroll
    for (int j = 0; j < 4 * DB; ++j) {
      if (j + AHEAD < 4 * DB) ring[(j + AHEAD) & 7] = read_cols(dot, j + AHEAD);
      const int ks4 = j / DB, db = j % DB, mq = ks4 >> 1, r0 = (ks4 & 1) * 4;
      const u32x4 bb = {pk[mq][r0], pk[mq][r0 + 1], pk[mq][r0 + 2], pk[mq][r0 + 3]};
      acc[db] = Mma<T>::run(ring[j & 7], bb, acc[db]);
      if (j < 2 * DB) slot_probs(1, j);
      if (j == 2 * DB - 1) hand_over(1);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // every key of this block lies above the diagonal of the tile's rows / past the keys / below their
  // windows, or the mask's skip table says that it keeps no score of the tile's rows and the block's keys
  auto dead_tile = [&](int it, int tb) {
    const int q0 = item_q0(it);
    if constexpr (SMOD) {
      // (sorted ids: the tile's rows lie outside the run of rows with this wavefront's keys' ids)
      if (sm_doc && p.sm.doc_sorted && (min(q0 + BQ, p.L) <= doc_run_w[0] || q0 >= doc_run_w[1])) return true;
    }
    if constexpr (MASK == 2) {
      if (listed) {
        const int qt = q0 / BQ;
        const int hg = h0 + item_id(it) % rep;
        if (!compact && !((__builtin_amdgcn_readfirstlane((int)live_s[hg * p.live_t_words + (qt >> 5)]) >> (qt & 31)) & 1)) return true;
      }
    }
    return (ma.causal && q0 + BQ - 1 < kw0) || kw0 >= S || (W > 0 && q0 - kw0 - 31 >= W && kw0 >= n_sink);
  };
  auto role_a = [&](int it, int tb, int pb) {
    const int q0 = item_q0(it);
    if (dead_tile(it, tb)) return;
    bool edge = (ma.causal && q0 < kw0 + 31) || (kw0 + 31 >= S) || (W > 0 && q0 + BQ - 1 - kw0 >= W && kw0 + 31 >= n_sink);
    if constexpr (SMOD) {
      // every score compared, unless (sorted ids) the wavefront's keys carry one id and the tile's rows lie
      // inside the run of rows with that id
      if (sm_doc) edge |= !(p.sm.doc_sorted && sm_dk_first == sm_dk_last && q0 >= doc_run_w[0] && min(q0 + BQ, p.L) <= doc_run_w[1]);
    }
    role_a_tile(it, tb, pb, edge);
  };
  // Role B splits a tile over two iterations, so that its vector work falls on role A's first
  // matrix ops and its matrix ops on role A's vector work: dP of tile it at the end of iteration
  // it, dS and dK of that tile at the start of iteration it + 1.
  f32x16 dp[2];
  auto role_b_scores = [&](int it, int tb) {
    if (dead_tile(it, tb)) return;
    scores(do_t + tb * TILE, dp);
  };
  // One tile of role B, pipelined like role A's:
  //   phase 0  dS of rows 0-31
  //   phase 1  dK from rows 0-31           | dS of rows 32-63
  //   phase 2  dK from rows 32-63
  auto role_b = [&](int it, int tb, int pb) {
    constexpr int EPS = 16 / KS;  // elements per slot (2 or 4)
    constexpr int SPG = 4 / EPS;  // slots per group of four consecutive rows
    if (dead_tile(it, tb)) return;
    const uint32_t* px = pex + (pb * 4 + kb) * 1024 + lane * 4;
    const uint16_t* qt = q_t + tb * TILE;
    const float* drow = &dl_s[tb * BQ + half * 4];
    uint32_t pk[2][8];
    u32x4 w[2][2];  // P of this lane's key in the tile's 64 rows, packed as role A fed it to the matrix pipe
    f32x4 d4[2][4];
    u32x4 ring[8];
    auto load_d4 = [&](int mq, int r4) { d4[mq][r4] = *(const f32x4*)(drow + mq * 32 + r4 * 8); };
    auto ds_pair = [&](int mq, int r) {  // elements r, r + 1
      const uint32_t word = w[mq][r >> 3][(r >> 1) & 3];
      float s0, s1;
      if constexpr (DROP) {  // a negative probability was dropped: its dP counts as zero
        const float p0 = Mma<T>::unpack(word, 0), p1 = Mma<T>::unpack(word, 1);
        const float t0 = p0 < 0.f ? 0.f : dp[mq][r] * p.keep_scale, t1 = p1 < 0.f ? 0.f : dp[mq][r + 1] * p.keep_scale;
        s0 = fabsf(p0) * (t0 - d4[mq][r >> 2][r & 3]);
        s1 = fabsf(p1) * (t1 - d4[mq][(r + 1) >> 2][(r + 1) & 3]);
      } else {
        s0 = Mma<T>::unpack(word, 0) * (dp[mq][r] - d4[mq][r >> 2][r & 3]);
        s1 = Mma<T>::unpack(word, 1) * (dp[mq][r + 1] - d4[mq][(r + 1) >> 2][(r + 1) & 3]);
      }
      pk[mq][r >> 1] = Mma<T>::pack(s0, s1);
    };
    w[0][0] = *(const u32x4*)(px), w[0][1] = *(const u32x4*)(px + 256);
    load_d4(0, 0);
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) ring[i] = read_cols(qt, i);
    __builtin_amdgcn_sched_barrier(0);
    // ---- phase 0
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      if (r4 + 1 < 4) load_d4(0, r4 + 1);
      ds_pair(0, r4 * 4), ds_pair(0, r4 * 4 + 2);
    }
    w[1][0] = *(const u32x4*)(px + 512), w[1][1] = *(const u32x4*)(px + 768);
    load_d4(1, 0);
    __builtin_amdgcn_sched_barrier(0);
    // ---- phases 1 and 2: operand j = DB * (16-row step) + d block of Q^T
#pragma unroll
    for (int j = 0; j < 4 * DB; ++j) {
      if (j + AHEAD < 4 * DB) ring[(j + AHEAD) & 7] = read_cols(qt, j + AHEAD);
      const int ks4 = j / DB, db = j % DB, mq = ks4 >> 1, r0 = (ks4 & 1) * 4;
      const u32x4 bb = {pk[mq][r0], pk[mq][r0 + 1], pk[mq][r0 + 2], pk[mq][r0 + 3]};
      acc[db] = Mma<T>::run(ring[j & 7], bb, acc[db]);
      if (j < 2 * DB) {
        if ((j + 1) % SPG == 0 && (j + 1) / SPG < 4) load_d4(1, (j + 1) / SPG);
#pragma unroll
        for (int k = 0; k < EPS; k += 2) ds_pair(1, j * EPS + k);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  if constexpr (MASK == 2) {
    if (listed) {  // this key block's row of the skip table, for every head of the group
      if (tid < rep_all * p.live_t_words) {
        const int hd = hk * rep_all + tid / p.live_t_words;
        live_s[tid] = p.live_t[(((int64_t)(p.bias_sb ? b : 0) * p.live_hm + (p.bias_sh ? hd : 0)) * ((p.S + BK - 1) / BK) + kt) * p.live_t_words +
                               tid % p.live_t_words];
      }
      __syncthreads();
      if (n_items > 0 && n_items <= 1024) {
        if (wave == 0) {
          int cnt = 0;
          for (int j0 = 0; j0 < n_items; j0 += 64) {
            const int it = j0 + lane, qt = qs_end - 1 - it / rep;
            const bool live = it < n_items && ((live_s[(h0 + it % rep) * p.live_t_words + (qt >> 5)] >> (qt & 31)) & 1u);
            const uint64_t m = __builtin_amdgcn_ballot_w64(live);
            if (live) items_s[cnt + __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u))] = (uint16_t)it;
            cnt += __builtin_popcountll(m);
          }
          if (lane == 0) *(int*)(items_s + 1024) = cnt;
        }
        __syncthreads();
        n_items = __builtin_amdgcn_readfirstlane(*(const int*)(items_s + 1024));
        compact = true;
      }
    }
  }
  if (p.parts > 1) {  // this workgroup's share of the (live) items
    const bool fixed = p.chunk_items > 0 && !listed;
    const int parts_q = p.parts / p.parts_h;
    const int chunk = fixed ? p.chunk_items : (n_items + parts_q - 1) / parts_q;
    it0 = pq * chunk;
    n_items = max(min(n_items - it0, chunk), 0);
    // (a share past the key block's items: bwd_dkdv_merge_kernel, which counts them in the same way,
    // does not read it)
    if (fixed && n_items == 0 && pq > 0) return;
  }
  if (n_items > 0) {
    load_item(0, 0);
    wait_tiles();
    finish_item(0, 0);
    __syncthreads();
    if (n_items > 1) load_item(1, 1);
  }
  // iteration `it`: role A works on tile it, role B on tile it - 1; tile it + 1 goes to LDS
  // (one loop per role, with the same barriers: in a shared loop the registers that one role
  // carries across iterations would count as live in the other role's code)
  int tb_a = 0, tb_b = 2;  // tile buffers of tiles it and it - 1: it % 3 and (it - 1) % 3
  auto stage_and_sync = [&](int it) {
    const int tb_n = tb_a == 2 ? 0 : tb_a + 1;
    wait_tiles();
    if (it + 1 < n_items) finish_item(it + 1, tb_n);
    __syncthreads();
    // (the buffer of tile it - 1: its last reader, role B, passed the barrier above)
    if (it + 2 < n_items) load_item(it + 2, tb_b);
    tb_b = tb_a, tb_a = tb_n;
  };
  if (role == 0) {
    for (int it = 0; it <= n_items && n_items > 0; ++it) {
      if (it < n_items) role_a(it, tb_a, it & 1);
      stage_and_sync(it);
    }
  } else {
    for (int it = 0; it <= n_items && n_items > 0; ++it) {
      if (it >= 1) role_b(it - 1, tb_b, (it - 1) & 1);
      if (it < n_items) role_b_scores(it, tb_a);
      stage_and_sync(it);
    }
  }

  const float sc = role ? p.scale : DROP ? p.keep_scale : 1.f;
  if (p.parts > 1) {  // float32 rows for bwd_dkdv_merge_kernel, which also applies the factor
    if (key < p.S) {
      float* g = (role ? p.part_dk : p.part_dv) + ((((int64_t)part * p.B + b) * p.Hkv + hk) * p.S + key) * dr + half * 4;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int gq = 0; gq < 4; ++gq)
          if (!MASK || db * 32 + gq * 8 + half * 4 < dr) *(f32x4*)(g + db * 32 + gq * 8) = f32x4{acc[db][gq * 4], acc[db][gq * 4 + 1], acc[db][gq * 4 + 2], acc[db][gq * 4 + 3]};
    }
  } else if (key < p.S) {
    uint16_t* g = role ? (uint16_t*)p.gk + b * p.gk_sb + hk * p.gk_sh + (int64_t)key * p.gk_sl
                       : (uint16_t*)p.gv + b * p.gv_sb + hk * p.gv_sh + (int64_t)key * p.gv_sl;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        u32x2 w;
        w[0] = Mma<T>::pack(acc[db][gq * 4] * sc, acc[db][gq * 4 + 1] * sc);
        w[1] = Mma<T>::pack(acc[db][gq * 4 + 2] * sc, acc[db][gq * 4 + 3] * sc);
        if (!MASK || db * 32 + gq * 8 + half * 4 < dr) *(u32x2*)(g + db * 32 + gq * 8 + half * 4) = w;
      }
  }
}

// The kernel of a variant.  A call whose bias comes with a verdict about it (see MaskArgs) is launched
// twice: as the variant with a bias (MASK = 2), and as the variant with key counts marked PATTERN; the
// verdict lets one of them run.
template <typename T, int D, int MASK, bool PATTERN = false>
__global__ __launch_bounds__(512, 1) void bwd_dkdv_w32_kernel(BwdM p) {
  static_assert(!PATTERN || MASK == 1 || MASK == 3, "the pattern kernels are the variants with key counts, without and with dropout");
  MaskArgs ma = mask_args_of(p);
  if constexpr (MASK == 2 || MASK == 5 || PATTERN) {
    if (verdict_pattern(p, ma) != PATTERN) return;
  } else if constexpr (MASK == 1) {
    verdict_pattern(p, ma);  // (a bias per key that comes with a verdict: this variant takes the bias or the key counts)
  }
  bwd_dkdv_w32_body<T, D, MASK>(p, ma);
}

// Sum of the parts' float32 rows, one 64-thread block per key row of a (batch, kv head): four columns
// per thread, dK's d_real columns first, dV's dv_real behind them.  The factors that the kernels apply
// when they write dK and dV themselves are applied here: the scale for dK, 1 / (1 - p) of dropout for dV.
template <typename T>
__global__ __launch_bounds__(64) void bwd_dkdv_merge_kernel(BwdM p) {
  MaskArgs ma = mask_args_of(p);
  verdict_pattern(p, ma);  // (the item counts below are those of the kernel that filled the parts)
  const int64_t row = blockIdx.x;  // (b * Hkv + hk) * S + key
  const int key = (int)(row % p.S);
  const int hk = (int)((row / p.S) % p.Hkv), b = (int)(row / ((int64_t)p.S * p.Hkv));
  const int er = p.d_real, dvr = p.dv_real;
  const int64_t rows = (int64_t)p.B * p.Hkv * p.S;
  int parts = p.parts;
  if (p.chunk_items > 0 && p.live_t == nullptr) {
    // the parts that bwd_dkdv_w32_kernel filled for this row's key block: its items, counted as there
    const int k0 = key / BK * BK, nqs = (p.L + BQ - 1) / BQ;
    int S = p.S;
    if (ma.kv_lens) S = min(S, max(ma.kv_lens[b], 0));
    const int qs_begin = ma.causal ? min(k0 / BQ, nqs) : 0;
    const int qs_end = (ma.window > 0 && k0 >= ma.sink_keys) ? max(min(nqs, (k0 + BK + ma.window - 2) / BQ + 1), qs_begin) : nqs;
    const int n_items = k0 >= S ? 0 : (p.Hq / p.Hkv / p.parts_h) * (qs_end - qs_begin);
    parts = min(max((n_items + p.chunk_items - 1) / p.chunk_items, 1), p.parts / p.parts_h) * p.parts_h;
  }
  for (int c = threadIdx.x * 4; c < er + dvr; c += 64 * 4) {
    const bool is_v = c >= er;
    const int col = is_v ? c - er : c, width = is_v ? dvr : er;
    const float* src = (is_v ? p.part_dv : p.part_dk) + row * width + col;
    f32x4 a = {0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < parts; ++i) a += *(const f32x4*)(src + i * rows * width);
    a *= is_v ? (p.keep_scale != 0.f ? p.keep_scale : 1.f) : p.scale;
    uint16_t* g = is_v ? (uint16_t*)p.gv + b * p.gv_sb + hk * p.gv_sh + (int64_t)key * p.gv_sl
                       : (uint16_t*)p.gk + b * p.gk_sb + hk * p.gk_sh + (int64_t)key * p.gk_sl;
    u32x2 w;
    w[0] = Mma<T>::pack(a[0], a[1]);
    w[1] = Mma<T>::pack(a[2], a[3]);
    *(u32x2*)(g + col) = w;
  }
}

// Launch order of the key blocks for a call with sorted document ids.  Workgroups are dispatched in
// order, one per compute unit at a time, so the heaviest should go first; without documents that is
// the order of the key blocks under a causal mask, with them the weight of a block is the number of
// query tiles between itself and the end of its documents, which only the ids tell.  One workgroup
// per batch counts every key block's query tiles the way bwd_dkdv_w32_kernel does and ranks them.
__global__ __launch_bounds__(256) void bwd_key_order_kernel(BwdM p) {
  __shared__ int weight[1024];
  const int b = blockIdx.x, n_kt = p.n_kt;
  const int32_t* dqr = p.sm.doc_q + (int64_t)b * p.L;
  const int32_t* dkr = p.sm.doc_k + (int64_t)b * p.S;
  int S = p.S;
  if (p.kv_lens) S = min(S, max(p.kv_lens[b], 0));
  const int nqs = (p.L + BQ - 1) / BQ;
  auto lower_bound = [&](int x) {  // first row whose id is >= x
    int lo = 0, hi = p.L;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (dqr[mid] < x) lo = mid + 1;
      else hi = mid;
    }
    return lo;
  };
  for (int kt = threadIdx.x; kt < n_kt; kt += 256) {
    const int k0 = kt * BK;
    int items = 0;
    if (k0 < S) {
      const int d_lo = dkr[k0], d_hi = dkr[min(k0 + BK, S) - 1];
      const int r_lo = lower_bound(d_lo), r_hi = d_hi == INT_MAX ? p.L : lower_bound(d_hi + 1);
      int qs_begin = p.causal ? min(k0 / BQ, nqs) : 0;
      int qs_end = (p.window > 0 && k0 >= p.sink_keys) ? max(min(nqs, (k0 + BK + p.window - 2) / BQ + 1), qs_begin) : nqs;
      qs_begin = max(qs_begin, r_lo / BQ);
      qs_end = r_hi > r_lo ? max(min(qs_end, (r_hi + BQ - 1) / BQ), qs_begin) : qs_begin;
      items = qs_end - qs_begin;
    }
    weight[kt] = items;
  }
  __syncthreads();
  for (int kt = threadIdx.x; kt < n_kt; kt += 256) {  // rank = blocks that are heavier, or as heavy and earlier
    const int w = weight[kt];
    int rank = 0;
    for (int j = 0; j < n_kt; ++j) rank += (weight[j] > w) | ((weight[j] == w) & (j < kt));
    p.kt_order[b * n_kt + rank] = kt;
  }
}

template <typename T, int D, int MASK, bool PATTERN = false>
int launch_t(const BwdM& g, hipStream_t s) {
  // (MASK = 2: with the skip table's row of the key block and the item list; MASK = 4: with the document ids of three tiles' rows)
  constexpr int kSmemBytes = smem_bytes<D>() + (MASK == 2 ? 1024 + 2048 + 16 : MASK == 4 ? 3 * BQ * 4 : 0);
  static LdsOnce once;
  const hipError_t attr = reserve_lds(once, (const void*)bwd_dkdv_w32_kernel<T, D, MASK, PATTERN>, kSmemBytes);
  if (attr != hipSuccess) {
    set_error("SDPA: cannot reserve %d bytes of LDS for bwd_dkdv_w32_kernel: %s", kSmemBytes, hipGetErrorString(attr));
    return MI355_SDPA_ERR_LAUNCH;
  }
  hipLaunchKernelGGL((bwd_dkdv_w32_kernel<T, D, MASK, PATTERN>), dim3((unsigned)(g.B * g.Hkv * g.n_kt * g.parts)), dim3(512), kSmemBytes, s, g);
  const int rc = check_launch("bwd_dkdv_w32_kernel");
  if (rc != MI355_SDPA_OK || g.parts == 1 || PATTERN) return rc;  // (the parts are added up once, behind the other kernel of the pair)
  return launch_bwd_dkdv_merge(g, std::is_same<T, bf16_t>::value ? MI355_SDPA_BF16 : MI355_SDPA_F16, s);
}
template <typename T, int D>
int launch_m(const BwdM& g, hipStream_t s) {
  if (g.sm.any) {
    if (g.keep_scale != 0.f || g.bias_kind) {
      set_error("SDPA: score functors in bwd_dkdv_w32_kernel need a call without bias and dropout");
      return MI355_SDPA_ERR_UNSUPPORTED;
    }
    if (g.kt_order) {
      hipLaunchKernelGGL(bwd_key_order_kernel, dim3((unsigned)g.B), dim3(256), 0, s, g);
      const int rc = check_launch("bwd_key_order_kernel");
      if (rc != MI355_SDPA_OK) return rc;
    }
    return launch_t<T, D, 4>(g, s);
  }
  if (g.keep_scale != 0.f) {
    if (!g.keep || g.live_t) {
      set_error("SDPA: dropout in bwd_dkdv_w32_kernel needs a keep-mask and no tile table");
      return MI355_SDPA_ERR_UNSUPPORTED;
    }
    if (!g.bias_kind) return launch_t<T, D, 3>(g, s);
    if (g.verdict) {  // (see bwd_dkdv_w32_kernel: the pair with dropout)
      if (int rc = launch_t<T, D, 3, true>(g, s)) return rc;
    }
    return launch_t<T, D, 5>(g, s);
  }
  if (g.bias_kind && g.bias_sl != 0) {
    if (g.verdict) {  // (see bwd_dkdv_w32_kernel)
      if (int rc = launch_t<T, D, 1, true>(g, s)) return rc;
    }
    return launch_t<T, D, 2>(g, s);
  }
  return (g.bias_kind || g.kv_lens || g.d_real != D || g.window > 0) ? launch_t<T, D, 1>(g, s) : launch_t<T, D, 0>(g, s);
}

}  // namespace

bool bwd_dkdv_w32_fits(const BwdM& g, int head_dim) {
  // 32-bit byte offsets from the start of a batch for Q and dO
  const int64_t q_ext = ((int64_t)(g.Hq - 1) * g.q_sh + (int64_t)(g.L + BQ) * g.q_sl + head_dim) * 2;
  const int64_t go_ext = ((int64_t)(g.Hq - 1) * g.go_sh + (int64_t)(g.L + BQ) * g.go_sl + head_dim) * 2;
  return q_ext < (1ll << 31) && go_ext < (1ll << 31) && g.q_sh >= 0 && g.q_sl >= 0 && g.go_sh >= 0 && g.go_sl >= 0;
}

// Fewer key blocks than would give every compute unit a workgroup or two: a key block's items (an
// item is a 64-row query tile of one head, about a microsecond) are dealt to about 768 workgroups in
// all.  The heads of the group are divided first (every share walks all query tiles, in the order the
// other key blocks' workgroups walk them, so that they keep finding the tiles in their XCD's L2),
// then the query tiles, in shares of chunk_items items: at least 8 items each, and only from 24 items
// on: below that the second kernel costs what the split saves.
void bwd_dkdv_w32_plan(const BwdM& g, int& parts_h, int& parts) {
  parts_h = parts = 1;
  const int64_t wgs = (int64_t)g.B * g.Hkv * g.n_kt;
  if (wgs >= 384 || wgs <= 0) return;
  const int rep = g.Hq / g.Hkv, nqs = (g.L + BQ - 1) / BQ;
  if ((int64_t)rep * nqs < 24) return;
  const int64_t want = (768 + wgs - 1) / wgs;
  for (int d = 1; d <= rep && d <= want; ++d)
    if (rep % d == 0 && (int64_t)(rep / d) * nqs >= 8) parts_h = d;
  const int64_t items = (int64_t)(rep / parts_h) * nqs;  // of a workgroup that every query of its heads sees
  const int64_t parts_q = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>((want + parts_h - 1) / parts_h, items / 8), 32));
  parts = (int)(parts_h * parts_q);
}
int bwd_dkdv_w32_parts(const BwdM& g) {
  int parts_h, parts;
  bwd_dkdv_w32_plan(g, parts_h, parts);
  return parts;
}

int launch_bwd_dkdv_merge(const BwdM& g, int dtype, hipStream_t s) {
  const dim3 rows((unsigned)((int64_t)g.B * g.Hkv * g.S));
  if (dtype == MI355_SDPA_BF16) hipLaunchKernelGGL((bwd_dkdv_merge_kernel<bf16_t>), rows, dim3(64), 0, s, g);
  else hipLaunchKernelGGL((bwd_dkdv_merge_kernel<f16_t>), rows, dim3(64), 0, s, g);
  return check_launch("bwd_dkdv_merge_kernel");
}

int launch_bwd_dkdv_w32(const BwdM& g0, int dtype, int head_dim, hipStream_t s) {
  BwdM g = g0;
  if (g.d_real <= 0 || g.d_real > head_dim) g.d_real = head_dim;
  g.dv_real = g.d_real;
  g.parts_h = 1, g.chunk_items = 0;
  if (!g.part_dk || !g.part_dv) g.parts = 1;
  if (g.parts > 1) {
    int parts;
    bwd_dkdv_w32_plan(g, g.parts_h, parts);
    if (parts != g.parts) {
      set_error("SDPA: bwd_dkdv_w32_kernel was given %d parts where its plan has %d", g.parts, parts);
      return MI355_SDPA_ERR_INVALID;
    }
    // the heaviest workgroup (every query tile of its heads) fills all the tile shares
    const int parts_q = g.parts / g.parts_h;
    g.chunk_items = ((g.Hq / g.Hkv / g.parts_h) * ((g.L + BQ - 1) / BQ) + parts_q - 1) / parts_q;
    // (sorted document ids bound a key block's query tiles in a way that bwd_dkdv_merge_kernel does not
    // count: every key block then deals its items to all the parts in equal shares)
    if (g.sm.doc_sorted) g.chunk_items = 0;
  }
  if (!g.sm.doc_sorted || g.n_kt > 1024) g.kt_order = nullptr;  // (the ranking kernel holds 1024 weights)
  if (head_dim == 128) return dtype == MI355_SDPA_BF16 ? launch_m<bf16_t, 128>(g, s) : launch_m<f16_t, 128>(g, s);
  return dtype == MI355_SDPA_BF16 ? launch_m<bf16_t, 64>(g, s) : launch_m<f16_t, 64>(g, s);
}

}  // namespace mi355
