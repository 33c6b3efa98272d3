// Flash-attention backward for head dims above 128 and for D_qk != D_v (D_v <= D_qk <= 256,
// multiples of 8; e.g. 192 / 128 of multi-head latent attention, or 256 / 256), bf16/f16, on the
// 32x32x16 MFMA.  Two kernels built for the widest case, rows narrower than 256 counting as zero
// padded; one wavefront per SIMD with the 512-register budget (the dK/dV kernel holds two 128-register
// accumulators and two 64-register fragments), LDS operands two or three matrix ops ahead through a
// register ring in a pinned order.
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
// Tiles sit in LDS row-major, unpadded and XOR swizzled; transposed operands come out of the
// transposing LDS read.  Math follows torch_neuronx/_sdpa_math.py:98-176: float32 accumulation, rows with
// lse = -inf give zero gradients, scale multiplies dQ and dK once at the end.
#include "bwd_mfma.h"

namespace mi355 {
namespace {

constexpr int DW = 256;           // the width the kernels are built for
constexpr int KS = DW / 16;       // contraction steps over the head dim
constexpr int DB = DW / 32;       // 32-row blocks of a transposed product
constexpr int BT = 32;            // rows of a staged tile

typedef short s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 tr_read(const uint16_t* ptr) {
  const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(ptr));
  return __builtin_bit_cast(u32x2, v);
}

// Both kernels stage their 32-row tiles from global memory straight into LDS (buffer loads with the
// LDS bit, 16 bytes per lane, 1 KB of contiguous LDS per wavefront and instruction), one tile ahead,
// into two buffers per operand.  The tiles are unpadded and XOR swizzled (tile_swz: the lane that owns
// LDS chunk position c of row r fetches the row's chunk c ^ tile_swz(r)), which keeps both the row
// reads and the transposing reads free of bank conflicts (with a padded pitch the transposing reads
// of four consecutive rows overlap in their banks).  16 loads cover a tile; a chunk past a narrow
// row's end asks for an offset beyond the buffer and gets zeros, and so do rows past the buffer's end.
constexpr int TILE_LOADS = BT * (DW / 8) / 64;
constexpr int TILE_ELEMS = BT * DW;
constexpr int WIDE_DKDV_LDS = 2 * 2 * TILE_ELEMS * 2 + 2 * 2 * BT * 4;
constexpr int WIDE_DQ_LDS = 2 * 2 * TILE_ELEMS * 2;
constexpr int WIDE_LIST_LDS = 2048 + 16;   // masked dQ instances: the list of live key tiles (1024 entries and the count)
constexpr int WIDE_LIVE_LDS = 1024;        // masked dK/dV instances: the key block's row of the transposed skip table

// The swizzle moves a chunk inside its 256-byte window of a 512-byte row: the offsets of the reads
// are not additive in the contraction step / d block within a window (one offset register per
// combination), and the second window is the first plus 256 bytes, which travels in the read's
// immediate offset.
constexpr int WIN = 128;  // elements per window

// element offsets of the transposing reads of a swizzled tile, [second read of a pair][d block of a window]
struct TrOffSwz {
  int off[2][4];
  __device__ __forceinline__ void init(int lane) {
    const int jj = lane & 15, g = lane >> 4;
#pragma unroll
    for (int sec = 0; sec < 2; ++sec)
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const int row = 8 * sec + (g >> 1) * 4 + (jj >> 2), d = db * 32 + 16 * (g & 1) + 4 * (jj & 3);
        off[sec][db] = row * DW + (((d >> 3) ^ tile_swz<DW>(row)) << 3) + (d & 7);
      }
  }
  // operand i = DB * (16-row step) + d block of the transposed tile (rows 16 apart share a swizzle)
  __device__ __forceinline__ u32x4 cols(const uint16_t* tile, int i) const {
    const int db = i % DB;
    const u32x2 lo = tr_read(tile + off[0][db % 4] + (db / 4) * WIN + (i / DB) * 16 * DW);
    const u32x2 hi = tr_read(tile + off[1][db % 4] + (db / 4) * WIN + (i / DB) * 16 * DW);
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
  }
};
// element offset of the row read of contraction step j (this lane: row col, 8 elements at 16 j + 8 half)
__device__ __forceinline__ int wide_row_off(int j, int col, int half, int swz_col) {
  return col * DW + (((2 * (j % 8) + half) ^ swz_col) << 3) + (j / 8) * WIN;
}

// raw buffer resource, in scalar registers
__device__ __forceinline__ u32x4 wide_descriptor(const void* base, int64_t bytes) {
  const uint64_t a = (uint64_t)base;
  return u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a),
               (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu)),
               (uint32_t)__builtin_amdgcn_readfirstlane((int)bytes), 0x00020000u};
}
// (m0 holds the LDS address of such a load, one wait state after it is written)
__device__ __forceinline__ void wide_tile_load(const u32x4& rsrc, uint32_t voffset, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :: "s"(__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(voffset), "s"(rsrc) : "memory", "m0");
}
// byte offset of this lane's chunk of load `ld` inside a tile whose first row is the buffer's base
__device__ __forceinline__ uint32_t wide_chunk_off(int ld, int lane, int row_stride, int width) {
  const int pos = ld * 64 + lane, r = pos / (DW / 8), ch = (pos % (DW / 8)) ^ tile_swz<DW>(r);
  return ch * 8 < width ? (uint32_t)((r * row_stride + ch * 8) * 2) : 0xfffffff0u;
}

// compile-time loop: f(std::integral_constant<int, 0>{}) ... f(std::integral_constant<int, N - 1>{})
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// The kernels are instantiated for the widths they serve, ER for Q / K and DVR for V / dO / O
// (multiples of 32 up to 256): contraction steps and output blocks that would lie wholly in the
// zero padding of the 256-wide layout do not exist in the instruction stream, nor do the registers
// of their fragments and accumulators (192 / 128: 40 matrix ops per item instead of 64 in the
// dK/dV kernel, 32 instead of 48 in the dQ kernel).  An item's LDS operands in the order of their use:
struct WideOp {
  int kind, j;  // dQ kernel: 0 K rows (S), 1 V rows (dP), 2 K^T columns (dQ); dK/dV kernel: 0 Q rows (S), 1 dO rows (dP),
                // 2 dO^T columns (dV), 3 Q^T columns (dK); j = contraction step, or DB * (16-row step) + d block
};
template <int ER, int DVR>
constexpr WideOp dq_op(int k) {  // the S steps, the dP steps, then the columns of K^T
  constexpr int KSE = ER / 16, KSV = DVR / 16, DBE = ER / 32;
  if (k < KSE) return {0, k};
  if (k < KSE + KSV) return {1, k - KSE};
  return {2, ((k - KSE - KSV) / DBE) * DB + (k - KSE - KSV) % DBE};
}
template <int ER, int DVR>
constexpr WideOp dkdv_op(int k) {  // S steps and dP steps (in turns where both accumulators fit: two
                                   // independent chains), the columns of dO^T, the columns of Q^T
  constexpr int KSE = ER / 16, KSV = DVR / 16, DBE = ER / 32, DBV = DVR / 32;
  if (k < KSE + KSV) {
    if constexpr (ER + DVR <= 320) {
      int c = 0;
      for (int j = 0; j < (KSE > KSV ? KSE : KSV); ++j) {
        if (j < KSE) {
          if (c == k) return {0, j};
          ++c;
        }
        if (j < KSV) {
          if (c == k) return {1, j};
          ++c;
        }
      }
    }
    return k < KSE ? WideOp{0, k} : WideOp{1, k - KSE};
  }
  k -= KSE + KSV;
  if (k < 2 * DBV) return {2, (k / DBV) * DB + k % DBV};
  k -= 2 * DBV;
  return {3, (k / DBE) * DB + k % DBE};
}

// MODE 1 (MASKED): per-batch key counts and an additive bias / bool keep-mask, per key or per score (a
// lane is a query row in the dQ kernel and reads its own row of it, a key in the dK/dV kernel and reads
// one element per score register); the gradient of the bias, P (dP - delta) in the input dtype, leaves
// the dQ kernel four keys at a time: the packed dS pairs it feeds to the matrix pipe are its elements.
// MODE 3 (DROP): MODE 1 without the skip tables, and a dropout keep-mask beside the bias (bytes,
// (B, Hq, L, S) contiguous, read the way a bool mask per score is): it leaves the scores alone, feeds dV
// with the kept probabilities and multiplies dP, together with 1 / (1 - p)
// (torch_neuronx/_sdpa_math.py:36-48, :154-158).
// MODE 2 (FUNC): per-batch key counts, a sliding window with sink keys (the tiles it drops whole are not
// walked) and the score functors and document ids of score_mod.h, each score through score_mod_at where
// its probability is formed; the derivative of the functors multiplies the gradient of the scores.
template <typename T, int ER, int DVR, int MODE>
__global__ __launch_bounds__(256, 1) void bwd_wide_dq_kernel(BwdM p) {
  constexpr bool MASKED = MODE == 1 || MODE == 3, FUNC = MODE == 2, DROP = MODE == 3;
  constexpr int KSE = ER / 16, KSV = DVR / 16, DBE = ER / 32;
  extern __shared__ __attribute__((aligned(16))) uint16_t wide_lds[];
  uint16_t* const k_buf = wide_lds;                    // [2][TILE_ELEMS]
  uint16_t* const v_buf = wide_lds + 2 * TILE_ELEMS;   // [2][TILE_ELEMS]
  uint16_t* const tile_list = wide_lds + 4 * TILE_ELEMS;  // (masked instances) [1024] and the count
  const int n_qt = (p.L + 127) / 128;
  const int qt = n_qt - 1 - blockIdx.x / (p.B * p.Hq);  // heavy query tiles first
  const int bh = blockIdx.x % (p.B * p.Hq), b = bh / p.Hq, h = bh % p.Hq, hk = h / (p.Hq / p.Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 31, half = lane >> 5;
  const int q0 = qt * 128, qw0 = q0 + wave * 32, qrow = qw0 + col, qc = min(qrow, p.L - 1);
  const int er = p.d_real, dvr = p.dv_real;

  u32x4 qf[KSE], dof[KSV];
  float lse2, dl;
  {
    const uint16_t* qr = (const uint16_t*)p.q + b * p.q_sb + h * p.q_sh + (int64_t)qc * p.q_sl + half * 8;
    const uint16_t* gr = (const uint16_t*)p.go + b * p.go_sb + h * p.go_sh + (int64_t)qc * p.go_sl + half * 8;
    const uint16_t* orow = (const uint16_t*)p.out + b * p.o_sb + h * p.o_sh + (int64_t)qc * p.o_sl + half * 8;
    float dsum = 0.f;
#pragma unroll
    for (int ks = 0; ks < KSE; ++ks) qf[ks] = half * 8 + ks * 16 < er ? *(const u32x4*)(qr + ks * 16) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int ks = 0; ks < KSV; ++ks) {
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
  TrOffSwz tr;
  tr.init(lane);
  const int swz_col = tile_swz<DW>(col);
  f32x16 dqacc[DBE];
#pragma unroll
  for (int i = 0; i < DBE; ++i) {
    zero(dqacc[i]);
    asm volatile("" : "+a"(dqacc[i]));
  }
  const float c = p.scale * kLog2eF;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const uint16_t* kp = (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh;
  const uint16_t* vp = (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh;
  int S = p.S;  // keys of this batch that take part
  if constexpr (MODE != 0) {
    if (p.kv_lens) S = min(S, max(p.kv_lens[b], 0));
  }
  int nt = (S + BT - 1) / BT;
  if (p.causal) nt = min(nt, (min(q0 + 128, p.L) - 1) / BT + 1);
  // sliding window: the tiles below the lowest window of the workgroup's rows are dropped whole, except
  // the leading ones that hold sink keys: stream position u is key tile u + (u >= n_lead ? skip : 0)
  int n_lead = 0, skip = 0;
  if constexpr (FUNC) {
    if (p.window > 0) {
      const int t_lo = max(q0 - p.window + 1, 0) / BT;
      n_lead = min(min((p.sink_keys + BT - 1) / BT, t_lo), nt);
      skip = min(t_lo, nt) - n_lead;
      nt -= skip;
    }
  }
  // With a skip table: the key tiles in which the mask keeps at least one score of this workgroup's
  // rows (the first wavefront ORs the bitmaps of its two 64-row blocks and expands the set bits into a
  // list in LDS); stream position u is then key tile tile_of(u).
  bool listed = false;
  if constexpr (MODE == 1) {
    if (p.live_tiles && !p.causal && !p.gbias) {  // (with a bias gradient every tile is walked: its zeros are written there)
      if (wave == 0) {
        const int nrb = (p.L + 63) / 64, rb0 = q0 / 64;
        const uint32_t* map = p.live_tiles + ((int64_t)((p.bias_sb ? b : 0) * p.live_hm + (p.bias_sh ? h : 0)) * nrb + rb0) * p.live_words;
        uint32_t w = 0u;
        if (lane < p.live_words) {
#pragma unroll
          for (int r = 0; r < 2; ++r)
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
    if constexpr (MODE == 1) return listed ? __builtin_amdgcn_readfirstlane((int)tile_list[u]) : u;
    else if constexpr (FUNC) return u + (u >= n_lead ? skip : 0);
    else return u;
  };
  const int nt_w = p.causal ? min(nt, (qw0 + 31) / BT + 1 - skip) : nt;  // tiles with work for this wavefront
  const int lim = p.causal ? min(qrow, S - 1) : S - 1;
  // (MASKED) this lane's row of the bias gradient, at its first key of a tile
  uint16_t* const gb_row = (MASKED && p.gbias && qrow < p.L)
                               ? (uint16_t*)p.gbias + b * p.gbias_sb + h * p.gbias_sh + (int64_t)qrow * p.gbias_sl + half * 4 : nullptr;
  // (FUNC) the window of this lane's row, and what the derivative of the functors needs
  const int lo_w = (FUNC && p.window > 0) ? qrow - p.window + 1 : (int)0x80000000;
  const int n_sink = FUNC ? p.sink_keys : 0;
  const float inv_scale = FUNC ? 1.f / p.scale : 0.f;
  const float icap = (FUNC && p.sm.softcap > 0.f) ? p.scale / p.sm.softcap : 0.f;
  const float* const f_kw = (FUNC && p.sm.key_weight) ? p.sm.key_weight + (int64_t)h * p.S : nullptr;
  const bool need_dfac = FUNC && (p.sm.softcap > 0.f || p.sm.key_weight != nullptr);

  // the buffers end with the last key row: rows of a ragged last tile beyond it read as zeros
  const u32x4 k_rsrc = wide_descriptor(kp, S > 0 ? ((int64_t)(S - 1) * p.k_sl + er) * 2 : 0);
  const u32x4 v_rsrc = wide_descriptor(vp, S > 0 ? ((int64_t)(S - 1) * p.v_sl + dvr) * 2 : 0);
  // bias of a score tile: this lane's 16 keys of its query row (row stride 0: a bias per key), as 4
  // groups of 4 consecutive keys, requested ahead of the tile's score products; keys past the row
  // read the next row or, past the last row, zeros (they are masked anyway)
  const int bkind = MASKED ? __builtin_amdgcn_readfirstlane(p.bias_kind) : 0;  // 0 none, 1 float32, 2 float16, 3 bfloat16, 4 bool
  const int besz = __builtin_amdgcn_readfirstlane(bkind == 1 ? 4 : bkind == 4 ? 1 : 2);  // (in a scalar register: a descriptor built from a vector register is looked up lane by lane)
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      uniform_ptr((const char*)p.bias + (bkind ? (b * p.bias_sb + h * p.bias_sh) * besz : 0)), 0,
      __builtin_amdgcn_readfirstlane(bkind ? (int)(((int64_t)(p.L - 1) * p.bias_sl + p.S) * besz) : 0), 0x00020000);
  const uint32_t b_row = MASKED ? (uint32_t)(((int64_t)qc * p.bias_sl + half * 4) * besz) : 0u;
  uint32_t braw[16];
  // (DROP) the keep bytes of the same 16 keys, four dwords
  const __amdgpu_buffer_rsrc_t kp_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      uniform_ptr((const char*)p.keep + (DROP ? ((int64_t)b * p.Hq + h) * p.L * p.keep_ld : 0)), 0,
      __builtin_amdgcn_readfirstlane(DROP ? (int)((int64_t)p.L * p.keep_ld) : 0), 0x00020000);  // (whole rows: dword loads)
  const uint32_t kp_row = DROP ? (uint32_t)((int64_t)qc * p.keep_ld + half * 4) : 0u;
  uint32_t kraw[DROP ? 4 : 1];
  auto load_bias = [&](int t) {
    if constexpr (DROP) {
#pragma unroll
      for (int g = 0; g < 4; ++g) kraw[g] = __builtin_amdgcn_raw_buffer_load_b32(kp_rsrc, kp_row + (uint32_t)(t * BT + g * 8), 0, 0);
    }
    if constexpr (MASKED) {
      const uint32_t off = b_row + (uint32_t)(t * BT * besz);
      if (bkind == 1) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const u32x4 w = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, off + g * 32, 0, 0);
          braw[4 * g] = w[0], braw[4 * g + 1] = w[1], braw[4 * g + 2] = w[2], braw[4 * g + 3] = w[3];
        }
      } else if (bkind == 4) {
#pragma unroll
        for (int g = 0; g < 4; ++g) braw[g] = __builtin_amdgcn_raw_buffer_load_b32(b_rsrc, off + g * 8, 0, 0);
      } else if (bkind) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(b_rsrc, off + g * 16, 0, 0);
          braw[2 * g] = w[0], braw[2 * g + 1] = w[1];
        }
      }
    }
  };
  // ... in the log2 domain (the element type is tested once, outside the loop: inside, every element
  // would carry the branch)
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
  typedef __attribute__((address_space(3))) unsigned char* lds_bytes;
  const uint32_t lds_k = (uint32_t)(uintptr_t)(lds_bytes)k_buf, lds_v = (uint32_t)(uintptr_t)(lds_bytes)v_buf;
  uint32_t k_off[TILE_LOADS / 4], v_off[TILE_LOADS / 4];
#pragma unroll
  for (int n = 0; n < TILE_LOADS / 4; ++n) {
    k_off[n] = wide_chunk_off(wave + 4 * n, lane, (int)p.k_sl, er);
    v_off[n] = wide_chunk_off(wave + 4 * n, lane, (int)p.v_sl, dvr);
  }
  auto request_tile = [&](int t) {  // the tile at stream position t into buffer t % 2
    const int ta = tile_of(t);
    const uint32_t kt = (uint32_t)(ta * BT * p.k_sl * 2), vt = (uint32_t)(ta * BT * p.v_sl * 2);
    const uint32_t boff = (uint32_t)((t & 1) * TILE_ELEMS * 2);
#pragma unroll
    for (int n = 0; n < TILE_LOADS / 4; ++n) {
      // (an offset that stands for "no such chunk" stays beyond the buffer whatever the tile)
      wide_tile_load(k_rsrc, k_off[n] >= 0xfffffff0u ? k_off[n] : k_off[n] + kt, lds_k + boff + (wave + 4 * n) * 1024);
      wide_tile_load(v_rsrc, v_off[n] >= 0xfffffff0u ? v_off[n] : v_off[n] + vt, lds_v + boff + (wave + 4 * n) * 1024);
    }
  };
  auto publish_tile = [&]() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  if (nt > 0) {
    request_tile(0);
    publish_tile();
  }
  for (int t = 0; t < nt; ++t) {
    // (the other buffer was last read before the barrier that ended the previous tile)
    if (t + 1 < nt) request_tile(t + 1);
    // (FUNC: GENERAL is the tile as the functors, a window's edge or the diagonal need it; a tile inside
    // the window of every row of a call without score functors is the plain tile, at the plain speed: tests
    // per score, even uniform ones, cost this kernel a third of its time)
    auto tile = [&](auto general_c) {
      constexpr bool GENERAL = decltype(general_c)::value;
      const uint16_t* k_t = k_buf + (t & 1) * TILE_ELEMS;
      const uint16_t* v_t = v_buf + (t & 1) * TILE_ELEMS;
      // The LDS operands of a tile - row fragments of K and V in turns, then the transposed fragments
      // of K - travel through a register ring, three matrix ops ahead of their use, in an order
      // pinned by scheduling fences (one wavefront per SIMD has nobody to hide an LDS round trip behind).
      constexpr int AHEAD = 3, NA = KSE + KSV, NOPS = NA + 2 * DBE;
      auto operand = [&](auto kc) {
        constexpr WideOp op = dq_op<ER, DVR>(decltype(kc)::value);
        if constexpr (op.kind == 2) return tr.cols(k_t, op.j);
        else return *(const u32x4*)((op.kind ? v_t : k_t) + wide_row_off(op.j, col, half, swz_col));
      };
      const int ta = tile_of(t);
      load_bias(ta);
      u32x4 ring[8];
      static_for<AHEAD>([&](auto kc) { ring[decltype(kc)::value] = operand(kc); });
      f32x16 sacc = zero16, dpacc = zero16;
      // (the dQ accumulators stay in the accumulation registers across the tile: left to itself the
      // register allocator keeps part of them in vector registers and copies 16 values in and out
      // around every matrix op that adds to them)
#pragma unroll
      for (int i = 0; i < DBE; ++i) asm volatile("" : "+a"(dqacc[i]));
      // One wavefront per SIMD has nobody to hide its vector work behind, so the tile is scheduled by
      // hand: the scores first; the probabilities are formed under the dP steps, spread over their
      // slots; dS of the first 16 keys is the only vector work nothing covers, dS of the other 16 keys
      // is formed under the dQ ops of the first 16.
      float bl[16], pr[16];
      uint32_t pS[8];
      if constexpr (FUNC && GENERAL) {
#pragma unroll
        for (int r = 0; r < 16; ++r) bl[r] = 1.f;
      }
      auto prob = [&](int r) {
        const int kv = ta * BT + (r >> 2) * 8 + half * 4 + (r & 3);
        float x;
        if constexpr (FUNC && GENERAL) {
          // (the scores went through the functors in a block of their own, see below; only dS is formed
          // from this probability, so the functors' derivative rides on it: 1 - tanh^2 of the soft cap,
          // recovered from the capped score, times the key's weight)
          const bool dead = (kv > lim) | ((kv < lo_w) & (kv >= n_sink));
          const float e = __builtin_amdgcn_exp2f(dead ? -INFINITY : fmaf(sacc[r], c, -lse2));
          const float th = sacc[r] * icap;
          pr[r] = e == 0.f ? 0.f : e * fmaf(-th, th, 1.f) * bl[r];  // (a dropped score may carry any derivative)
          return;
        }
        if constexpr (FUNC) {  // (a tile that no mask touches)
          pr[r] = __builtin_amdgcn_exp2f(fmaf(sacc[r], c, -lse2));
          return;
        }
        if constexpr (MASKED) x = fmaf(sacc[r], c, bl[r]) - lse2;
        else x = fmaf(sacc[r], c, -lse2);
        pr[r] = __builtin_amdgcn_exp2f(kv > lim ? -INFINITY : x);  // (masked before the exponential: no branch)
      };
      auto form_ds = [&](int r) {  // elements r, r + 1
        if constexpr (DROP) {
          const float k0 = (float)((kraw[r >> 2] >> (8 * (r & 3))) & 0xffu), k1 = (float)((kraw[r >> 2] >> (8 * (r & 3) + 8)) & 0xffu);
          pS[r >> 1] = Mma<T>::pack(pr[r] * fmaf(dpacc[r] * k0, p.keep_scale, -dl), pr[r + 1] * fmaf(dpacc[r + 1] * k1, p.keep_scale, -dl));
        } else {
          pS[r >> 1] = Mma<T>::pack(pr[r] * (dpacc[r] - dl), pr[r + 1] * (dpacc[r + 1] - dl));
        }
      };
      static_for<NA>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        constexpr WideOp op = dq_op<ER, DVR>(k);
        ring[(k + AHEAD) & 7] = operand(std::integral_constant<int, k + AHEAD>{});
        if constexpr (op.kind) {
          dpacc = Mma<T>::run(ring[k & 7], dof[op.j], dpacc);
          if constexpr (op.j == 0 && MASKED) bias_log2(bl);
          if constexpr (op.j == 0 && FUNC && GENERAL) {
            // every score through the functors, in one block behind one test: s = mod(scale * s) / scale,
            // so that the code around it is the common one (a call with a window alone skips the block)
            // (one loop per functor behind one test each: tested per score, even a uniform test costs this
            // kernel more than the functor; the soft cap through one exponential and one reciprocal)
            if (p.sm.any) {
              auto kv_of = [&](int r) { return min(ta * BT + (r >> 2) * 8 + half * 4 + (r & 3), p.S - 1); };
#pragma unroll
              for (int r = 0; r < 16; ++r) sacc[r] *= p.scale;
              if (f_kw) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                  bl[r] = f_kw[kv_of(r)];  // (the key's weight is the part of the derivative that the score does not tell)
                  sacc[r] *= bl[r];
                }
              }
              if (p.sm.key_bias) {
                const float* kb = p.sm.key_bias + (int64_t)h * p.S;
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[r] += kb[kv_of(r)];
              }
              if (p.sm.alibi) {
                const float slope = p.sm.alibi[h], base = (float)(ta * BT + half * 4 - qc);  // (keys past S are masked whatever they get)
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[r] = fmaf(slope, base + (float)((r >> 2) * 8 + (r & 3)), sacc[r]);
              }
              if (p.sm.softcap > 0.f) {
                const float cap = p.sm.softcap, inv_cap = 1.f / p.sm.softcap;
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[r] = cap * tanh_fast(sacc[r] * inv_cap);
              }
              if (p.sm.doc_q && p.sm.doc_k) {
                const int32_t mine = p.sm.doc_q[(int64_t)b * p.L + qc];
                const int32_t* dk = p.sm.doc_k + (int64_t)b * p.S;
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[r] = dk[kv_of(r)] != mine ? -INFINITY : sacc[r];
              }
#pragma unroll
              for (int r = 0; r < 16; ++r) sacc[r] *= inv_scale;
            }
          }
#pragma unroll
          for (int r = (op.j * 16) / KSV; r < ((op.j + 1) * 16) / KSV; ++r) prob(r);
        } else {
          sacc = Mma<T>::run(ring[k & 7], qf[op.j], sacc);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
#pragma unroll
      for (int r = 0; r < 8; r += 2) form_ds(r);
      __builtin_amdgcn_sched_barrier(0);
      static_for<2 * DBE>([&](auto ic) {
        constexpr int i = decltype(ic)::value, k = NA + i;
        constexpr WideOp op = dq_op<ER, DVR>(k);
        if constexpr (k + AHEAD < NOPS) ring[(k + AHEAD) & 7] = operand(std::integral_constant<int, k + AHEAD>{});
        constexpr int r0 = (op.j / DB) * 4;
        const u32x4 bS = {pS[r0], pS[r0 + 1], pS[r0 + 2], pS[r0 + 3]};
        dqacc[op.j % DB] = Mma<T>::run(ring[k & 7], bS, dqacc[op.j % DB]);
        if constexpr (i < DBE) {  // the four pairs of the second 16 keys, spread over the first DBE slots
#pragma unroll
          for (int q = (i * 4) / DBE; q < ((i + 1) * 4) / DBE; ++q) form_ds(8 + 2 * q);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      if constexpr (MASKED) {
        if (gb_row) {
#pragma unroll
          for (int g = 0; g < 4; ++g)
            if (ta * BT + g * 8 + half * 4 < p.S) *(u32x2*)(gb_row + ta * BT + g * 8) = u32x2{pS[2 * g], pS[2 * g + 1]};
        }
      }
    };
    if (t < nt_w) {
      if constexpr (FUNC) {
        // does the tile cross the diagonal, the end of the keys or the edge of a window of this wavefront's rows?
        const int k_lo = tile_of(t) * BT, k_hi = k_lo + BT - 1;
        const bool edge_t = k_hi >= S || (p.causal && k_hi > qw0) || (p.window > 0 && k_lo < qw0 + 31 - p.window + 1 && k_hi >= p.sink_keys);
        if (edge_t || need_dfac || p.sm.any) tile(std::true_type{});
        else tile(std::false_type{});
      } else {
        tile(std::true_type{});
      }
    }
#pragma unroll
    for (int i = 0; i < DBE; ++i) asm volatile("" : "+a"(dqacc[i]));
    if (t + 1 < nt) publish_tile();
  }
  if constexpr (MASKED) {
    if (gb_row) {  // the tiles this wavefront did not walk: above the diagonal, past the batch's keys
      for (int t = min(nt_w, nt); t * BT < p.S; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          if (t * BT + g * 8 + half * 4 < p.S) *(u32x2*)(gb_row + t * BT + g * 8) = u32x2{0u, 0u};
    }
  }
  if (qrow < p.L) {
    uint16_t* gq = (uint16_t*)p.gq + b * p.gq_sb + h * p.gq_sh + (int64_t)qrow * p.gq_sl;
#pragma unroll
    for (int db = 0; db < DBE; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        w[0] = Mma<T>::pack(dqacc[db][g * 4] * p.scale, dqacc[db][g * 4 + 1] * p.scale);
        w[1] = Mma<T>::pack(dqacc[db][g * 4 + 2] * p.scale, dqacc[db][g * 4 + 3] * p.scale);
        if (db * 32 + g * 8 + half * 4 < er) *(u32x2*)(gq + db * 32 + g * 8 + half * 4) = w;
      }
  }
}

// TABLES (masked instances): the tile skip table of a per-score mask is honoured.  At full width the
// kernel has scalar registers for the table or for the split of a key block's query tiles over
// workgroups, not for both: one instance of each.
template <typename T, int ER, int DVR, int MODE, bool TABLES>
__global__ __launch_bounds__(256, 1) void bwd_wide_dkdv_kernel(BwdM p) {
  constexpr bool MASKED = MODE == 1 || MODE == 3, FUNC = MODE == 2, DROP = MODE == 3;  // (see bwd_wide_dq_kernel)
  constexpr int KSE = ER / 16, KSV = DVR / 16, DBE = ER / 32, DBV = DVR / 32;
  extern __shared__ __attribute__((aligned(16))) uint16_t wide_lds[];
  uint16_t* const q_buf = wide_lds;                        // [2][TILE_ELEMS]
  uint16_t* const do_buf = wide_lds + 2 * TILE_ELEMS;      // [2][TILE_ELEMS]
  float* const lse_buf = (float*)(wide_lds + 4 * TILE_ELEMS);  // [2][BT]
  float* const dl_buf = lse_buf + 2 * BT;                      // [2][BT]
  uint32_t* const live_s = (uint32_t*)(dl_buf + 2 * BT);       // (masked instances) [heads of the group][words]
  const int streams = p.B * p.Hkv;
  // (split query tiles: part by part, so that a (batch, kv head) keeps its place modulo 8 in the launch order)
  constexpr bool SPLIT = !(TABLES && ER + DVR > 320);
  // (the part is worked out again where the results are written rather than kept in a register all along)
  auto parts_of = [&]() { return SPLIT ? p.parts : 1; };
  auto part_of = [&]() { return parts_of() > 1 ? (int)blockIdx.x / (p.B * p.Hkv * p.n_kt) : 0; };
  const int blk = parts_of() > 1 ? blockIdx.x - part_of() * (streams * p.n_kt) : blockIdx.x;
  const int kt = blk / streams;  // low key tiles see the most queries under a causal mask: first
  const int st = blk % streams, b = st / p.Hkv, hk = st % p.Hkv, rep = p.Hq / p.Hkv;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 31, half = lane >> 5;
  const int k0 = kt * 128, kw0 = k0 + wave * 32, key = kw0 + col;
  const int er = p.d_real, dvr = p.dv_real;

  int S = p.S;  // keys of this batch that take part
  if constexpr (MODE != 0) {
    if (p.kv_lens) S = min(S, max(p.kv_lens[b], 0));
  }
  // the first query row that sees this lane's key: the key itself under a causal mask, none for a key
  // past the batch's count
  const int first_q = key >= S ? INT_MAX : p.causal ? key : INT_MIN;
  // (FUNC) ... and the first row past its window, unless it is a sink key; what the functors' derivative needs
  const int past_q = (FUNC && p.window > 0 && key >= p.sink_keys) ? key + p.window : INT_MAX;
  const float inv_scale = FUNC ? 1.f / p.scale : 0.f;
  const float icap = (FUNC && p.sm.softcap > 0.f) ? p.scale / p.sm.softcap : 0.f;
  u32x4 kf[KSE], vf[KSV];
  {
    const int kc = max(min(key, S - 1), 0);  // (a live row: rows past the batch's keys may hold anything)
    const uint16_t* kr = (const uint16_t*)p.k + b * p.k_sb + hk * p.k_sh + (int64_t)kc * p.k_sl + half * 8;
    const uint16_t* vr = (const uint16_t*)p.v + b * p.v_sb + hk * p.v_sh + (int64_t)kc * p.v_sl + half * 8;
#pragma unroll
    for (int ks = 0; ks < KSE; ++ks) kf[ks] = half * 8 + ks * 16 < er ? *(const u32x4*)(kr + ks * 16) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int ks = 0; ks < KSV; ++ks) vf[ks] = half * 8 + ks * 16 < dvr ? *(const u32x4*)(vr + ks * 16) : u32x4{0u, 0u, 0u, 0u};
  }
  TrOffSwz tr;
  tr.init(lane);
  const int swz_col = tile_swz<DW>(col);
  f32x16 dkacc[DBE], dvacc[DBV];
#pragma unroll
  for (int i = 0; i < DBE; ++i) zero(dkacc[i]);
#pragma unroll
  for (int i = 0; i < DBV; ++i) zero(dvacc[i]);
  const float c = p.scale * kLog2eF;
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int nqs = (p.L + BT - 1) / BT;
  const int qs_begin = p.causal ? min(k0 / BT, nqs) : 0;

  // Items: query tile by query tile from the last one down, heads inside: the workgroups of a kv head,
  // which share an XCD, then want the same Q / dO tile at about the same time and find it in its L2.
  // (sliding window: rows past the window of the block's last key see none of its keys, unless it holds sink keys)
  int qs_top = nqs;
  if constexpr (FUNC) {
    if (p.window > 0 && k0 >= p.sink_keys) qs_top = max(min(nqs, (k0 + 128 + p.window - 2) / BT + 1), qs_begin);
  }
  int qs_hi = qs_top, qs_lo = qs_begin;  // this workgroup's query tiles: qs_hi - 1 down to qs_lo
  if (parts_of() > 1) {
    const int chunk = (qs_top - qs_begin + parts_of() - 1) / parts_of();
    qs_hi = qs_top - part_of() * chunk, qs_lo = max(qs_hi - chunk, qs_begin);
  }
  const int n_items = (MODE != 0 && k0 >= S) ? 0 : max(qs_hi - qs_lo, 0) * rep;  // no live key in this block: zeros
  // bias of this lane's key in the 32 rows of an item, one element per score register, requested
  // ahead of the item's first product through a resource that ends with the (batch, head)'s last row
  const int bkind = MASKED ? __builtin_amdgcn_readfirstlane(p.bias_kind) : 0;  // 0 none, 1 float32, 2 float16, 3 bfloat16, 4 bool
  const int besz = __builtin_amdgcn_readfirstlane(bkind == 1 ? 4 : bkind == 4 ? 1 : 2);  // (in a scalar register: a descriptor built from a vector register is looked up lane by lane)
  const uint32_t b_rowbytes = MASKED ? (uint32_t)(p.bias_sl * besz) : 0u;
  const uint32_t b_lane = MASKED ? (uint32_t)((half * 4 * p.bias_sl + min(key, p.S - 1)) * besz) : 0u;
  const int b_records = MASKED ? __builtin_amdgcn_readfirstlane((int)(((int64_t)(p.L - 1) * p.bias_sl + p.S) * besz)) : 0;
  uint32_t braw[16];
  // (DROP) the keep bytes of the same 16 scores, requested with the bias; then one bit each: bit r says
  // that the score of accumulator register r is kept
  uint32_t kbits = 0u;
  auto request_keep = [&](int hg, int q0, uint32_t (&kb)[DROP ? 16 : 1]) {
    if constexpr (DROP) {
      const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
          uniform_ptr((const char*)p.keep + ((int64_t)b * p.Hq + hk * rep + hg) * p.L * p.keep_ld), 0,
          __builtin_amdgcn_readfirstlane((int)((int64_t)(p.L - 1) * p.keep_ld + p.S)), 0x00020000);
      const uint32_t base = (uint32_t)((q0 + half * 4) * p.keep_ld + min(key, p.S - 1));
#pragma unroll
      for (int r = 0; r < 16; ++r) kb[r] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b8(k_rsrc, base + (uint32_t)(((r >> 2) * 8 + (r & 3)) * p.keep_ld), 0, 0);
    }
  };
  auto pack_keep = [&](const uint32_t (&kb)[DROP ? 16 : 1]) {
    if constexpr (DROP) {
      kbits = 0u;
#pragma unroll
      for (int r = 0; r < 16; ++r) kbits |= min(kb[r], 1u) << r;
    }
  };
  auto load_bias = [&](int hg, int q0) {
    if constexpr (MASKED) {
      if (!bkind) return;
      const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
          uniform_ptr((const char*)p.bias + (b * p.bias_sb + (hk * rep + hg) * p.bias_sh) * besz), 0, b_records, 0x00020000);
      const uint32_t base = b_lane + (uint32_t)q0 * b_rowbytes;
      auto each = [&](auto fetch) {
#pragma unroll
        for (int r = 0; r < 16; ++r) braw[r] = fetch(base + (uint32_t)((r >> 2) * 8 + (r & 3)) * b_rowbytes);
      };
      if (bkind == 1) each([&](uint32_t off) { return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(b_rsrc, off, 0, 0); });
      else if (bkind == 4) each([&](uint32_t off) { return (uint32_t)__builtin_amdgcn_raw_buffer_load_b8(b_rsrc, off, 0, 0); });
      else each([&](uint32_t off) { return (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(b_rsrc, off, 0, 0); });
    }
  };
  // ... turned into floats in the log2 domain in place (the element type is tested once, outside the loop)
  auto bias_to_log2 = [&]() {
    auto each = [&](auto conv) {
#pragma unroll
      for (int r = 0; r < 16; ++r) braw[r] = __builtin_bit_cast(uint32_t, conv(braw[r]));
    };
    if (bkind == 1) each([](uint32_t x) { return __builtin_bit_cast(float, x) * kLog2eF; });
    else if (bkind == 4) each([](uint32_t x) { return x ? 0.f : -INFINITY; });
    else if (bkind == 3) each([](uint32_t x) { return __builtin_bit_cast(float, x << 16) * kLog2eF; });
    else if (bkind == 2) each([](uint32_t x) { return (float)__builtin_bit_cast(_Float16, (uint16_t)x) * kLog2eF; });
    else each([](uint32_t) { return 0.f; });
  };
  typedef __attribute__((address_space(3))) unsigned char* lds_bytes;
  const uint32_t lds_q = (uint32_t)(uintptr_t)(lds_bytes)q_buf, lds_do = (uint32_t)(uintptr_t)(lds_bytes)do_buf;
  constexpr int NLD = TILE_LOADS / 4;  // loads per wavefront and tile
  // With a skip table: an item whose 64-row block holds no kept score for this key block is neither
  // fetched nor computed.
  bool listed = false;
  if constexpr (TABLES) {
    if (p.live_t && !p.causal && rep * p.live_t_words <= 256) {
      listed = true;
      if (tid < rep * p.live_t_words) {
        const int hd = hk * rep + tid / p.live_t_words;
        live_s[tid] = p.live_t[(((int64_t)(p.bias_sb ? b : 0) * p.live_hm + (p.bias_sh ? hd : 0)) * ((p.S + 127) / 128) + kt) * p.live_t_words +
                               tid % p.live_t_words];
      }
      __syncthreads();
    }
  }
  auto item_live = [&](int qs, int hg) {
    if constexpr (MASKED) {
      if (listed) {
        const int qt = qs >> 1;  // 64-row blocks of the table, 32-row items here
        return ((__builtin_amdgcn_readfirstlane((int)live_s[hg * p.live_t_words + (qt >> 5)]) >> (qt & 31)) & 1) != 0;
      }
    }
    return true;
  };
  // item `it` into buffer it % 2; the row statistics travel in two registers of the first 32 threads.
  // The buffers start at the tile's first row and end with the head's last row: rows past L read as zeros.
  float lse_n = INFINITY, dl_n = 0.f;
  auto request_item = [&](int qs, int hg, int buf) {
    const int h = hk * rep + hg, q0 = qs * BT;
    if (tid < BT) {  // (ordinary loads, ahead of the tile loads: the compiler's wait for them then waits for nothing else)
      const int qi = q0 + tid;
      const int64_t row = ((int64_t)b * p.Hq + h) * p.L + min(qi, p.L - 1);
      // rows past L are switched off through lse = +inf
      lse_n = qi < p.L ? p.lse2[row] : INFINITY;
      dl_n = qi < p.L ? p.delta[row] : 0.f;
    }
    const int rows = p.L - q0;  // >= 1
    const u32x4 q_rsrc = wide_descriptor((const uint16_t*)p.q + b * p.q_sb + h * p.q_sh + (int64_t)q0 * p.q_sl, ((int64_t)(rows - 1) * p.q_sl + er) * 2);
    const u32x4 go_rsrc = wide_descriptor((const uint16_t*)p.go + b * p.go_sb + h * p.go_sh + (int64_t)q0 * p.go_sl, ((int64_t)(rows - 1) * p.go_sl + dvr) * 2);
    const uint32_t boff = (uint32_t)(buf * TILE_ELEMS * 2);
#pragma unroll
    for (int n = 0; n < NLD; ++n) {
      const int ld = wave + 4 * n;  // (uniform per wavefront)
      // (offsets recomputed per item, a handful of vector instructions, rather than held in registers
      // that this kernel does not have)
      wide_tile_load(q_rsrc, wide_chunk_off(ld, lane, (int)p.q_sl, er), lds_q + boff + ld * 1024);
      wide_tile_load(go_rsrc, wide_chunk_off(ld, lane, (int)p.go_sl, dvr), lds_do + boff + ld * 1024);
    }
  };
  auto publish_item = [&](int buf) {  // after this, the item in `buf` may be read by every wavefront
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (tid < BT) lse_buf[buf * BT + tid] = lse_n, dl_buf[buf * BT + tid] = dl_n;
    __syncthreads();
  };
  if (n_items > 0) {
    if (item_live(qs_hi - 1, 0)) request_item(qs_hi - 1, 0, 0);
    publish_item(0);
  }
  int buf = 0;
  // (two nested loops on purpose: written as one loop over items, the compiler spills the fragments)
  for (int qs = qs_hi - 1; qs >= qs_lo; --qs) {
    for (int hg = 0; hg < rep; ++hg) {
    const bool last = qs == qs_lo && hg == rep - 1;
    // (the other buffer was last read before the barrier that ended the previous item)
    const int qs_n = hg + 1 < rep ? qs : qs - 1, hg_n = hg + 1 < rep ? hg + 1 : 0;
    if (!last && item_live(qs_n, hg_n)) request_item(qs_n, hg_n, buf ^ 1);
    const int q0 = qs * BT;
    // (FUNC: every row of the tile past the window of every key of this wavefront, none of them a sink key)
    const bool past_window = FUNC && p.window > 0 && q0 - (kw0 + 31) >= p.window && kw0 >= p.sink_keys;
    if (!((p.causal && q0 + BT - 1 < kw0) || kw0 >= S || past_window) && item_live(qs, hg)) {  // (uniform per wavefront)
      // (written in place, not as a lambda with a plain and a general variant as in the dQ kernel: wrapped,
      // the full-width instances spill more, and the items of a window's inside gain little)
      constexpr bool GENERAL = true;
      // (at full width the bias is requested behind the score products: ahead of them its 16
      // registers are more than the register file has left)
      uint32_t kb[DROP ? 16 : 1];
      if constexpr (ER + DVR <= 320) load_bias(hg, q0), request_keep(hg, q0, kb);
      const uint16_t* q_t = q_buf + buf * TILE_ELEMS;
      const uint16_t* do_t = do_buf + buf * TILE_ELEMS;
      const float* lse_s = lse_buf + buf * BT;
      const float* dl_s = dl_buf + buf * BT;
      // the accumulators are touched by matrix ops only: accumulation registers; the K / V fragments
      // feed every matrix op as a source operand: ordinary vector registers
#pragma unroll
      for (int i = 0; i < DBE; ++i) asm volatile("" : "+a"(dkacc[i]));
#pragma unroll
      for (int i = 0; i < DBV; ++i) asm volatile("" : "+a"(dvacc[i]));
      // The matrix ops of an item in the order S, dP, dV, dK, with the vector work between them placed
      // where the matrix pipe still has the previous ops to execute: the probabilities are formed
      // while dP runs, dS (from the probabilities as they feed the matrix pipe, rounded to the input
      // dtype) while dV runs.  One wavefront per SIMD has nobody else to overlap with.  The LDS
      // operands - row fragments of Q, then of dO, then the transposed fragments of dO, then of Q -
      // travel through one register ring, two to four matrix ops ahead of their use, with the order
      // pinned by scheduling fences.
      constexpr int AHEAD = ER + DVR <= 320 ? 4 : 2, NOPS = KSE + KSV + 2 * (DBE + DBV);  // (deeper where the widths leave registers)
      auto operand = [&](auto kc) {
        constexpr WideOp op = dkdv_op<ER, DVR>(decltype(kc)::value);
        if constexpr (op.kind >= 2) return tr.cols(op.kind == 3 ? q_t : do_t, op.j);
        else return *(const u32x4*)((op.kind ? do_t : q_t) + wide_row_off(op.j, col, half, swz_col));
      };
      u32x4 ring[8];
      static_for<AHEAD>([&](auto kc) { ring[decltype(kc)::value] = operand(kc); });
      uint32_t pP[8], pS[8];
      uint32_t pF[FUNC && GENERAL ? 8 : 1];  // (FUNC) the probabilities times the derivative of the functors, for dS
      uint32_t pM[DROP ? 8 : 1];             // (DROP) the kept probabilities, for dV
      // (at full width the register file has no room for the score and the dP accumulator at once next
      // to the two fragments: there the probabilities are formed before dP is issued, uncovered)
      constexpr bool BOTH = ER + DVR <= 320;
      f32x16 sacc = zero16, dpacc = zero16;
      auto issue = [&](auto first, auto count) {  // ops first .. first + count - 1 of the S / dP part
        static_for<decltype(count)::value>([&](auto jc) {
          constexpr int k = decltype(first)::value + decltype(jc)::value;
          constexpr WideOp op = dkdv_op<ER, DVR>(k);
          ring[(k + AHEAD) & 7] = operand(std::integral_constant<int, k + AHEAD>{});
          if constexpr (op.kind) dpacc = Mma<T>::run(ring[k & 7], vf[op.j], dpacc);
          else sacc = Mma<T>::run(ring[k & 7], kf[op.j], sacc);
          __builtin_amdgcn_sched_barrier(0);
        });
      };
      auto issue_dp = [&]() { issue(std::integral_constant<int, KSE>{}, std::integral_constant<int, KSV>{}); };
      if constexpr (BOTH) issue(std::integral_constant<int, 0>{}, std::integral_constant<int, KSE + KSV>{});
      else issue(std::integral_constant<int, 0>{}, std::integral_constant<int, KSE>{});
      if constexpr (!BOTH) load_bias(hg, q0), request_keep(hg, q0, kb);
      if constexpr (MASKED) bias_to_log2();
      pack_keep(kb);
      // (FUNC) what the functors take from this lane's key, for the item's head
      float f_w = 1.f;
      if constexpr (FUNC && GENERAL) {
        // every score through the functors, in one block behind one test: s = mod(scale * s) / scale, so
        // that the code below is the common one (a call with a window alone skips the block)
        if (p.sm.any) {
          const int hq = hk * rep + hg, kc = max(min(key, p.S - 1), 0);
          float f_kb = 0.f, f_slope = 0.f;
          int f_doc = 0;
          if (p.sm.key_weight) f_w = p.sm.key_weight[(int64_t)hq * p.S + kc];
          if (p.sm.key_bias) f_kb = p.sm.key_bias[(int64_t)hq * p.S + kc];
          if (p.sm.alibi) f_slope = p.sm.alibi[hq];
          const bool docs = p.sm.doc_q && p.sm.doc_k;
          if (docs) f_doc = p.sm.doc_k[(int64_t)b * p.S + kc];
          // (one loop per functor behind one test each, as in the dQ kernel)
          const float sw = p.scale * f_w;
#pragma unroll
          for (int r = 0; r < 16; ++r) sacc[r] = fmaf(sacc[r], sw, f_kb);
          if (p.sm.alibi) {
            const float base = (float)(key - q0 - half * 4);
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[r] = fmaf(f_slope, base - (float)((r >> 2) * 8 + (r & 3)), sacc[r]);
          }
          if (p.sm.softcap > 0.f) {
            const float cap = p.sm.softcap, inv_cap = 1.f / p.sm.softcap;
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[r] = cap * tanh_fast(sacc[r] * inv_cap);
          }
          if (docs) {
            const int32_t* dq = p.sm.doc_q + (int64_t)b * p.L;
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[r] = dq[min(q0 + (r >> 2) * 8 + half * 4 + (r & 3), p.L - 1)] != f_doc ? -INFINITY : sacc[r];
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) sacc[r] *= inv_scale;
        }
      }
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const f32x4 l4 = *(const f32x4*)(&lse_s[r4 * 8 + half * 4]);
        float pr[4];
        float df[FUNC && GENERAL ? 4 : 1];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = r4 * 4 + e, qi = q0 + r4 * 8 + half * 4 + e;
          float x;
          if constexpr (FUNC && GENERAL) {
            // (the scores went through the functors in a block of their own, see above; the derivative:
            // 1 - tanh^2 of the soft cap, recovered from the capped score, times this key's weight)
            x = qi >= past_q ? -INFINITY : fmaf(sacc[r], c, -l4[e]);
            const float th = sacc[r] * icap;
            df[e] = fmaf(-th, th, 1.f) * f_w;
          } else if constexpr (MASKED) {
            x = fmaf(sacc[r], c, __builtin_bit_cast(float, braw[r])) - l4[e];
          } else {
            x = fmaf(sacc[r], c, -l4[e]);
          }
          // (masked before the exponential: a select around it is compiled into a branch per element)
          pr[e] = __builtin_amdgcn_exp2f(qi < first_q ? -INFINITY : x);
        }
        pP[r4 * 2] = Mma<T>::pack(pr[0], pr[1]), pP[r4 * 2 + 1] = Mma<T>::pack(pr[2], pr[3]);
        if constexpr (DROP) {  // dV gets the kept probabilities, dS all of them
#pragma unroll
          for (int e = 0; e < 4; ++e) pr[e] = ((kbits >> (r4 * 4 + e)) & 1u) ? pr[e] : 0.f;
          pM[r4 * 2] = Mma<T>::pack(pr[0], pr[1]), pM[r4 * 2 + 1] = Mma<T>::pack(pr[2], pr[3]);
        }
        if constexpr (FUNC && GENERAL) {  // (a dropped score may carry any derivative)
#pragma unroll
          for (int e = 0; e < 4; ++e) df[e] = pr[e] == 0.f ? 0.f : pr[e] * df[e];
          pF[r4 * 2] = Mma<T>::pack(df[0], df[1]), pF[r4 * 2 + 1] = Mma<T>::pack(df[2], df[3]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (!BOTH) issue_dp();
      auto form_ds = [&]() {
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const f32x4 d4 = *(const f32x4*)(&dl_s[r4 * 8 + half * 4]);
          float ds[4];
#pragma unroll
          for (int e = 0; e < 4; ++e)
          {
            uint32_t w;
            if constexpr (FUNC && GENERAL) w = pF[r4 * 2 + (e >> 1)];
            else w = pP[r4 * 2 + (e >> 1)];
            if constexpr (DROP) {
              const float kf = ((kbits >> (r4 * 4 + e)) & 1u) ? p.keep_scale : 0.f;
              ds[e] = Mma<T>::unpack(w, e & 1) * fmaf(dpacc[r4 * 4 + e], kf, -d4[e]);
            } else {
              ds[e] = Mma<T>::unpack(w, e & 1) * (dpacc[r4 * 4 + e] - d4[e]);
            }
          }
          pS[r4 * 2] = Mma<T>::pack(ds[0], ds[1]), pS[r4 * 2 + 1] = Mma<T>::pack(ds[2], ds[3]);
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      if constexpr (!BOTH) form_ds();
      static_for<2 * DBV>([&](auto ic) {
        constexpr int k = KSE + KSV + decltype(ic)::value;
        constexpr WideOp op = dkdv_op<ER, DVR>(k);
        if constexpr (k + AHEAD < NOPS) ring[(k + AHEAD) & 7] = operand(std::integral_constant<int, k + AHEAD>{});
        constexpr int r0 = (op.j / DB) * 4;
        u32x4 bP;
        if constexpr (DROP) bP = u32x4{pM[r0], pM[r0 + 1], pM[r0 + 2], pM[r0 + 3]};
        else bP = u32x4{pP[r0], pP[r0 + 1], pP[r0 + 2], pP[r0 + 3]};
        dvacc[op.j % DB] = Mma<T>::run(ring[k & 7], bP, dvacc[op.j % DB]);
        __builtin_amdgcn_sched_barrier(0);
      });
      if constexpr (BOTH) form_ds();
      static_for<2 * DBE>([&](auto ic) {
        constexpr int k = KSE + KSV + 2 * DBV + decltype(ic)::value;
        constexpr WideOp op = dkdv_op<ER, DVR>(k);
        if constexpr (k + AHEAD < NOPS) ring[(k + AHEAD) & 7] = operand(std::integral_constant<int, k + AHEAD>{});
        constexpr int r0 = (op.j / DB) * 4;
        const u32x4 bS = {pS[r0], pS[r0 + 1], pS[r0 + 2], pS[r0 + 3]};
        dkacc[op.j % DB] = Mma<T>::run(ring[k & 7], bS, dkacc[op.j % DB]);
        __builtin_amdgcn_sched_barrier(0);
      });
    }
    buf ^= 1;
    if (!last) publish_item(buf);
    }
  }
  // Results leave through buffer stores whose offset is pushed past the buffer's end where a lane has
  // nothing to write (a key past S, columns past the real width): the hardware drops such a store, and
  // the write-out is one straight run of stores (as tests per store it is a chain of 64 branches around
  // which the compiler parks accumulators in scratch).
  constexpr uint32_t kDrop = 0xfffffff0u;
  const bool live_key = key < p.S;
  if (parts_of() > 1) {  // float32 rows for bwd_dkdv_merge_kernel, which also multiplies dK by the scale
    const int64_t row0 = (((int64_t)part_of() * p.B + b) * p.Hkv + hk) * p.S;
    const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr((char*)(p.part_dk + row0 * er)), 0,
                                                                       __builtin_amdgcn_readfirstlane((int)((int64_t)p.S * er * 4)), 0x00020000);
    const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr((char*)(p.part_dv + row0 * dvr)), 0,
                                                                       __builtin_amdgcn_readfirstlane((int)((int64_t)p.S * dvr * 4)), 0x00020000);
    const uint32_t ok = (uint32_t)((key * er + half * 4) * 4), ov = (uint32_t)((key * dvr + half * 4) * 4);
#pragma unroll
    for (int db = 0; db < DBE; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = db * 32 + g * 8;
        const f32x4 w = {dkacc[db][g * 4], dkacc[db][g * 4 + 1], dkacc[db][g * 4 + 2], dkacc[db][g * 4 + 3]};
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, w), rk, (live_key && d + half * 4 < er) ? ok + d * 4 : kDrop, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);  // (block by block: left alone, every accumulator is read out before the first store)
    }
#pragma unroll
    for (int db = 0; db < DBV; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = db * 32 + g * 8;
        const f32x4 w = {dvacc[db][g * 4], dvacc[db][g * 4 + 1], dvacc[db][g * 4 + 2], dvacc[db][g * 4 + 3]};
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, w), rv, (live_key && d + half * 4 < dvr) ? ov + d * 4 : kDrop, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  } else {
    const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
        uniform_ptr((char*)((uint16_t*)p.gk + b * p.gk_sb + hk * p.gk_sh)), 0,
        __builtin_amdgcn_readfirstlane((int)(((int64_t)(p.S - 1) * p.gk_sl + er) * 2)), 0x00020000);
    const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
        uniform_ptr((char*)((uint16_t*)p.gv + b * p.gv_sb + hk * p.gv_sh)), 0,
        __builtin_amdgcn_readfirstlane((int)(((int64_t)(p.S - 1) * p.gv_sl + dvr) * 2)), 0x00020000);
    const uint32_t ok = (uint32_t)(((int64_t)key * p.gk_sl + half * 4) * 2), ov = (uint32_t)(((int64_t)key * p.gv_sl + half * 4) * 2);
    const float v_scale = DROP ? p.keep_scale : 1.f;  // (dropout's 1 / (1 - p) on the kept probabilities)
#pragma unroll
    for (int db = 0; db < DBE; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = db * 32 + g * 8;
        u32x2 wk;
        wk[0] = Mma<T>::pack(dkacc[db][g * 4] * p.scale, dkacc[db][g * 4 + 1] * p.scale);
        wk[1] = Mma<T>::pack(dkacc[db][g * 4 + 2] * p.scale, dkacc[db][g * 4 + 3] * p.scale);
        __builtin_amdgcn_raw_buffer_store_b64(wk, rk, (live_key && d + half * 4 < er) ? ok + d * 2 : kDrop, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int db = 0; db < DBV; ++db) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = db * 32 + g * 8;
        u32x2 wv;
        wv[0] = Mma<T>::pack(dvacc[db][g * 4] * v_scale, dvacc[db][g * 4 + 1] * v_scale);
        wv[1] = Mma<T>::pack(dvacc[db][g * 4 + 2] * v_scale, dvacc[db][g * 4 + 3] * v_scale);
        __builtin_amdgcn_raw_buffer_store_b64(wv, rv, (live_key && d + half * 4 < dvr) ? ov + d * 2 : kDrop, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

template <typename T, int ER, int DVR, int MODE, bool TABLES>
int launch_dkdv(const BwdM& g, int64_t k_blocks, hipStream_t s) {
  constexpr int kDkdvLds = WIDE_DKDV_LDS + (MODE == 1 ? WIDE_LIVE_LDS : 0);
  static LdsOnce once;
  const hipError_t attr = reserve_lds(once, (const void*)bwd_wide_dkdv_kernel<T, ER, DVR, MODE, TABLES>, kDkdvLds);
  if (attr != hipSuccess) {
    set_error("SDPA: cannot reserve %d bytes of LDS for bwd_wide_dkdv_kernel: %s", kDkdvLds, hipGetErrorString(attr));
    return MI355_SDPA_ERR_LAUNCH;
  }
  hipLaunchKernelGGL((bwd_wide_dkdv_kernel<T, ER, DVR, MODE, TABLES>), dim3((unsigned)(k_blocks * g.parts)), dim3(256), kDkdvLds, s, g);
  return check_launch("bwd_wide_dkdv_kernel");
}

// NO_TABLES: the masked full-width dK/dV instance that splits instead of reading a skip table
template <typename T, int ER, int DVR, int MODE, bool NO_TABLES = false>
int launch_t(const BwdM& g, hipStream_t s) {
  const int64_t q_blocks = (int64_t)g.B * g.Hq * ((g.L + 127) / 128), k_blocks = (int64_t)g.B * g.Hkv * ((g.S + 127) / 128);
  if (q_blocks > 0x7fffffff || k_blocks > 0x7fffffff) {
    set_error("SDPA: too many tiles for the wide backward kernels");
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  constexpr int kDqLds = WIDE_DQ_LDS + (MODE == 1 ? WIDE_LIST_LDS : 0);
  static LdsOnce once_q;
  const hipError_t attr_q = reserve_lds(once_q, (const void*)bwd_wide_dq_kernel<T, ER, DVR, MODE>, kDqLds);
  if (attr_q != hipSuccess) {
    set_error("SDPA: cannot reserve %d bytes of LDS for bwd_wide_dq_kernel: %s", kDqLds, hipGetErrorString(attr_q));
    return MI355_SDPA_ERR_LAUNCH;
  }
  hipLaunchKernelGGL((bwd_wide_dq_kernel<T, ER, DVR, MODE>), dim3((unsigned)q_blocks), dim3(256), kDqLds, s, g);
  int rc = check_launch("bwd_wide_dq_kernel");
  if (rc) return rc;
  rc = launch_dkdv<T, ER, DVR, MODE, MODE == 1 && !(NO_TABLES && ER + DVR > 320)>(g, k_blocks, s);
  if (rc || g.parts == 1) return rc;
  return launch_bwd_dkdv_merge(g, std::is_same<T, bf16_t>::value ? MI355_SDPA_BF16 : MI355_SDPA_F16, s);
}
// widths the kernels are instantiated for: 192 / 128 (multi-head latent attention) and the full 256 / 256
template <typename T>
int launch_w(const BwdM& g, hipStream_t s) {
  const bool func = g.window > 0 || g.sm.any;  // (never together with a bias: refused before)
  const bool masked = g.bias_kind || g.kv_lens;  // (a bias gradient comes with a bias)
  const bool drop = g.keep_scale != 0.f;          // (never together with a functor or a skip table: refused before)
  if (drop && (!g.keep || func || g.live_t || g.live_tiles)) {
    set_error("SDPA: dropout in the wide backward kernels needs a keep-mask, no functor and no tile table");
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  if (g.d_real <= 192 && g.dv_real <= 128)
    return drop ? launch_t<T, 192, 128, 3>(g, s)
           : func ? launch_t<T, 192, 128, 2>(g, s) : masked ? launch_t<T, 192, 128, 1>(g, s) : launch_t<T, 192, 128, 0>(g, s);
  if (drop) return launch_t<T, 256, 256, 3>(g, s);
  if (func) return launch_t<T, 256, 256, 2>(g, s);
  if (masked && g.parts > 1) return launch_t<T, 256, 256, 1, true>(g, s);  // (bwd_wide_parts: no skip table then)
  return masked ? launch_t<T, 256, 256, 1>(g, s) : launch_t<T, 256, 256, 0>(g, s);
}

}  // namespace

// As in bwd_dkdv_w32.hip: with fewer key blocks than keep the compute units busy, the query tiles of a
// key block go to `parts` workgroups (every head of the group with each tile), at least 16 items - a
// 32-row tile of one head here - a part.
int bwd_wide_parts(const BwdM& g) {
  const int64_t wgs = (int64_t)g.B * g.Hkv * g.n_kt;
  if (wgs >= 384 || wgs <= 0) return 1;
  // (the masked instance at full width either reads a skip table or splits)
  if ((g.bias_kind || g.kv_lens) && !(g.d_real <= 192 && g.dv_real <= 128) && g.live_t) return 1;
  const int64_t tiles = (g.L + BT - 1) / BT;
  const int64_t items = tiles * (g.Hq / g.Hkv);
  if (items < 48) return 1;
  return (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>((768 + wgs - 1) / wgs, std::min(items / 16, tiles)), 16));
}

int launch_bwd_wide(const BwdM& g0, int dtype, hipStream_t s) {
  BwdM g = g0;
  if (!g.part_dk || !g.part_dv) g.parts = 1;
  return dtype == MI355_SDPA_BF16 ? launch_w<bf16_t>(g, s) : launch_w<f16_t>(g, s);
}

}  // namespace mi355
