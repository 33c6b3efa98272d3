// Flash attention for float32 inputs on the float32 matrix op (v_mfma_f32_32x32x2_f32), forward and
// backward, head dims up to 256 with D_v <= D_qk (multiples of 8; narrower rows count as zero padded:
// instances of width 64, 128 and 256), causal or
// unmasked, with per-batch key counts; instances with a per-score bias / keep-mask (and its gradient)
// and / or dropout, and instances with the mask and score functors (sliding window with sink keys, sink
// logits, the functors and document ids of score_mod.h, element by element).  The reference's fused gate takes float32 (decompositions.py:2131-2158); everything
// stays in float32 as in torch_neuronx/_sdpa_math.py (float32 inputs accumulate in float32, and the
// probabilities that multiply V are not rounded, :94).
//
// Products are computed transposed, as in the half-precision kernels: a query row (forward, dQ)
// or a key (dK / dV) is a lane, so softmax statistics are per-lane scalars.  With this matrix op a
// lane supplies ONE element per operand (row / column lane % 32, contraction index lane / 32),
// so an accumulator register of one product IS the B operand of a step of the next product, and
// transposed operands are plain 4-byte LDS reads: no packing, no transposing reads.  A 32 x 32 x 2
// op keeps the matrix pipe busy for 64 cycles, which leaves the compiler's own schedule enough
// room: these kernels are not pipelined by hand.
//
//   fwd_f32_kernel        128 query rows per workgroup (4 wavefronts x 32), 32-key tiles
//   bwd_f32_dq_kernel     the same shape; also leaves delta = rowsum(dO * O) and the log2-domain
//                         log-sum-exp in the workspace
//   bwd_f32_dkdv_kernel   128 keys per workgroup; loops over the query heads of the group (the GQA
//                         sum of decompositions.py:2569-2599 happens in registers) and 32-row tiles
#include "bwd_mfma.h"
#include "fwd_mfma.h"

namespace mi355 {
namespace {

constexpr int BT = 32;  // rows of a staged tile
// Width 256 (head dims above 128, D_v <= D_qk): the two tiles of a kernel are more than the 64 KB of
// LDS that a kernel may declare, so they live in the launch's dynamic LDS; and the register file has
// no room for a tile on its way next to the row fragments and accumulators, so a tile is fetched
// where it is stored (FetchAhead false).
extern __shared__ __attribute__((aligned(16))) float wide_f32_lds[];
template <int D> constexpr bool kFetchAhead = D <= 128;
template <int D> constexpr int kTileFloats = BT * (D + 4);

__device__ __forceinline__ f32x16 mma(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// A 32-row tile of a (rows, width) float matrix on its way to LDS, zeros beyond `width` and
// `rows_left`: fetched into registers one tile ahead (the loads travel under the matrix ops of the
// current tile), written to LDS between two barriers.  NT threads, 16-byte chunks; row pitch D + 4
// floats (16-byte row reads of 16 lanes hit every bank once)
template <int D, int NT>
struct TileF32 {
  static constexpr int N = (BT * (D / 4)) / NT;
  f32x4 w[N];
  __device__ __forceinline__ void fetch(const float* base, int64_t row_stride, int rows_left, int width, int tid) {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int u = tid + n * NT, r = u / (D / 4), ch = u % (D / 4);
      w[n] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (r < rows_left && ch * 4 < width) w[n] = *(const f32x4*)(base + (int64_t)r * row_stride + ch * 4);
    }
  }
  __device__ __forceinline__ void put(float* lds, int tid) const {
#pragma unroll
    for (int n = 0; n < N; ++n) {
      const int u = tid + n * NT, r = u / (D / 4), ch = u % (D / 4);
      *(f32x4*)(lds + r * (D + 4) + ch * 4) = w[n];
    }
  }
};

// this lane's half of a row (elements half * D/2 .. +D/2-1), zeros beyond `width`
template <int D>
__device__ __forceinline__ void load_half_row(float (&f)[D / 2], const float* row, int half, int width) {
#pragma unroll
  for (int i = 0; i < D / 8; ++i) {
    const int d = half * (D / 2) + i * 4;
    const f32x4 w = d < width ? *(const f32x4*)(row + d) : f32x4{0.f, 0.f, 0.f, 0.f};
    f[i * 4] = w[0], f[i * 4 + 1] = w[1], f[i * 4 + 2] = w[2], f[i * 4 + 3] = w[3];
  }
}

// acc = rows(tile)[lane % 32] . f over this lane's half of the head dim (A from LDS, B in registers)
template <int D>
__device__ __forceinline__ f32x16 row_product(const float* tile, int col, int half, const float (&f)[D / 2]) {
  f32x16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const float* r = tile + col * (D + 4) + half * (D / 2);
#pragma unroll
  for (int i = 0; i < D / 8; ++i) {
    const f32x4 a = *(const f32x4*)(r + i * 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc = mma(a[e], f[i * 4 + e], acc);
  }
  return acc;
}

// acc[db] += cols(tile)^T . x : contraction over the tile's 32 rows in the order the accumulators of
// a row product hold them (register r of lane half h is row 8 (r / 4) + 4 h + r % 4)
// (NB column blocks of 32, from the column that `tile` points at: the whole width, or the share of one pass)
template <int D, int NB = D / 32>
__device__ __forceinline__ void col_product(f32x16 (&acc)[NB], const float* tile, int col, int half, const f32x16& x) {
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float* row = tile + ((r >> 2) * 8 + half * 4 + (r & 3)) * (D + 4) + col;
#pragma unroll
    for (int db = 0; db < NB; ++db) acc[db] = mma(row[db * 32], x[r], acc[db]);
  }
}

// MASKED instances: an additive bias / bool keep-mask per score (any of the bias dtypes, stride 0 on
// broadcast dimensions) and / or a dropout keep-mask (bytes, (B, Hq, L, S) contiguous, with a nonzero
// keep_scale), one element load per score: a lane's 16 scores of a tile are 4 groups of 4
// consecutive keys of its row (forward, dQ) or 16 rows of its key (dK / dV).
// bias elements as floats, the element type tested once (inside the loop every element carries the branch)
template <typename IDX>
__device__ __forceinline__ void load_bias16(float (&bl)[16], const void* base, int kind, IDX&& idx) {
  if (kind == 1) {
#pragma unroll
    for (int r = 0; r < 16; ++r) bl[r] = ((const float*)base)[idx(r)];
  } else if (kind == 4) {
#pragma unroll
    for (int r = 0; r < 16; ++r) bl[r] = ((const uint8_t*)base)[idx(r)] ? 0.f : -INFINITY;
  } else if (kind == 3) {
#pragma unroll
    for (int r = 0; r < 16; ++r) bl[r] = __builtin_bit_cast(float, (uint32_t)((const uint16_t*)base)[idx(r)] << 16);
  } else {
#pragma unroll
    for (int r = 0; r < 16; ++r) bl[r] = (float)((const _Float16*)base)[idx(r)];
  }
}

template <int D, int WAVES, int MODE>
__global__ __launch_bounds__(64 * WAVES, 1) void fwd_f32_kernel(FwdM p) {
  constexpr bool MASKED = MODE == 1, FUNC = MODE == 2;  // a per-score tensor | window, sinks, score functors
  constexpr int DB = D / 32;
  __shared__ __attribute__((aligned(16))) float k_st[D > 128 ? 4 : BT * (D + 4)];
  __shared__ __attribute__((aligned(16))) float v_st[D > 128 ? 4 : BT * (D + 4)];
  float* const k_t = D > 128 ? wide_f32_lds : k_st;
  float* const v_t = D > 128 ? wide_f32_lds + kTileFloats<D> : v_st;
  const int qt = p.n_qt - 1 - blockIdx.x / (p.B * p.Hq);  // heavy query tiles first
  const int bh = blockIdx.x % (p.B * p.Hq), b = bh / p.Hq, h = bh % p.Hq, hk = h / (p.Hq / p.Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 31, half = lane >> 5;
  constexpr int BM = 32 * WAVES;  // query rows per workgroup
  const int q0 = qt * BM, qw0 = q0 + wave * 32, qrow = qw0 + col, qc = min(qrow, p.L - 1);
  float qf[D / 2];
  load_half_row<D>(qf, (const float*)p.q + b * p.q_sb + h * p.q_sh + (int64_t)qc * p.q_sl, half, p.d_real);
  f32x16 oacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) zero(oacc[i]);
  float m_run = -INFINITY, l_run = 0.f;  // (l_run: this lane half's keys only; the halves share m_run)
  const float c = p.scale * kLog2eF;
  const float inv_scale = 1.f / p.scale;
  const float* kp = (const float*)p.k + b * p.k_sb + hk * p.k_sh;
  const float* vp = (const float*)p.v + b * p.v_sb + hk * p.v_sh;
  const int S = p.kv_lens ? min(p.S, max(p.kv_lens[b], 0)) : p.S;  // keys of this batch that take part
  int nt = (S + BT - 1) / BT;
  if (p.causal) nt = min(nt, (min(q0 + BM, p.L) - 1) / BT + 1);
  const int lim = p.causal ? min(qrow, S - 1) : S - 1;
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
  // (few rows against many keys: the key tiles are split over blockIdx.y, each part leaves its normalised
  // rows and their log-sum-exp in the workspace for fwd_f32_merge_kernel; no causal flag, no window then)
  const int split = p.split_tiles ? blockIdx.y : 0;
  int t_first = 0;
  if (!FUNC && p.split_tiles) {
    t_first = split * p.split_tiles;
    nt = max(min(nt - t_first, p.split_tiles), 0);
  }
  auto tile_of = [&](int u) { return FUNC ? u + (u >= n_lead ? skip : 0) : u + t_first; };
  const int nt_w = p.causal ? min(nt, (qw0 + 31) / BT + 1 - skip) : nt;
  TileF32<D, 64 * WAVES> kn, vn;
  auto fetch = [&](int u) {
    const int t = tile_of(u);
    kn.fetch(kp + (int64_t)t * BT * p.k_sl, p.k_sl, S - t * BT, p.d_real, tid);
    if constexpr (!kFetchAhead<D>) kn.put(k_t, tid);  // (one tile's registers serve both operands)
    auto& v_regs = kFetchAhead<D> ? vn : kn;
    v_regs.fetch(vp + (int64_t)t * BT * p.v_sl, p.v_sl, S - t * BT, p.dv_real, tid);
    if constexpr (!kFetchAhead<D>) v_regs.put(v_t, tid);
  };
  if (kFetchAhead<D> && nt > 0) fetch(0);
  for (int u = 0; u < nt; ++u) {
    __syncthreads();  // the previous tile has been read by every wavefront
    if constexpr (kFetchAhead<D>) kn.put(k_t, tid), vn.put(v_t, tid);
    else fetch(u);
    __syncthreads();
    if (kFetchAhead<D> && u + 1 < nt) fetch(u + 1);
    if (u >= nt_w) continue;
    const int t = tile_of(u);
    f32x16 s = row_product<D>(k_t, col, half, qf);
    if constexpr (FUNC) {
      // each score through the functors, s = mod(scale * s) / scale: everything downstream is the common code
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kv = t * BT + (r >> 2) * 8 + half * 4 + (r & 3);
        float dfac;
        s[r] = score_mod_at(p.sm, s[r] * p.scale, b, h, qc, min(kv, p.S - 1), p.L, p.S, dfac) * inv_scale;
        if (p.window > 0 && qrow - kv >= p.window && kv >= p.sink_keys) s[r] = -INFINITY;
      }
    }
    float keepf[MASKED ? 16 : 1];
    if constexpr (MASKED) {
      // this lane's row of the bias / keep-mask plane of the (batch, head), keys clamped into the row
      const int64_t row0 = b * p.bias_sb + h * p.bias_sh + (int64_t)qc * p.bias_sl;
      auto idx = [&](int r) { return row0 + min(t * BT + (r >> 2) * 8 + half * 4 + (r & 3), p.S - 1); };
      if (p.keep_scale != 0.f) {
        const uint8_t* krow = (const uint8_t*)p.keep + (((int64_t)b * p.Hq + h) * p.L + qc) * p.keep_ld;
#pragma unroll
        for (int r = 0; r < 16; ++r) keepf[r] = (float)krow[min(t * BT + (r >> 2) * 8 + half * 4 + (r & 3), p.S - 1)];
      }
      if (p.bias_kind) {
        float bl[16];
        load_bias16(bl, p.bias, p.bias_kind, idx);
        // folded into the raw scores, s += bias / scale: everything downstream is the unbiased code
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = fmaf(bl[r], inv_scale, s[r]);
      }
    }
    float tm = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int kv = t * BT + (r >> 2) * 8 + half * 4 + (r & 3);
      if (kv > lim) s[r] = -INFINITY;
      tm = fmaxf(tm, s[r]);
    }
    tm = fmaxf(tm, __shfl_xor(tm, 32, 64));
    const float m_new = fmaxf(m_run, tm);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row without a live key so far
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);
    m_run = m_new;
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      s[r] = __builtin_amdgcn_exp2f((s[r] - m_use) * c);
      psum += s[r];
    }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
    if constexpr (MASKED) {  // dropout: the row sum above keeps the dropped probabilities (torch_neuronx/_sdpa_math.py:36-48)
      if (p.keep_scale != 0.f) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] *= keepf[r];
      }
    }
    col_product<D>(oacc, v_t, col, half, s);
  }
  float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  float lse_row = l_tot > 0.f ? m_run * p.scale + __builtin_logf(l_tot) : -INFINITY;
  float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if constexpr (FUNC) {
    if (p.sink_logit) {
      // the sink logits of this (batch, head) join the row's softmax as one more column without a value
      // (several act as one: the logarithm of the sum of their exponentials)
      const float* zs = p.sink_logit + ((int64_t)b * p.Hq + h) * p.n_sinks;
      float zm = -INFINITY, zl = 0.f;
      for (int n = 0; n < p.n_sinks; ++n) zm = fmaxf(zm, zs[n]);
      for (int n = 0; n < p.n_sinks; ++n) zl += zm == -INFINITY ? 0.f : __expf(zs[n] - zm);
      if (zm != -INFINITY) {
        const float z = zm + __builtin_logf(zl);
        const float top = fmaxf(lse_row, z);
        const float both = __expf(lse_row - top) + __expf(z - top);  // (exp(-inf) = 0 for a row without a live key)
        inv *= __expf(lse_row - top) / both;
        lse_row = top + __builtin_logf(both);
      }
    }
  }
  if constexpr (MASKED) {
    if (p.keep_scale != 0.f) inv *= p.keep_scale;
  }
  if (qrow < p.L) {
    const int64_t prow = (((int64_t)b * p.Hq + h) * p.n_split + split) * p.L + qrow;  // (split keys: this part's row)
    const bool part = !FUNC && p.split_tiles != 0;
    float* orow = part ? p.part_o + prow * p.dv_real : (float*)p.out + b * p.o_sb + h * p.o_sh + (int64_t)qrow * p.o_sl;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = db * 32 + g * 8 + half * 4;
        if (d < p.dv_real)
          *(f32x4*)(orow + d) = f32x4{oacc[db][g * 4] * inv, oacc[db][g * 4 + 1] * inv, oacc[db][g * 4 + 2] * inv, oacc[db][g * 4 + 3] * inv};
      }
    if (part) {
      if (half == 0) p.part_lse[prow] = lse_row;
    } else if (p.lse && half == 0) {
      p.lse[((int64_t)b * p.Hq + h) * p.L + qrow] = lse_row;
    }
  }
}

// Merge of the parts of a call whose keys were split: out = sum_s w_s O_s with w_s = exp(lse_s - lse),
// lse = log sum_s exp(lse_s).  One workgroup per query row, a thread per output column (two at widths
// above 128); the parts' lse are read side by side and their weights left in LDS, the parts' rows are
// requested eight at a time.
__global__ __launch_bounds__(128) void fwd_f32_merge_kernel(FwdM p) {
  constexpr int MAXP = 512;  // (fwd_f32_plan never makes more parts)
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
    const float w = ls[i] == -INFINITY ? 0.f : __expf(ls[i] - m);  // (a part without live keys: weight 0)
    w_s[sp] = w;  // (every slot: the loop below multiplies the slots past the last part by a zero, which a stale NaN would survive)
    sum += w;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
  if (lane == 0) red_s[2 + wave] = sum;
  __syncthreads();
  sum = red_s[2] + red_s[3];
  float acc[2] = {0.f, 0.f};
  const int d = tid;
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
    if (d + 128 * i < p.dv_real)
      ((float*)p.out)[b * p.o_sb + h * p.o_sh + (int64_t)l * p.o_sl + d + 128 * i] = sum > 0.f ? acc[i] / sum : 0.f;
  if (d == 0 && p.lse) p.lse[row] = sum > 0.f ? m + __builtin_logf(sum) : -INFINITY;
}

template <int D, int WAVES, int MODE>
__global__ __launch_bounds__(64 * WAVES, 1) void bwd_f32_dq_kernel(BwdM p) {
  constexpr bool MASKED = MODE == 1, FUNC = MODE == 2;  // a per-score tensor | window, sink keys, score functors
  constexpr int DB = D / 32;
  __shared__ __attribute__((aligned(16))) float k_st[D > 128 ? 4 : BT * (D + 4)];
  __shared__ __attribute__((aligned(16))) float v_st[D > 128 ? 4 : BT * (D + 4)];
  float* const k_t = D > 128 ? wide_f32_lds : k_st;
  float* const v_t = D > 128 ? wide_f32_lds + kTileFloats<D> : v_st;
  constexpr int BM = 32 * WAVES;  // query rows per workgroup
  const int n_qt = (p.L + BM - 1) / BM;
  const int qt = n_qt - 1 - blockIdx.x / (p.B * p.Hq);
  const int bh = blockIdx.x % (p.B * p.Hq), b = bh / p.Hq, h = bh % p.Hq, hk = h / (p.Hq / p.Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 31, half = lane >> 5;
  const int q0 = qt * BM, qw0 = q0 + wave * 32, qrow = qw0 + col, qc = min(qrow, p.L - 1);
  float qf[D / 2], dof[D / 2];
  load_half_row<D>(qf, (const float*)p.q + b * p.q_sb + h * p.q_sh + (int64_t)qc * p.q_sl, half, p.d_real);
  load_half_row<D>(dof, (const float*)p.go + b * p.go_sb + h * p.go_sh + (int64_t)qc * p.go_sl, half, p.dv_real);
  float lse2, dl;
  {
    // delta = rowsum(dO * O) (torch_neuronx/_sdpa_math.py:160-163): dO is in registers already
    const float* orow = (const float*)p.out + b * p.o_sb + h * p.o_sh + (int64_t)qc * p.o_sl;
    float dsum = 0.f;
#pragma unroll
    for (int i = 0; i < D / 8; ++i) {
      const int d = half * (D / 2) + i * 4;
      if (d < p.dv_real) {
        const f32x4 o = *(const f32x4*)(orow + d);
#pragma unroll
        for (int e = 0; e < 4; ++e) dsum = fmaf(dof[i * 4 + e], o[e], dsum);
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
  f32x16 dqacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) zero(dqacc[i]);
  const float c = p.scale * kLog2eF;
  const float* kp = (const float*)p.k + b * p.k_sb + hk * p.k_sh;
  const float* vp = (const float*)p.v + b * p.v_sb + hk * p.v_sh;
  const int S = p.kv_lens ? min(p.S, max(p.kv_lens[b], 0)) : p.S;  // keys of this batch that take part
  int nt = (S + BT - 1) / BT;
  if (p.causal) nt = min(nt, (min(q0 + BM, p.L) - 1) / BT + 1);
  const int lim = p.causal ? min(qrow, S - 1) : S - 1;
  int n_lead = 0, skip = 0;  // (sliding window: the tiles that it drops whole, as in the forward)
  if constexpr (FUNC) {
    if (p.window > 0) {
      const int t_lo = max(q0 - p.window + 1, 0) / BT;
      n_lead = min(min((p.sink_keys + BT - 1) / BT, t_lo), nt);
      skip = min(t_lo, nt) - n_lead;
      nt -= skip;
    }
  }
  auto tile_of = [&](int u) { return FUNC ? u + (u >= n_lead ? skip : 0) : u; };
  const int nt_w = p.causal ? min(nt, (qw0 + 31) / BT + 1 - skip) : nt;
  // gradient of the bias: P (dP - delta) per score, this lane's row; zeros where a score takes no part
  float* const gb_row = (MASKED && p.gbias && qrow < p.L)
                            ? (float*)p.gbias + b * p.gbias_sb + h * p.gbias_sh + (int64_t)qrow * p.gbias_sl : nullptr;
  TileF32<D, 64 * WAVES> kn, vn;
  auto fetch = [&](int u) {
    const int t = tile_of(u);
    kn.fetch(kp + (int64_t)t * BT * p.k_sl, p.k_sl, S - t * BT, p.d_real, tid);
    if constexpr (!kFetchAhead<D>) kn.put(k_t, tid);  // (one tile's registers serve both operands)
    auto& v_regs = kFetchAhead<D> ? vn : kn;
    v_regs.fetch(vp + (int64_t)t * BT * p.v_sl, p.v_sl, S - t * BT, p.dv_real, tid);
    if constexpr (!kFetchAhead<D>) v_regs.put(v_t, tid);
  };
  if (kFetchAhead<D> && nt > 0) fetch(0);
  for (int u = 0; u < nt; ++u) {
    __syncthreads();  // the previous tile has been read by every wavefront
    if constexpr (kFetchAhead<D>) kn.put(k_t, tid), vn.put(v_t, tid);
    else fetch(u);
    __syncthreads();
    if (kFetchAhead<D> && u + 1 < nt) fetch(u + 1);
    if (u >= nt_w) continue;
    const int t = tile_of(u);
    f32x16 s = row_product<D>(k_t, col, half, qf);
    const f32x16 dp = row_product<D>(v_t, col, half, dof);
    f32x16 ds;
    float dfac[FUNC ? 16 : 1];  // derivative of the functors, the factor on the gradient of the scores
    if constexpr (FUNC) {
      const float inv_scale = 1.f / p.scale;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kv = t * BT + (r >> 2) * 8 + half * 4 + (r & 3);
        s[r] = score_mod_at(p.sm, s[r] * p.scale, b, h, qc, min(kv, p.S - 1), p.L, p.S, dfac[r]) * inv_scale;
        if (p.window > 0 && qrow - kv >= p.window && kv >= p.sink_keys) s[r] = -INFINITY;
      }
    }
    float bl[MASKED ? 16 : 1];  // the bias in the log2 domain
    float kpf[MASKED ? 16 : 1];  // (dropout) keep / (1 - p)
    bool drop = false;
    if constexpr (MASKED) {
      const int64_t row0 = b * p.bias_sb + h * p.bias_sh + (int64_t)qc * p.bias_sl;
      auto idx = [&](int r) { return row0 + min(t * BT + (r >> 2) * 8 + half * 4 + (r & 3), p.S - 1); };
      drop = p.keep_scale != 0.f;
      if (drop) {
        const uint8_t* krow = (const uint8_t*)p.keep + (((int64_t)b * p.Hq + h) * p.L + qc) * p.keep_ld;
#pragma unroll
        for (int r = 0; r < 16; ++r) kpf[r] = (float)krow[min(t * BT + (r >> 2) * 8 + half * 4 + (r & 3), p.S - 1)] * p.keep_scale;
      }
      if (p.bias_kind) {
        load_bias16(bl, p.bias, p.bias_kind, idx);
#pragma unroll
        for (int r = 0; r < 16; ++r) bl[r] *= kLog2eF;
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) bl[r] = 0.f;
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int kv = t * BT + (r >> 2) * 8 + half * 4 + (r & 3);
      float x = fmaf(s[r], c, -lse2);
      if constexpr (MASKED) x = fmaf(s[r], c, bl[r]) - lse2;
      const float pr = __builtin_amdgcn_exp2f(kv > lim ? -INFINITY : x);
      float g = dp[r];
      if constexpr (MASKED) g = drop ? g * kpf[r] : g;
      ds[r] = pr * (g - dl);
      if constexpr (MASKED) {
        if (gb_row && kv < p.S) gb_row[kv] = ds[r];
      }
      if constexpr (FUNC) ds[r] *= dfac[r];
    }
    col_product<D>(dqacc, k_t, col, half, ds);
  }
  if constexpr (MASKED) {
    if (gb_row) {  // the tiles this wavefront did not walk: above the diagonal, past the batch's keys
      for (int kv = min(nt_w, nt) * BT + half * 4; kv < p.S; kv += 8)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (kv + e < p.S) gb_row[kv + e] = 0.f;
    }
  }
  if (qrow < p.L) {
    float* gq = (float*)p.gq + b * p.gq_sb + h * p.gq_sh + (int64_t)qrow * p.gq_sl;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = db * 32 + g * 8 + half * 4;
        if (d < p.d_real)
          *(f32x4*)(gq + d) = f32x4{dqacc[db][g * 4] * p.scale, dqacc[db][g * 4 + 1] * p.scale, dqacc[db][g * 4 + 2] * p.scale,
                                    dqacc[db][g * 4 + 3] * p.scale};
      }
  }
}

template <int D, int WAVES, int MODE>
__global__ __launch_bounds__(64 * WAVES, 1) void bwd_f32_dkdv_kernel(BwdM p) {
  constexpr bool MASKED = MODE == 1, FUNC = MODE == 2;  // a per-score tensor | window, sink keys, score functors
  // Width 256: the K and V fragments of a key are 256 registers, so the accumulators of a workgroup
  // are half of the columns of dK and dV (128 registers) and a key block is visited by two workgroups,
  // one per half; both form every score and every dP.
  constexpr int NP = D > 128 ? 2 : 1;  // passes = workgroups per key block
  constexpr int DB = D / 32 / NP;      // 32-column blocks of dK / dV per pass
  __shared__ __attribute__((aligned(16))) float q_st[D > 128 ? 4 : BT * (D + 4)];
  __shared__ __attribute__((aligned(16))) float do_st[D > 128 ? 4 : BT * (D + 4)];
  float* const q_t = D > 128 ? wide_f32_lds : q_st;
  float* const do_t = D > 128 ? wide_f32_lds + kTileFloats<D> : do_st;
  __shared__ __attribute__((aligned(16))) float lse_s[BT];
  __shared__ __attribute__((aligned(16))) float dl_s[BT];
  const int streams = p.B * p.Hkv;
  const int pass = blockIdx.x % NP, c0 = pass * DB * 32;  // this pass's first column
  const int kt = blockIdx.x / NP / streams;  // low key tiles see the most queries under a causal mask: first
  const int st = blockIdx.x / NP % streams, b = st / p.Hkv, hk = st % p.Hkv, rep = p.Hq / p.Hkv;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 31, half = lane >> 5;
  const int k0 = kt * 32 * WAVES, kw0 = k0 + wave * 32, key = kw0 + col, kc = min(key, p.S - 1);
  const int S = p.kv_lens ? min(p.S, max(p.kv_lens[b], 0)) : p.S;  // keys of this batch that take part
  // the first query row that sees this lane's key: the key itself under a causal mask, none for a key
  // past the batch's count
  const int first_q = key >= S ? INT_MAX : p.causal ? key : INT_MIN;
  float kf[D / 2], vf[D / 2];
  load_half_row<D>(kf, (const float*)p.k + b * p.k_sb + hk * p.k_sh + (int64_t)kc * p.k_sl, half, p.d_real);
  load_half_row<D>(vf, (const float*)p.v + b * p.v_sb + hk * p.v_sh + (int64_t)kc * p.v_sl, half, p.dv_real);
  f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) zero(dkacc[i]), zero(dvacc[i]);
  const float c = p.scale * kLog2eF;
  const int nqs = (p.L + BT - 1) / BT;
  const int qs_begin = p.causal ? min(k0 / BT, nqs) : 0;
  // items: (query head of the group, 32-row query tile)
  const int per_head = nqs - qs_begin, n_items = rep * per_head;
  // (few key blocks: the items of a key block are shared out over p.parts workgroups, blockIdx.y, which
  // leave their rows in the workspace for bwd_f32_dkdv_merge_kernel)
  int it0 = 0, it1 = n_items;
  if (p.parts > 1) {
    const int chunk = (n_items + p.parts - 1) / p.parts;
    it0 = min((int)blockIdx.y * chunk, n_items), it1 = min(it0 + chunk, n_items);
  }
  TileF32<D, 64 * WAVES> qn, gn;
  float lse_n = INFINITY, dl_n = 0.f;
  auto fetch_item = [&](int it) {
    // (query tile by query tile from the last one down, heads inside: the workgroups of a kv head, which
    // share an XCD, then want the same Q / dO tile at about the same time and find it in its L2)
    const int h = hk * rep + it % rep, q0 = (nqs - 1 - it / rep) * BT;
    qn.fetch((const float*)p.q + b * p.q_sb + h * p.q_sh + (int64_t)q0 * p.q_sl, p.q_sl, p.L - q0, p.d_real, tid);
    if constexpr (!kFetchAhead<D>) qn.put(q_t, tid);  // (one tile's registers serve both operands)
    auto& g_regs = kFetchAhead<D> ? gn : qn;
    g_regs.fetch((const float*)p.go + b * p.go_sb + h * p.go_sh + (int64_t)q0 * p.go_sl, p.go_sl, p.L - q0, p.dv_real, tid);
    if constexpr (!kFetchAhead<D>) g_regs.put(do_t, tid);
    if (tid < BT) {
      const int qi = q0 + tid;
      const int64_t row = ((int64_t)b * p.Hq + h) * p.L + min(qi, p.L - 1);
      // rows past L are switched off through lse = +inf
      lse_n = qi < p.L ? p.lse2[row] : INFINITY;
      dl_n = qi < p.L ? p.delta[row] : 0.f;
    }
  };
  if (kFetchAhead<D> && it1 > it0) fetch_item(it0);
  {
    for (int it = it0; it < it1; ++it) {
      const int q0 = (nqs - 1 - it / rep) * BT;
      __syncthreads();
      if constexpr (kFetchAhead<D>) qn.put(q_t, tid), gn.put(do_t, tid);
      else fetch_item(it);
      if (tid < BT) lse_s[tid] = lse_n, dl_s[tid] = dl_n;
      __syncthreads();
      if (kFetchAhead<D> && it + 1 < it1) fetch_item(it + 1);
      if ((p.causal && q0 + BT - 1 < kw0) || kw0 >= S) continue;  // (uniform per wavefront)
      if constexpr (FUNC) {  // every row of the tile lies past the window of every key of this wavefront, none of them a sink
        if (p.window > 0 && q0 - (kw0 + 31) >= p.window && kw0 >= p.sink_keys) continue;
      }
      f32x16 s = row_product<D>(q_t, col, half, kf);
      const f32x16 dp = row_product<D>(do_t, col, half, vf);
      f32x16 pr, ds;
      float dfac[FUNC ? 16 : 1];  // derivative of the functors, the factor on the gradient of the scores
      if constexpr (FUNC) {
        const int hq = hk * rep + it % rep;
        const float inv_scale = 1.f / p.scale;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int qi = q0 + (r >> 2) * 8 + half * 4 + (r & 3);
          s[r] = score_mod_at(p.sm, s[r] * p.scale, b, hq, min(qi, p.L - 1), kc, p.L, p.S, dfac[r]) * inv_scale;
          if (p.window > 0 && qi - key >= p.window && key >= p.sink_keys) s[r] = -INFINITY;
        }
      }
      float bl[MASKED ? 16 : 1];  // the bias in the log2 domain
      float kpf[MASKED ? 16 : 1];  // (dropout) keep / (1 - p)
      bool drop = false;
      if constexpr (MASKED) {
        const int hq = hk * rep + it % rep;
        const int64_t col0 = b * p.bias_sb + hq * p.bias_sh + min(key, p.S - 1);
        auto idx = [&](int r) { return col0 + (int64_t)min(q0 + (r >> 2) * 8 + half * 4 + (r & 3), p.L - 1) * p.bias_sl; };
        drop = p.keep_scale != 0.f;
        if (drop) {
          const uint8_t* kcol = (const uint8_t*)p.keep + ((int64_t)b * p.Hq + hq) * p.L * p.keep_ld + min(key, p.S - 1);
#pragma unroll
          for (int r = 0; r < 16; ++r) kpf[r] = (float)kcol[(int64_t)min(q0 + (r >> 2) * 8 + half * 4 + (r & 3), p.L - 1) * p.keep_ld] * p.keep_scale;
        }
        if (p.bias_kind) {
          load_bias16(bl, p.bias, p.bias_kind, idx);
#pragma unroll
          for (int r = 0; r < 16; ++r) bl[r] *= kLog2eF;
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) bl[r] = 0.f;
        }
      }
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const f32x4 l4 = *(const f32x4*)(&lse_s[r4 * 8 + half * 4]);
        const f32x4 d4 = *(const f32x4*)(&dl_s[r4 * 8 + half * 4]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = r4 * 4 + e, qi = q0 + r4 * 8 + half * 4 + e;
          float a = fmaf(s[r], c, -l4[e]);
          if constexpr (MASKED) a = fmaf(s[r], c, bl[r]) - l4[e];
          const float x = __builtin_amdgcn_exp2f(qi < first_q ? -INFINITY : a);
          float g = dp[r];
          pr[r] = x;
          if constexpr (MASKED) {
            if (drop) g *= kpf[r], pr[r] = x * kpf[r];  // dV from the kept probabilities, scaled; dP masked and scaled
          }
          ds[r] = x * (g - d4[e]);
          if constexpr (FUNC) ds[r] *= dfac[r];
        }
      }
      col_product<D, DB>(dvacc, do_t + c0, col, half, pr);
      col_product<D, DB>(dkacc, q_t + c0, col, half, ds);
    }
  }
  if (key < p.S) {
    float* gk = (float*)p.gk + b * p.gk_sb + hk * p.gk_sh + (int64_t)key * p.gk_sl;
    float* gv = (float*)p.gv + b * p.gv_sb + hk * p.gv_sh + (int64_t)key * p.gv_sl;
    if (p.parts > 1) {  // (this part's rows: (part, batch, kv head, key) x real columns, every part written)
      const int64_t row = (int64_t)blockIdx.y * p.B * p.Hkv * p.S + ((int64_t)b * p.Hkv + hk) * p.S + key;
      gk = p.part_dk + row * p.d_real, gv = p.part_dv + row * p.dv_real;
    }
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = c0 + db * 32 + g * 8 + half * 4;
        if (d < p.d_real)
          *(f32x4*)(gk + d) = f32x4{dkacc[db][g * 4] * p.scale, dkacc[db][g * 4 + 1] * p.scale, dkacc[db][g * 4 + 2] * p.scale,
                                    dkacc[db][g * 4 + 3] * p.scale};
        if (d < p.dv_real)
          *(f32x4*)(gv + d) = f32x4{dvacc[db][g * 4], dvacc[db][g * 4 + 1], dvacc[db][g * 4 + 2], dvacc[db][g * 4 + 3]};
      }
  }
}

// wavefronts (32 rows each) per workgroup
int pick_waves(int64_t, int) { return 4; }

// the bias / keep-mask fields of a call: an attn_bias as it is (strides in elements), and the dropout
// keep-mask, (B, Hq, L, S) contiguous bytes with keep_scale = 1 / (1 - p) (1 for p = 1)
template <typename G, typename P>
void set_score_mask(G& g, const P& p) {
  if (p.bias.data) {
    g.bias = p.bias.data;
    g.bias_sb = p.bias.stride[0], g.bias_sh = p.bias.stride[1], g.bias_sl = p.q.size[2] > 1 ? p.bias.stride[2] : 0;
    g.bias_kind = p.bias_dtype == MI355_SDPA_F32 ? 1 : p.bias_dtype == MI355_SDPA_F16 ? 2 : p.bias_dtype == MI355_SDPA_BF16 ? 3 : 4;
  }
  if (p.dropout_p > 0.f) {
    g.keep = p.dropout_keep;
    g.keep_ld = (p.dropout_keep_ld > 0 ? p.dropout_keep_ld : p.k.size[2]);
    g.keep_scale = p.dropout_p < 1.f ? 1.f / (1.f - p.dropout_p) : 1.f;
  }
}

bool tensors_fit(const mi355_sdpa_tensor* const* ts, int n) {
  for (int k = 0; k < n; ++k) {
    const mi355_sdpa_tensor* t = ts[k];
    if (t->stride[3] != 1 || ((uintptr_t)t->data & 15) != 0) return false;
    for (int i = 0; i < 3; ++i)
      if (t->size[i] > 1 && (t->stride[i] % 4) != 0) return false;
  }
  return true;
}

}  // namespace

bool fwd_f32_mfma_supported(const mi355_sdpa_fwd_params& p, const char** why) {
  *why = "";
  const int64_t E = p.q.size[3], Dv = p.v.size[3];
  if (p.dtype != MI355_SDPA_F32) return *why = "dtype is not float32", false;
  if (E < 8 || E > 256 || E % 8 != 0 || Dv < 8 || Dv > E || Dv % 8 != 0) return *why = "head dims are not multiples of 8 up to 256 with D_v <= D_qk", false;
  if ((p.mask.window > 0 || p.mask.sink_logit || score_mod_of(p.mask).any) && (p.bias.data || p.dropout_p > 0.f))
    return *why = "window / sink / score functor together with attn_bias or dropout", false;
  if (p.bias.data && p.k.size[2] > 1 && p.bias.stride[3] != 1) return *why = "attn_bias keys are not unit-stride", false;
  if (p.bias.data && p.bias_dtype != MI355_SDPA_F32 && p.bias_dtype != MI355_SDPA_F16 && p.bias_dtype != MI355_SDPA_BF16 &&
      p.bias_dtype != MI355_SDPA_BOOL)
    return *why = "attn_bias dtype", false;
  if (!(p.scale > 0.f)) return *why = "scale <= 0", false;
  if (p.q.size[2] < 1 || p.k.size[2] < 1) return *why = "empty sequence", false;
  const mi355_sdpa_tensor* ts[4] = {&p.q, &p.k, &p.v, &p.out};
  if (!tensors_fit(ts, 4)) return *why = "rows are not unit-stride and 16-byte aligned", false;
  if (p.q.size[0] * p.q.size[1] * ((p.q.size[2] + 127) / 128) > 0x7fffffff) return *why = "too many tiles", false;
  return true;
}

namespace {

// Few query rows against many keys (a decode step in float32).  A single query row per head leaves 31 of
// a wavefront's 32 rows empty and one workgroup per head walking every key: the heads of a kv group
// become the rows of one head (they read the same K and V; a view of q, out and the log-sum-exp, nothing
// moves) where no causal flag, functor or per-head bias tells the heads apart, and where that still
// leaves compute units short of workgroups the key tiles are split over blockIdx.y, at least 4
// tiles (128 keys) per part, into the caller's workspace (fwd_f32_merge_kernel adds the parts up).
void fwd_f32_plan(FwdM& g, const mi355_sdpa_fwd_params& p, int mode) {
  g.split_tiles = 0, g.n_split = 1;
  const int rep = g.Hq / g.Hkv;
  const bool plain = !g.causal && mode != 2;
  // (several rows per head: the rows of a group's heads are one run of rows where q and out are laid
  // out head by head, row by row; a bias must then be one per key)
  const bool one_row = g.L == 1, runs = g.q_sh == (int64_t)g.L * g.q_sl && g.o_sh == (int64_t)g.L * g.o_sl;
  if (plain && rep > 1 && (int64_t)rep * g.L <= 128 && (one_row || runs) && (!g.bias || (g.bias_sh == 0 && g.bias_sl == 0))) {
    if (one_row) g.q_sl = g.q_sh, g.o_sl = g.o_sh;
    g.q_sh *= rep, g.o_sh *= rep;
    g.Hq = g.Hkv, g.L *= rep;
  }
  const int nt = (g.S + BT - 1) / BT;
  const int64_t groups = (int64_t)g.B * g.Hq;
  if (plain && g.L <= 128 && groups < 1024 && nt >= 16) {  // (up to about four workgroups per compute unit)
    const int want = (int)std::min<int64_t>(std::min<int64_t>((1024 + groups - 1) / groups, 512), nt / 4);
    if (want > 1) {
      g.split_tiles = (nt + want - 1) / want;
      g.n_split = (nt + g.split_tiles - 1) / g.split_tiles;
    }
  }
}

void fwd_f32_fill(FwdM& g, const mi355_sdpa_fwd_params& p, int& mode) {
  g.q = p.q.data, g.k = p.k.data, g.v = p.v.data, g.out = p.out.data, g.lse = p.lse;
  g.q_sb = p.q.stride[0], g.q_sh = p.q.stride[1], g.q_sl = p.q.stride[2];
  g.k_sb = p.k.stride[0], g.k_sh = p.k.stride[1], g.k_sl = p.k.stride[2];
  g.v_sb = p.v.stride[0], g.v_sh = p.v.stride[1], g.v_sl = p.v.stride[2];
  g.o_sb = p.out.stride[0], g.o_sh = p.out.stride[1], g.o_sl = p.out.stride[2];
  g.B = (int)p.q.size[0], g.Hq = (int)p.q.size[1], g.Hkv = (int)p.k.size[1];
  g.L = (int)p.q.size[2], g.S = (int)p.k.size[2];
  g.causal = p.is_causal, g.scale = p.scale, g.xcd_map = 0;
  g.kv_lens = p.kv_lens;
  g.d_real = (int)p.q.size[3], g.dv_real = (int)p.v.size[3];
  set_score_mask(g, p);
  g.window = p.mask.window, g.sink_keys = p.mask.sink_keys, g.sink_logit = p.mask.sink_logit;
  g.n_sinks = p.mask.n_sink_logits > 0 ? p.mask.n_sink_logits : 1;
  g.sm = score_mod_of(p.mask);
  mode = (g.bias != nullptr || g.keep_scale != 0.f) ? 1 : (g.window > 0 || g.sink_logit || g.sm.any) ? 2 : 0;
  fwd_f32_plan(g, p, mode);
}

}  // namespace

size_t fwd_f32_mfma_workspace(const mi355_sdpa_fwd_params& p) {
  const char* why;
  if (!fwd_f32_mfma_supported(p, &why)) return 0;
  FwdM g;
  int mode;
  fwd_f32_fill(g, p, mode);
  if (!g.split_tiles) return 0;
  return (size_t)g.B * g.Hq * g.n_split * g.L * (g.dv_real + 1) * sizeof(float);
}

int launch_fwd_f32_mfma(const mi355_sdpa_fwd_params& p, hipStream_t s) {
  const char* why;
  if (!fwd_f32_mfma_supported(p, &why)) {
    set_error("SDPA: float32 MFMA forward kernel cannot take this call: %s", why);
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  FwdM g;
  int mode;
  fwd_f32_fill(g, p, mode);
  if (g.split_tiles) {  // (the caller's workspace: too small, misaligned or absent, and the call runs unsplit)
    const size_t rows = (size_t)g.B * g.Hq * g.n_split * g.L;
    if (p.workspace && ((uintptr_t)p.workspace & 255) == 0 && g.n_split <= 512 && p.workspace_bytes >= rows * (g.dv_real + 1) * sizeof(float))
      g.part_o = (float*)p.workspace, g.part_lse = g.part_o + rows * g.dv_real;
    else
      g.split_tiles = 0, g.n_split = 1;
  }
  // rows per workgroup: 128 (a workgroup is one wavefront per 32 rows; 64- and 32-row workgroups
  // measured slower even when 128-row ones leave compute units without work)
  const int waves = pick_waves((int64_t)g.B * g.Hq, g.L);
  g.n_qt = (g.L + 32 * waves - 1) / (32 * waves);
  const dim3 grid((unsigned)((int64_t)g.B * g.Hq * g.n_qt), (unsigned)g.n_split), block(64 * waves);
  // (width 256: both tiles in the launch's dynamic LDS)
#define LAUNCH(DD, WW, MM)                                                                                       \
  do {                                                                                                           \
    constexpr int kLds = DD > 128 ? 2 * kTileFloats<DD> * (int)sizeof(float) : 0;                                \
    if (kLds) {                                                                                                  \
      static LdsOnce once;                                                                                       \
      const hipError_t e = reserve_lds(once, (const void*)fwd_f32_kernel<DD, WW, MM>, kLds);                     \
      if (e != hipSuccess) {                                                                                     \
        set_error("SDPA: cannot reserve %d bytes of LDS for fwd_f32_kernel: %s", kLds, hipGetErrorString(e));   \
        return MI355_SDPA_ERR_LAUNCH;                                                                            \
      }                                                                                                          \
    }                                                                                                            \
    hipLaunchKernelGGL((fwd_f32_kernel<DD, WW, MM>), grid, block, kLds, s, g);                                   \
  } while (0)
#define LAUNCH_W(DD)                   \
  do {                                 \
    if (mode == 1) LAUNCH(DD, 4, 1);   \
    else if (mode == 2) LAUNCH(DD, 4, 2); \
    else LAUNCH(DD, 4, 0);             \
  } while (0)
  if (g.d_real <= 64) LAUNCH_W(64);
  else if (g.d_real <= 128) LAUNCH_W(128);
  else LAUNCH_W(256);
#undef LAUNCH_W
#undef LAUNCH
  const int rc = check_launch("fwd_f32_kernel");
  if (rc != MI355_SDPA_OK || !g.split_tiles) return rc;
  hipLaunchKernelGGL(fwd_f32_merge_kernel, dim3((unsigned)((int64_t)g.B * g.Hq * g.L)), dim3(128), 0, s, g);
  return check_launch("fwd_f32_merge_kernel");
}

bool bwd_f32_mfma_supported(const mi355_sdpa_bwd_params& p, const char** why) {
  *why = "";
  const int64_t E = p.q.size[3], Dv = p.v.size[3];
  if (p.dtype != MI355_SDPA_F32) return *why = "dtype is not float32", false;
  if (E < 8 || E > 256 || E % 8 != 0 || Dv < 8 || Dv > E || Dv % 8 != 0) return *why = "head dims are not multiples of 8 up to 256 with D_v <= D_qk", false;
  if ((p.mask.window > 0 || score_mod_of(p.mask).any) && (p.bias.data || p.dropout_p > 0.f))
    return *why = "window or score functor together with attn_bias or dropout", false;
  if (p.grad_bias.data && (!p.bias.data || (p.k.size[2] > 1 && p.grad_bias.stride[3] != 1)))
    return *why = "grad_attn_bias without attn_bias, or its keys are not unit-stride", false;
  if (p.bias.data && p.k.size[2] > 1 && p.bias.stride[3] != 1) return *why = "attn_bias keys are not unit-stride", false;
  if (p.bias.data && p.bias_dtype != MI355_SDPA_F32 && p.bias_dtype != MI355_SDPA_F16 && p.bias_dtype != MI355_SDPA_BF16 &&
      p.bias_dtype != MI355_SDPA_BOOL)
    return *why = "attn_bias dtype", false;
  if (!(p.scale > 0.f)) return *why = "scale <= 0", false;
  if (p.q.size[2] < 1 || p.k.size[2] < 1) return *why = "empty sequence", false;
  const mi355_sdpa_tensor* ts[8] = {&p.grad_out, &p.q, &p.k, &p.v, &p.out, &p.grad_q, &p.grad_k, &p.grad_v};
  if (!tensors_fit(ts, 8)) return *why = "rows are not unit-stride and 16-byte aligned", false;
  if (p.q.size[0] * p.q.size[1] * ((p.q.size[2] + 127) / 128) > 0x7fffffff ||
      p.k.size[0] * p.k.size[1] * ((p.k.size[2] + 127) / 128) > 0x7fffffff)
    return *why = "too many tiles", false;
  return true;
}

namespace {

// dK and dV of a call whose key blocks were shared out over several workgroups: the sum of the parts'
// rows, one 64-thread block per key row of a (batch, kv head), four columns per thread.
__global__ __launch_bounds__(64) void bwd_f32_dkdv_merge_kernel(BwdM p) {
  const int64_t row = blockIdx.x;  // (b * Hkv + hk) * S + key
  const int key = (int)(row % p.S), hk = (int)((row / p.S) % p.Hkv), b = (int)(row / ((int64_t)p.S * p.Hkv));
  const int64_t rows = (int64_t)p.B * p.Hkv * p.S;
  for (int c = threadIdx.x * 4; c < p.d_real + p.dv_real; c += 64 * 4) {
    const bool is_v = c >= p.d_real;
    const int col = is_v ? c - p.d_real : c, width = is_v ? p.dv_real : p.d_real;
    const float* src = (is_v ? p.part_dv : p.part_dk) + row * width + col;
    f32x4 a = {0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < p.parts; ++i) a += *(const f32x4*)(src + i * rows * width);
    float* g = is_v ? (float*)p.gv + b * p.gv_sb + hk * p.gv_sh + (int64_t)key * p.gv_sl
                    : (float*)p.gk + b * p.gk_sb + hk * p.gk_sh + (int64_t)key * p.gk_sl;
    *(f32x4*)(g + col) = a;
  }
}

// Few key blocks (one or a few kv heads, a small batch, short keys) leave most compute units without a
// workgroup of the dK/dV kernel while each one walks every query head of its group: the items of a key
// block (query head x 32-row tile) are then shared out over several workgroups, at least four items
// each, about four workgroups per compute unit in all (a compute unit holds one at a time: the
// later ones even out what a causal mask leaves uneven).
int bwd_f32_parts(const mi355_sdpa_bwd_params& p) {
  const int64_t B = p.q.size[0], Hq = p.q.size[1], L = p.q.size[2], Hkv = p.k.size[1], S = p.k.size[2];
  const int64_t kgrid = B * Hkv * ((S + 127) / 128) * (p.q.size[3] > 128 ? 2 : 1);
  const int64_t items = (Hq / Hkv) * ((L + BT - 1) / BT);
  if (kgrid >= 512 || items < 8) return 1;
  return (int)std::max<int64_t>(std::min<int64_t>(std::min<int64_t>((1024 + kgrid - 1) / kgrid, items / 4), 32), 1);
}

}  // namespace

size_t bwd_f32_mfma_workspace(const mi355_sdpa_bwd_params& p) {
  size_t bytes = (size_t)(p.q.size[0] * p.q.size[1] * p.q.size[2]) * 2 * sizeof(float);  // delta and lse2
  bytes = (bytes + 255) & ~(size_t)255;
  const int parts = bwd_f32_parts(p);
  if (parts > 1)  // the parts' float32 rows of dK and dV
    bytes += (size_t)parts * p.k.size[0] * p.k.size[1] * p.k.size[2] * (p.q.size[3] + p.v.size[3]) * sizeof(float);
  return bytes;
}

int launch_bwd_f32_mfma(const mi355_sdpa_bwd_params& p, hipStream_t s) {
  const char* why;
  if (!bwd_f32_mfma_supported(p, &why)) {
    set_error("SDPA: float32 MFMA backward kernel cannot take this call: %s", why);
    return MI355_SDPA_ERR_UNSUPPORTED;
  }
  BwdM g;
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
  g.causal = p.is_causal, g.scale = p.scale, g.xcd_map = 0;
  g.kv_lens = p.kv_lens;
  g.d_real = (int)p.q.size[3], g.dv_real = (int)p.v.size[3];
  set_score_mask(g, p);
  g.window = p.mask.window, g.sink_keys = p.mask.sink_keys;
  g.sm = score_mod_of(p.mask);
  if (p.grad_bias.data) {
    g.gbias = p.grad_bias.data;
    g.gbias_sb = p.grad_bias.stride[0], g.gbias_sh = p.grad_bias.stride[1], g.gbias_sl = p.grad_bias.stride[2];
  }
  const int mode = (g.bias != nullptr || g.keep_scale != 0.f) ? 1 : (g.window > 0 || g.sm.any) ? 2 : 0;
  g.parts = bwd_f32_parts(p);
  if (g.parts > 1) {  // (the parts' rows lie behind the two row vectors, 256-byte aligned)
    const size_t head = ((size_t)(p.q.size[0] * p.q.size[1] * p.q.size[2]) * 2 * sizeof(float) + 255) & ~(size_t)255;
    if (p.workspace_bytes < bwd_f32_mfma_workspace(p)) {
      g.parts = 1;
    } else {
      g.part_dk = (float*)((char*)p.workspace + head);
      g.part_dv = g.part_dk + (size_t)g.parts * g.B * g.Hkv * g.S * g.d_real;
    }
  }
  const int qw = pick_waves((int64_t)g.B * g.Hq, g.L), kw = pick_waves((int64_t)g.B * g.Hkv, g.S);
  const dim3 qgrid((unsigned)((int64_t)g.B * g.Hq * ((g.L + 32 * qw - 1) / (32 * qw))));
  // (width 256: two workgroups per key block, one per half of the columns of dK / dV)
  const dim3 kgrid((unsigned)((int64_t)g.B * g.Hkv * ((g.S + 32 * kw - 1) / (32 * kw)) * (g.d_real > 128 ? 2 : 1)), (unsigned)g.parts);
#define LAUNCH(KK, GRID, DD, WW, MM)                                                                             \
  do {                                                                                                           \
    constexpr int kLds = DD > 128 ? 2 * kTileFloats<DD> * (int)sizeof(float) : 0;                                \
    if (kLds) {                                                                                                  \
      static LdsOnce once;                                                                                       \
      const hipError_t e = reserve_lds(once, (const void*)KK<DD, WW, MM>, kLds);                                 \
      if (e != hipSuccess) {                                                                                     \
        set_error("SDPA: cannot reserve %d bytes of LDS for " #KK ": %s", kLds, hipGetErrorString(e));          \
        return MI355_SDPA_ERR_LAUNCH;                                                                            \
      }                                                                                                          \
    }                                                                                                            \
    hipLaunchKernelGGL((KK<DD, WW, MM>), GRID, dim3(64 * WW), kLds, s, g);                                       \
  } while (0)
#define LAUNCH_W(KK, GRID, WAVES_, DD)                 \
  do {                                                 \
    if (mode == 1) LAUNCH(KK, GRID, DD, 4, 1);         \
    else if (mode == 2) LAUNCH(KK, GRID, DD, 4, 2);    \
    else LAUNCH(KK, GRID, DD, 4, 0);                   \
  } while (0)
  if (g.d_real <= 64) LAUNCH_W(bwd_f32_dq_kernel, qgrid, qw, 64);
  else if (g.d_real <= 128) LAUNCH_W(bwd_f32_dq_kernel, qgrid, qw, 128);
  else LAUNCH_W(bwd_f32_dq_kernel, qgrid, qw, 256);
  int rc = check_launch("bwd_f32_dq_kernel");
  if (rc) return rc;
  if (g.d_real <= 64) LAUNCH_W(bwd_f32_dkdv_kernel, kgrid, kw, 64);
  else if (g.d_real <= 128) LAUNCH_W(bwd_f32_dkdv_kernel, kgrid, kw, 128);
  else LAUNCH_W(bwd_f32_dkdv_kernel, kgrid, kw, 256);
#undef LAUNCH_W
#undef LAUNCH
  rc = check_launch("bwd_f32_dkdv_kernel");
  if (rc == MI355_SDPA_OK && g.parts > 1) {
    hipLaunchKernelGGL(bwd_f32_dkdv_merge_kernel, dim3((unsigned)((int64_t)g.B * g.Hkv * g.S)), dim3(64), 0, s, g);
    rc = check_launch("bwd_f32_dkdv_merge_kernel");
  }
  if (rc == MI355_SDPA_OK && p.grad_sink_logit && p.mask.sink_logit)
    rc = launch_sink_grad(p.lse, g.delta, p.mask.sink_logit, p.grad_sink_logit, (int64_t)g.B * g.Hq, g.L, p.mask.n_sink_logits, s);
  return rc;
}

}  // namespace mi355
