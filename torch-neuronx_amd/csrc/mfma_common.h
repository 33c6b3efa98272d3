// Building blocks shared by the MFMA attention kernels (gfx950, 32x32x16 bf16/f16 MFMA).
//
// Operand convention used everywhere: a lane supplies 8 consecutive contraction elements of
// row/column (lane % 32), taken from offset 8*(lane / 32) of each 16-wide contraction step.
// In the 32x32 float32 accumulator, register r of a lane is row 8*(r/4) + 4*(lane/32) + r%4
// and column lane % 32.  Because A and B use the same lane->contraction mapping, the
// accumulator registers of one product, packed pairwise to 16 bit, ARE the B (or A) operand
// of a following product that contracts over that product's rows - as long as the other
// operand presents the rows in the order 8*(r/4) + 4*half + r%4.  Transposed LDS tiles below
// are stored in that order.
#pragma once

#include "common.h"

namespace mi355 {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr float kLog2eF = 1.4426950408889634f;

// A pointer that is the same in every lane, said so to the compiler (which otherwise wraps every
// buffer access built on it in a loop over the distinct values it might hold).
__device__ __forceinline__ void* uniform_ptr(const void* p) {
  const uint64_t a = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return (void*)(((uint64_t)hi << 32) | lo);
}

template <typename T>
struct Mma;
template <>
struct Mma<bf16_t> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) __bf16 v2;
    v2 r = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, r);
  }
  static __device__ __forceinline__ float unpack(uint32_t w, int hi) {  // element 0 or 1 of a packed pair
    return __builtin_bit_cast(float, hi ? (w & 0xffff0000u) : (w << 16));
  }
};
template <>
struct Mma<f16_t> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) _Float16 v2;
    v2 r = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, r);
  }
  static __device__ __forceinline__ float unpack(uint32_t w, int hi) {
    typedef __attribute__((ext_vector_type(2))) _Float16 v2;
    const v2 r = __builtin_bit_cast(v2, w);
    return (float)(hi ? r[1] : r[0]);
  }
};

// A matrix op whose result lands in ordinary vector registers.  The compiler picks one register
// class for the results of ALL matrix ops of a kernel, and in the attention kernels it must be the
// accumulation registers (the output accumulators alone fill half of the file); but every element
// of a score tile is consumed by the vector unit, which cannot read accumulation registers, so
// leaving score tiles there costs one copy instruction per element per tile.  Written as inline assembly the op is opaque to the
// compiler's hazard tracking: the caller owes kMfmaToValuNops idle cycles between the last op
// of a chain and the first vector instruction that touches its result (mfma_to_valu_gap).
template <typename T>
struct MmaV;
template <>
struct MmaV<bf16_t> {
  static __device__ __forceinline__ void first(f32x16& d, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void next(f32x16& d, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(b));
  }
  // B operand read from accumulation registers (a long-lived fragment parked there)
  static __device__ __forceinline__ void first_ba(f32x16& d, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
  }
  static __device__ __forceinline__ void next_ba(f32x16& d, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
  }
};
template <>
struct MmaV<f16_t> {
  static __device__ __forceinline__ void first(f32x16& d, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void next(f32x16& d, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void first_ba(f32x16& d, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
  }
  static __device__ __forceinline__ void next_ba(f32x16& d, const u32x4& a, const u32x4& b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
  }
};
// idle cycles after an 8-pass matrix op before the vector unit may touch its result (the
// architecture asks for 11; the margin is free).  The accumulators are operands of the statement:
// the matrix ops that write them are inline assembly, whose hazard the compiler does not know, so
// nothing else would keep it from placing a read of an accumulator between the last op and the idle
// cycles.
__device__ __forceinline__ void mfma_to_valu_gap(f32x16& a, f32x16& b) {
  asm volatile("s_nop 15\n\ts_nop 7" : "+v"(a), "+v"(b) :: "memory");
}
__device__ __forceinline__ void mfma_to_valu_gap(f32x16& a, f32x16& b, f32x16& c, f32x16& d) {
  asm volatile("s_nop 15\n\ts_nop 7" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) :: "memory");
}

__device__ __forceinline__ void zero(f32x16& a) {
#pragma unroll
  for (int r = 0; r < 16; ++r) a[r] = 0.f;
}

// ---- row-major tile, XOR-swizzled instead of padded ------------------------------------------
// A row is D 16-bit elements = D/8 chunks of 16 bytes.  Chunk c of row r lives at chunk
// c ^ swz(r).  swz is a bijection of the low three row bits for fixed high bits (eight
// consecutive rows reading the same chunk hit eight different 16-byte slots) and also of row
// bits 2..4 for fixed bits 0..1 (writers that own rows 4g+i hit different slots too).
__device__ __forceinline__ int swz(int r) {
  return (r & 4) | ((((r >> 1) ^ (r >> 4)) & 1) << 1) | ((r ^ (r >> 3)) & 1);
}
template <int D>
__device__ __forceinline__ int rm_off(int r, int chunk) {  // element offset in a row-major tile
  return r * D + ((chunk ^ swz(r)) << 3);
}

// ---- transposed tile: [d][row], rows in groups of four ------------------------------------------
// Within every 16 rows the 4-row groups are stored in the order 0,2,1,3, so the eight rows a
// lane needs for one contraction step (4*half .. +3 and 8 + 4*half .. +3) are one 16-byte read.
__device__ __forceinline__ int tr_pos(int g) {  // g = row / 4 -> position in 4-row units
  return (g & ~3) | ((g & 1) << 1) | ((g >> 1) & 1);
}
// rows[i][c] = dword c (two consecutive d) of row 4g+i; writes d = d0 .. d0+7 for 4 rows
template <int PITCH>
__device__ __forceinline__ void tr_store(uint16_t* tile, const u32x4 rows[4], int g, int d0) {
  const int pos = tr_pos(g) * 4;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const uint32_t a0 = rows[0][c], a1 = rows[1][c], a2 = rows[2][c], a3 = rows[3][c];
    u32x2 even, odd;
    even[0] = __builtin_amdgcn_perm(a1, a0, 0x05040100);
    even[1] = __builtin_amdgcn_perm(a3, a2, 0x05040100);
    odd[0] = __builtin_amdgcn_perm(a1, a0, 0x07060302);
    odd[1] = __builtin_amdgcn_perm(a3, a2, 0x07060302);
    *(u32x2*)(&tile[(d0 + 2 * c) * PITCH + pos]) = even;
    *(u32x2*)(&tile[(d0 + 2 * c + 1) * PITCH + pos]) = odd;
  }
}

// Swizzle of the row-major LDS tiles of the two-wavefronts-per-SIMD kernels.  A tile row is D/8
// chunks of 16 bytes; chunk c of row r lives at chunk c ^ tile_swz<D>(r).  Both ways of reading a
// tile are then free of bank conflicts: 16 consecutive rows reading the same chunk (row-major A
// operand) land in 16 different 16-byte slots of the 256-byte bank window, and 4 consecutive
// rows reading the same 4 consecutive chunks (one transposing read) land in 4 different 64-byte
// windows.  (With D = 64 two rows share a bank window, so the row parity does part of the job;
// with D = 256 a row is two windows, and the swizzle stays inside each.)
template <int D>
__device__ __forceinline__ int tile_swz(int r) {
  return D >= 128 ? (((r & 3) << 2) | ((r >> 2) & 3)) : ((((r >> 1) & 1) << 2) | ((r >> 2) & 3));
}

}  // namespace mi355
