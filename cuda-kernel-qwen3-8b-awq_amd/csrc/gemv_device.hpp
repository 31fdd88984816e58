// Device-side pieces of the fused dequant + matrix-vector product that more than one kernel file uses: the
// block fixed point of the inputs, the exact integer block products and the in-register reductions.
#pragma once

#include "common.hpp"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// ---------------------------------------------------------------------------
// fused dequant + matrix-vector product
//
// Arithmetic (awq_canon_math.h): the 32 inputs of a block are put into block
// fixed point once per workgroup, x[t] = I[t] * c with c a power of two taken
// from the block's largest exponent and I[t] a 16-bit integer (round to nearest
// even), and a row's block value is
//     fma(-z, S, D) * (s * c),   D = sum q[t] * I[t],  S = sum I[t]
// with D and S exact integers below 2^24.  The integers are kept in LDS as
// U = I + 32768 cut into four planes of nibbles laid out like the weight
// nibbles of a dword, so that v_dot8_u32_u4 multiplies eight weights by eight
// input nibbles at once with nothing to unpack: per 8 weights four dot products
// (one per plane) and a fifth against 0x11111111 that yields sum q for the
// offset, D = sum_p 16^p dot_p - 32768 sum q: 5 instructions per 8 weights
// (13 with binary32 multiply-adds on masked nibble pairs).
// ---------------------------------------------------------------------------
struct GroupConst {
  float s;   // scale
  float zn;  // -zero_point
};

__device__ __forceinline__ GroupConst make_group(half_t s, half_t z) { return GroupConst{(float)s, -(float)z}; }

// D of one block as a float (exact): 32 weights of this lane's row against the block's 16 plane dwords in LDS
__device__ __forceinline__ float block_dot(const u32x4& w, const unsigned char* xs) {
  const uint32_t d[4] = {w.x, w.y, w.z, w.w};
  uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0, aq = 0;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const uint4 xv = *reinterpret_cast<const uint4*>(xs + 16 * c);
    a0 = __builtin_amdgcn_udot8(d[c], xv.x, a0, false);
    a1 = __builtin_amdgcn_udot8(d[c], xv.y, a1, false);
    a2 = __builtin_amdgcn_udot8(d[c], xv.z, a2, false);
    a3 = __builtin_amdgcn_udot8(d[c], xv.w, a3, false);
    aq = __builtin_amdgcn_udot8(d[c], 0x11111111u, aq, false);
  }
  const uint32_t D = a0 + (a1 << 4) + (a2 << 8) + (a3 << 12) - (aq << 15);
  return (float)(int32_t)D;
}

// the same with the block's 16 plane dwords already in registers (shared by several row groups)
__device__ __forceinline__ float block_dot_regs(const u32x4& w, const uint4 (&xv)[4]) {
  const uint32_t d[4] = {w.x, w.y, w.z, w.w};
  uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0, aq = 0;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    a0 = __builtin_amdgcn_udot8(d[c], xv[c].x, a0, false);
    a1 = __builtin_amdgcn_udot8(d[c], xv[c].y, a1, false);
    a2 = __builtin_amdgcn_udot8(d[c], xv[c].z, a2, false);
    a3 = __builtin_amdgcn_udot8(d[c], xv[c].w, a3, false);
    aq = __builtin_amdgcn_udot8(d[c], 0x11111111u, aq, false);
  }
  const uint32_t D = a0 + (a1 << 4) + (a2 << 8) + (a3 << 12) - (aq << 15);
  return (float)(int32_t)D;
}

// A launch's output vector, which the next launch reads first of all: stored through the die's L2 into memory
// (system scope) instead of left dirty in it.  The next launch's workgroups, seven eighths of them on other dies,
// then find it in memory when they ask, not behind the write-back at the end of this kernel: 1021 -> 1033 tok/s
// for the decode step.  (Nontemporal or sc0 alone: no change; the cache rows and Q stored the same way: -0.2 %.)
__device__ __forceinline__ void store_through(half_t* ptr, half_t v) {
  const uint32_t bits = __builtin_bit_cast(unsigned short, v);
  asm volatile("global_store_short %0, %1, off sc0 sc1" ::"v"(ptr), "v"(bits) : "memory");
}

// value of another lane of the same row of 16 (DPP: no LDS round trip)
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
constexpr int kDppXor1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7 - i within 8
constexpr int kDppRor4 = 0x124, kDppRor8 = 0x128;

// (half)awq_rsqrtf(v), i.e. the binary16 rounding of a correctly rounded 1/sqrt (Inference.cu:137-138), in a
// handful of instructions for almost every argument.  The hardware's reciprocal square root e is within one
// unit in the last place of 1/sqrt(v), and so is the canonical value (a correctly rounded square root, then
// a correctly rounded reciprocal); both lie between e (1 - 2^-20) and e (1 + 2^-20).  When those two bounds
// round to the same binary16 number, everything between them does, so that number is the result; otherwise
// (one argument in a few hundred, and NaNs) the canonical sequence of some forty instructions decides.  The
// argument is the same in every lane, so the branch does not diverge.
__device__ __forceinline__ half_t rsqrt_half(float v) {
  const float e = __builtin_amdgcn_rsqf(v);
  const half_t lo = (half_t)(e * 0.99999905f), hi = (half_t)(e * 1.00000095f);
  if (__builtin_bit_cast(unsigned short, lo) == __builtin_bit_cast(unsigned short, hi) && lo == lo) return lo;
  return (half_t)awq_rsqrtf(v);
}

// v(lane) + v(lane ^ 16), then that + the same of lane ^ 32: the four rows of 16 lanes added as
// (row0 + row1) + (row2 + row3) in every lane.  gfx950's lane-swap instructions exchange rows between
// two registers without the LDS round trip of a general shuffle (the waits around them are the data
// hazard slots the compiler would insert if it saw the instruction): after the first swap a holds rows
// (0,0,2,2) and b rows (1,1,3,3) of v, after the second a holds the low and b the high half of s.
__device__ __forceinline__ float sum_rows_of_16(float v) {
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  float s = a + b;
  a = s, b = s;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}

typedef unsigned short ushort2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(ushort2_t, a), __builtin_bit_cast(ushort2_t, b)));
}

// Block fixed point of 8 consecutive block-order inputs h[0..3] (binary16 pairs, one weight dword's worth);
// the four threads tid & ~3 .. + 3 hold the 32 inputs of one block (awq_block_fixed in awq_canon_math.h).
// planes: dword p holds nibble p of U = I + 32768 of element t at the bit position of weight nibble t
// ({0,16,4,20,8,24,12,28}[t]); c: the block's power of two (NaN when the block holds an infinity or a
// NaN); S: the sum of the block's 32 integers.
__device__ __forceinline__ void stage_unit8(const uint32_t h[4], u32x4& planes, float& c, float& S) {
  // the largest magnitude: binary16 magnitudes order like their bit patterns
  uint32_t mm = pk_max_u16(pk_max_u16(h[0] & 0x7fff7fffu, h[1] & 0x7fff7fffu),
                           pk_max_u16(h[2] & 0x7fff7fffu, h[3] & 0x7fff7fffu));
  mm = max(mm & 0xffffu, mm >> 16);
  mm = max(mm, dpp_u<kDppXor1>(mm));
  mm = max(mm, dpp_u<kDppXor2>(mm));
  const uint32_t e = mm >> 10;                       // largest exponent field, 0..31
  const uint32_t cbits = (max(e, 1u) + 98u) << 23;   // c = 2^(max(e,1) - 29)
  c = __builtin_bit_cast(float, e == 31u ? 0x7fc00000u : cbits);
  const float inv = __builtin_bit_cast(float, 0x7f000000u - cbits);  // 1/c
  // x/c + (1.5 * 2^23 + 32768) rounds to an integer (nearest even) whose low 16 bits are U
  const float magic = 12615680.0f;
  uint32_t P[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const half2_t x2 = as_half2(h[i]);
    const uint32_t lo = __builtin_bit_cast(uint32_t, __builtin_fmaf((float)x2.x, inv, magic));
    const uint32_t hi = __builtin_bit_cast(uint32_t, __builtin_fmaf((float)x2.y, inv, magic));
    P[i] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);  // U of element 2i | U of element 2i+1 << 16
  }
  uint32_t su = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    su = __builtin_amdgcn_udot2(__builtin_bit_cast(ushort2_t, P[i]), ushort2_t{1, 1}, su, false);
  su += dpp_u<kDppXor1>(su);
  su += dpp_u<kDppXor2>(su);
  S = (float)((int32_t)su - (32 << 15));
  // nibble planes: bytes of A hold (element 2, element 0) of plane 0 | plane 2, of the low and the high half
  const uint32_t A0 = (P[0] & 0x0f0f0f0fu) | ((P[1] << 4) & 0xf0f0f0f0u);
  const uint32_t A1 = (P[2] & 0x0f0f0f0fu) | ((P[3] << 4) & 0xf0f0f0f0u);
  const uint32_t B0 = ((P[0] >> 4) & 0x0f0f0f0fu) | (P[1] & 0xf0f0f0f0u);
  const uint32_t B1 = ((P[2] >> 4) & 0x0f0f0f0fu) | (P[3] & 0xf0f0f0f0u);
  planes.x = __builtin_amdgcn_perm(A1, A0, 0x06020400u);
  planes.y = __builtin_amdgcn_perm(B1, B0, 0x06020400u);
  planes.z = __builtin_amdgcn_perm(A1, A0, 0x07030501u);
  planes.w = __builtin_amdgcn_perm(B1, B0, 0x07030501u);
}

// ---------------------------------------------------------------------------
// The same block products on the matrix cores.  v_mfma_i32_16x16x64_i8 multiplies a 16 x 64 byte
// operand by a 64 x 16 one; lane (g = lane / 16, n = lane % 16) supplies 16 consecutive k-bytes (group g)
// of row n of the first operand and of column n of the second, and receives rows 4g..4g+3 of column n.
// A lane's four weight dwords are 16 bytes of two nibbles each, so the second operand is the weights as
// they were loaded, once masked to the low nibbles and once to the high ones: lane (q, r) supplies k-group
// q of column r.  The first operand carries the inputs: row 4q' + p is plane p of the block of lane group
// q' in k-group q' and zero elsewhere, so that the sum over all 64 k-bytes picks one block, and lane (q, r)
// receives in its own four results exactly the planes of its own block against its own row.  Planes: the
// 16-bit integers I = lo + 256 hi, lo - 128 as a signed byte (plane 0), hi as a signed byte (plane 1), and
// all ones (plane 2, sum q):  D = sum q I = C0 + 256 C1 + 128 C2.  Three instructions per 8 weights to
// unpack and two matrix instructions per 64 (block, row) pairs instead of five dot products per 8 weights;
// the integers are the same, so every result keeps its bits.
// ---------------------------------------------------------------------------
typedef int i32x4 __attribute__((ext_vector_type(4)));

// Byte planes of 8 consecutive block-order inputs (stage_unit8's arguments): the unit's dword of plane 0 and
// plane 1 of the inputs under the low nibbles (lo0, lo1) and of those under the high nibbles (hi0, hi1).
// Byte i of a weight dword holds element {0, 4, 1, 5}[i] in its low and {2, 6, 3, 7}[i] in its high nibble.
__device__ __forceinline__ void stage_unit8_bytes(const uint32_t h[4], uint32_t& lo0, uint32_t& lo1, uint32_t& hi0,
                                                  uint32_t& hi1, float& c, float& S) {
  uint32_t mm = pk_max_u16(pk_max_u16(h[0] & 0x7fff7fffu, h[1] & 0x7fff7fffu),
                           pk_max_u16(h[2] & 0x7fff7fffu, h[3] & 0x7fff7fffu));
  mm = max(mm & 0xffffu, mm >> 16);
  mm = max(mm, dpp_u<kDppXor1>(mm));
  mm = max(mm, dpp_u<kDppXor2>(mm));
  const uint32_t e = mm >> 10;
  const uint32_t cbits = (max(e, 1u) + 98u) << 23;
  c = __builtin_bit_cast(float, e == 31u ? 0x7fc00000u : cbits);
  const float inv = __builtin_bit_cast(float, 0x7f000000u - cbits);
  // x/c + 1.5 * 2^23 rounds to an integer (nearest even) whose low 16 bits are I in two's complement
  const float magic = 12582912.0f;
  uint32_t P[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const half2_t x2 = as_half2(h[i]);
    const uint32_t lo = __builtin_bit_cast(uint32_t, __builtin_fmaf((float)x2.x, inv, magic));
    const uint32_t hi = __builtin_bit_cast(uint32_t, __builtin_fmaf((float)x2.y, inv, magic));
    P[i] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);  // I of element 2i | I of element 2i+1 << 16
  }
  typedef short short2_t __attribute__((ext_vector_type(2)));
  int su = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) su = __builtin_amdgcn_sdot2(__builtin_bit_cast(short2_t, P[i]), short2_t{1, 1}, su, false);
  su += (int)dpp_u<kDppXor1>((uint32_t)su);
  su += (int)dpp_u<kDppXor2>((uint32_t)su);
  S = (float)su;
  lo0 = __builtin_amdgcn_perm(P[2], P[0], 0x06020400u) ^ 0x80808080u;  // low bytes of elements 0, 4, 1, 5, less 128
  lo1 = __builtin_amdgcn_perm(P[2], P[0], 0x07030501u);                // their high bytes
  hi0 = __builtin_amdgcn_perm(P[3], P[1], 0x06020400u) ^ 0x80808080u;  // elements 2, 6, 3, 7
  hi1 = __builtin_amdgcn_perm(P[3], P[1], 0x07030501u);
}

// The first operands of a lane for one block column of its wavefront: LDS holds per block 64 bytes,
// [plane 0 | plane 1] of the inputs under the low nibbles, then the same under the high nibbles.  blocks:
// the 64 bytes of the block of this lane's own k-group (lane / 16).
__device__ __forceinline__ void load_planes(const unsigned char* block, int lane, u32x4& a_lo, u32x4& a_hi) {
  const int row = lane & 15, p = row & 3;
  const bool mine = (row >> 2) == (lane >> 4);
  const u32x4 zero = {0u, 0u, 0u, 0u}, ones = {0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};
  a_lo = a_hi = mine && p == 2 ? ones : zero;
  if (mine && p < 2) {
    a_lo = *reinterpret_cast<const u32x4*>(block + 16 * p);
    a_hi = *reinterpret_cast<const u32x4*>(block + 32 + 16 * p);
  }
}

// D of this lane's (block, row) as a float (exact); every lane of the wavefront must be here
__device__ __forceinline__ float block_dot_mfma(const u32x4& w, const u32x4& a_lo, const u32x4& a_hi) {
  const u32x4 lo = w & 0x0f0f0f0fu, hi = (w >> 4) & 0x0f0f0f0fu;
  i32x4 acc = {0, 0, 0, 0};
  acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, a_lo), __builtin_bit_cast(i32x4, lo), acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, a_hi), __builtin_bit_cast(i32x4, hi), acc, 0, 0, 0);
  return (float)(acc.x + (acc.y << 8) + (acc.z << 7));
}

}  // namespace
