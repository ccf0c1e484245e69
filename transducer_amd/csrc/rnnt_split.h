// fp32-accurate products on the bf16 matrix cores of gfx950.
//
// On this part v_mfma_f32_32x32x2_f32 runs at 64 flop/cycle/SIMD and blocks the SIMD's vector
// issue while it runs; v_mfma_f32_32x32x16_bf16 runs at 1024 flop/cycle/SIMD and executes beside
// vector instructions.  An fp32 value splits EXACTLY into three bf16 pieces (8 + 8 + 8 significant
// bits, by truncation): x = xh + xm + xl.  A product x*y is then the sum of nine piece products,
// each exact in fp32; the six of order <= 2^-14 are kept (hh, hm, mh, hl, mm, lh), the dropped
// three are below 2^-21 of x*y.  Six bf16 instructions replace sixteen-passes-worth of fp32 ones
// at 3/8 of the time, accumulate in fp32 like them, and leave the vector ALUs free for the
// exponentials.  For non-negative operands the dropped terms are non-negative: a sum comes out
// low by about 2^-22 relative (a quarter of an fp32 ulp of the log-normaliser).
#pragma once

#include <hip/hip_runtime.h>

namespace rnnt {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// Eight consecutive k of one operand row/column: the three bf16 pieces, as the instruction
// wants them (four 32-bit registers of two bf16 each per piece).
struct Frag3 {
  uint4 h, m, l;
};

// Two fp32 values -> one 32-bit register per piece holding {piece(x0), piece(x1)}.
__device__ inline void split_pair(float x0, float x1, unsigned& h, unsigned& m, unsigned& l) {
  constexpr unsigned kTop = 0xFFFF0000u, kSel = 0x07060302u;  // perm: upper halves of (x1, x0)
  const float r0 = x0 - __uint_as_float(__float_as_uint(x0) & kTop);
  const float r1 = x1 - __uint_as_float(__float_as_uint(x1) & kTop);
  const float q0 = r0 - __uint_as_float(__float_as_uint(r0) & kTop);
  const float q1 = r1 - __uint_as_float(__float_as_uint(r1) & kTop);
  h = __builtin_amdgcn_perm(__float_as_uint(x1), __float_as_uint(x0), kSel);
  m = __builtin_amdgcn_perm(__float_as_uint(r1), __float_as_uint(r0), kSel);
  l = __builtin_amdgcn_perm(__float_as_uint(q1), __float_as_uint(q0), kSel);
}

__device__ inline Frag3 split8(const float (&x)[8]) {
  Frag3 f;
  split_pair(x[0], x[1], f.h.x, f.m.x, f.l.x);
  split_pair(x[2], x[3], f.h.y, f.m.y, f.l.y);
  split_pair(x[4], x[5], f.h.z, f.m.z, f.l.z);
  split_pair(x[6], x[7], f.h.w, f.m.w, f.l.w);
  return f;
}

__device__ inline bf16x8 as_bf16x8(const uint4& v) { return __builtin_bit_cast(bf16x8, v); }

__device__ inline floatx16 mfma_bf16(const uint4& a, const uint4& b, const floatx16& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(a), as_bf16x8(b), c, 0, 0, 0);
}

}  // namespace rnnt
