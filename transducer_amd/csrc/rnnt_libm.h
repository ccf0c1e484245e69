// expf and log1pf with the bits of the C library the reference's CPU backend links against.
//
// The reference's lattice recursions call std::exp and std::log1p on floats
// (transducer/transducer_cpu.cpp:16-24, 124-135), i.e. glibc's expf and log1pf.  At T = 2000 the
// alphas reach 1e4, where one fp32 spacing is 1e-3: an alpha that rounds the other way changes
// the transition weights exp(alpha + e + p - LN - alpha') around it by 1e-3 relative, ten times
// the tolerance of the gradients.  Hardware exp/log (one ulp off in a few percent of calls) flip
// 0.1-0.5 % of the alphas of such a lattice, and a few thousandths of a percent of the gradient
// entries leave the tolerance although nothing is wrong with either side.  So the two functions
// are restated here operation for operation, from the published algorithms of glibc 2.35:
//
//   expf    sysdeps/ieee754/flt-32/e_expf.c with exp2f_data.c (N = 32): x*N/ln2 = k + r in
//           double, 2^(k/N) from a 32-entry table, a cubic in r, one rounding to float.  x86-64
//           selects the build of that file made with fused multiply-adds (ifunc, __expf_fma),
//           where the compiler fuses k's and r's products as well; this is that variant.
//   log1pf  sysdeps/ieee754/flt-32/s_log1pf.c (the fdlibm algorithm in float arithmetic, no
//           fused operations): k and f with 1 + x = 2^k (1 + f), s = f / (2 + f), a degree-7
//           polynomial in s^2 evaluated by Horner's rule, each product and sum rounded.
//
// Every operation below is an IEEE operation with one correct rounding (v_fma_f64, v_mul_f64,
// v_add_f32, the correctly rounded float division), so the results are the library's bit for bit:
// checked on the host over all 2.2e9 floats in [-104.5, 2] (expf) and all 1.07e9 floats in
// [0, 1.5] (log1pf) against the library, and on the device by the tests.  This file must be
// compiled with -ffp-contract=off.
#pragma once

#include <hip/hip_runtime.h>

namespace rnnt {

// bits of 2^(i/32), i = 0..31, less i << 47 (exp2f_data.c: the subtraction lets `k << 47` add the
// exponent and take the table index out again in one go)
__device__ static const unsigned long long kExp2Table[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};

// Copies the table into LDS (`tab`: 32 entries); the caller synchronises before the first use.
// A lane's index depends on its argument, and LDS answers such a read in a fraction of the time
// a global load takes.
__device__ inline void exp2_table_to_lds(unsigned long long* tab) {
  if (threadIdx.x < 32) tab[threadIdx.x] = kExp2Table[threadIdx.x];
}

// The body of expf: every argument that is neither NaN nor beyond the early returns of
// e_expf.c goes through these operations.
__device__ inline float expf_glibc_core(float x, const unsigned long long* tab) {
  constexpr double kN = 32.0;
  constexpr double kInvLn2N = 0x1.71547652b82fep+0 * kN;
  constexpr double kShift = 0x1.8p+52;
  constexpr double kC0 = 0x1.c6af84b912394p-5 / kN / kN / kN;
  constexpr double kC1 = 0x1.ebfce50fac4f3p-3 / kN / kN;
  constexpr double kC2 = 0x1.62e42ff0c52d6p-1 / kN;
  const double xd = (double)x;
  double kd = __builtin_fma(kInvLn2N, xd, kShift);  // k in the low bits of the sum
  const unsigned long long ki = (unsigned long long)__double_as_longlong(kd);
  kd -= kShift;
  const double r = __builtin_fma(kInvLn2N, xd, -kd);
  const unsigned long long t = tab[ki & 31] + (ki << 47);
  const double s = __longlong_as_double((long long)t);
  const double z = __builtin_fma(kC0, r, kC1);
  const double r2 = r * r;
  double y = __builtin_fma(kC2, r, 1.0);
  y = __builtin_fma(z, r2, y);
  y = y * s;
  return (float)y;
}

// expf for x <= 0 (or NaN): what the log-sum-exp of the recursions needs.  NaN passes through
// the arithmetic as NaN.
__device__ inline float expf_glibc_nonpositive(float x, const unsigned long long* tab) {
  const float out = expf_glibc_core(x, tab);
  return (x < -0x1.9fe368p6f) ? 0.0f : out;  // below log(2^-150), -inf included
}

// glibc 2.35 expf, fused variant.  `tab`: the table above, in LDS.
__device__ inline float expf_glibc(float x, const unsigned long long* tab) {
  float out = expf_glibc_core(x, tab);
  // |x| >= 88 (e_expf.c: the early returns; between them the formula above applies, with a
  // subnormal or infinite result from the final rounding)
  out = (x < -0x1.9fe368p6f) ? 0.0f : out;                  // below log(2^-150), -inf included
  out = (x > 0x1.62e42ep6f) ? __builtin_huge_valf() : out;  // above log(2^128)
  out = (x != x) ? x + x : out;
  return out;
}

// a / b with one correct rounding, for operands whose quotient, reciprocal and residuals are
// normal numbers (no scaling, no fix-up of special values): the hardware reciprocal refined by
// one Newton step, the quotient by two residual corrections, all fused -- the sequence the
// compiler emits for a float division, less the range handling the callers below do not need.
__device__ inline float div_rn_normal(float a, float b) {
  float y = __builtin_amdgcn_rcpf(b);
  const float e = __builtin_fmaf(-b, y, 1.0f);
  y = __builtin_fmaf(e, y, y);
  float q = a * y;
  float r = __builtin_fmaf(-b, q, a);
  q = __builtin_fmaf(r, y, q);
  r = __builtin_fmaf(-b, q, a);
  return __builtin_fmaf(r, y, q);
}

// glibc 2.35 log1pf for 0 <= x <= 1 (and NaN, which comes back as NaN).  The recursions only
// feed it exp(-|a - b|), which lies in [0, 1]; the branches for other arguments are not
// restated.  A wavefront issues one instruction at a time, so what counts on the recursion's
// dependent chain is the number of instructions; three observations keep it down, each leaving
// the library's bits untouched (the tests sweep the whole of [0, 1]):
//   * the two regimes of the algorithm (x below or above sqrt(2) - 1) share one closing formula:
//         k ln2_hi - ((hfsq - (s (hfsq + R) + (k ln2_lo + c))) - f)
//     with k = 0 and c = 0 equals f - (hfsq - s (hfsq + R)) bit for bit (adding 0 and negating
//     are exact);
//   * the library's shortcut x - x^2/2 for x < 2^-29 is what that formula gives there anyway
//     (s (hfsq + R) is below a quarter of hfsq's last bit, and halving commutes with rounding);
//   * 1 + x reaches 2 only for x within 2^-24 of 1, which is inside the rare |f| < 2^-20 case, so
//     the exponent of the sum is only looked at there.
__device__ inline float log1pf_glibc(float x) {
  constexpr float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f;
  constexpr float Lp1 = 6.6666668653e-01f, Lp2 = 4.0000000596e-01f, Lp3 = 2.8571429849e-01f,
                  Lp4 = 2.2222198546e-01f, Lp5 = 1.8183572590e-01f, Lp6 = 1.5313838422e-01f,
                  Lp7 = 1.4798198640e-01f;
  const int hx = __float_as_int(x);
  // x >= sqrt(2) - 1: 1 + x = 2^k u with u in [sqrt(1/2), sqrt(2)) and k = 1 unless the sum is
  // still below sqrt(2) (or is 2: then u = 1, handled with the rare case)
  const float up = 1.0f + x;
  const int hup = __float_as_int(up);
  const float lost = x - (up - 1.0f);                           // what the sum 1 + x lost
  const int hm = hup & 0x007fffff;
  const bool low = hm < 0x3504f7;                               // u = sum; else u = sum / 2
  const float un = __int_as_float(hm | (low ? 0x3f800000 : 0x3f000000));
  const int hu = low ? hm : (0x00800000 - hm) >> 2;             // 0 only when |u - 1| < 2^-20
  const bool small = hx < 0x3ed413d7;                           // x < sqrt(2) - 1: k = 0, f = x
  const float f = small ? x : un - 1.0f;
  const bool k1 = !small && !low;                               // k == 1 (else 0)
  // c = lost / sum, and 0 where k = 0 and f = x.  The quotient is formed in every lane and
  // masked afterwards: a branch around it would cost the wavefront more than the division.
  const float c = __int_as_float(__float_as_int(div_rn_normal(lost, up)) & (small ? 0 : -1));
  const float k_hi = k1 ? ln2_hi : 0.0f, k_lo = k1 ? ln2_lo : 0.0f;  // k * ln2_hi, k * ln2_lo
  const float hfsq = (0.5f * f) * f;
  const float s = div_rn_normal(f, 2.0f + f);
  const float z = s * s;
  float R = z * Lp7;
  R = Lp6 + R; R = z * R;
  R = Lp5 + R; R = z * R;
  R = Lp4 + R; R = z * R;
  R = Lp3 + R; R = z * R;
  R = Lp2 + R; R = z * R;
  R = Lp1 + R; R = z * R;
  float out = k_hi - ((hfsq - (s * (hfsq + R) + (k_lo + c))) - f);
  if (__builtin_expect(!small && hu == 0, 0)) {  // |f| < 2^-20: x within 2^-20 of 1 (or just
                                                 // above sqrt(2) - 1); its own short formulas
    const bool two = hup >= 0x40000000;          // the sum is 2: k = 1, u = 1, f = 0
    const float c2 = two ? div_rn_normal(1.0f - (up - x), up) : c;
    const bool kk = k1 || two;
    const float kh = kk ? ln2_hi : 0.0f, kl = kk ? ln2_lo : 0.0f;
    if (f == 0.0f) {
      out = kk ? kh + (c2 + kl) : 0.0f;
    } else {
      const float R2 = hfsq * (1.0f - 0.66666666666666666f * f);
      out = kk ? kh - ((R2 - (kl + c2)) - f) : f - R2;
    }
  }
  return out;
}

}  // namespace rnnt
