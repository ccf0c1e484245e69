// Element types of the score arrays (emissions, predictions) and of their gradients at the
// library's interface: fp32, as in the reference, or bf16 / fp16 for a caller whose projection
// layers produce 16-bit logits.  The kernels are written once over these helpers; all arithmetic
// stays fp32 (a 16-bit score converts exactly), only the loads and the final stores differ.
#pragma once

#include <hip/hip_runtime.h>

namespace rnnt {

struct bf16_t {
  unsigned short bits;
};

__device__ inline float bf16_to_float(unsigned short b) {
  return __uint_as_float((unsigned)b << 16);
}
// round to nearest even (one v_cvt_pk_bf16_f32)
__device__ inline unsigned short float_to_bf16(float v) {
  return __builtin_bit_cast(unsigned short, (__bf16)v);
}

struct f16_t {
  unsigned short bits;
};
__device__ inline float f16_to_float(unsigned short b) {
  return (float)__builtin_bit_cast(_Float16, b);
}
// round to nearest even (v_cvt_f16_f32); values past 65504 become infinity
__device__ inline unsigned short float_to_f16(float v) {
  return __builtin_bit_cast(unsigned short, (_Float16)v);
}

__device__ inline float ldf(const float* p) { return *p; }
__device__ inline float ldf(const f16_t* p) { return f16_to_float(p->bits); }
__device__ inline void stf(f16_t* p, float v) { p->bits = float_to_f16(v); }
__device__ inline float ldf(const bf16_t* p) { return bf16_to_float(p->bits); }
__device__ inline void stf(float* p, float v) { *p = v; }
__device__ inline void stf(bf16_t* p, float v) { p->bits = float_to_bf16(v); }

// Four consecutive, naturally aligned elements (16 bytes of fp32, 8 of bf16).
__device__ inline float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ inline float4 widen4(uint2 w, const bf16_t*) {
  return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u),
                     __uint_as_float(w.y << 16), __uint_as_float(w.y & 0xffff0000u));
}
__device__ inline float4 widen4(uint2 w, const f16_t*) {
  return make_float4(f16_to_float((unsigned short)(w.x & 0xffffu)),
                     f16_to_float((unsigned short)(w.x >> 16)),
                     f16_to_float((unsigned short)(w.y & 0xffffu)),
                     f16_to_float((unsigned short)(w.y >> 16)));
}
__device__ inline float4 load4(const bf16_t* p) {
  return widen4(*reinterpret_cast<const uint2*>(p), p);
}
__device__ inline float4 load4(const f16_t* p) {
  return widen4(*reinterpret_cast<const uint2*>(p), p);
}
__device__ inline float4 widen4(float4 x, const float*) { return x; }
// The same four elements as the load returns them (widen4 makes floats of them), for data that
// a kernel reads once: the load says so, and L2 keeps its lines for what the kernel's
// workgroups share.  Keeping the bits as they are leaves the load's wait to their first use.
__device__ inline float4 load4_bits_once(const float* p) {
  typedef float vec4 __attribute__((ext_vector_type(4)));
  const vec4 x = __builtin_nontemporal_load(reinterpret_cast<const vec4*>(p));
  return make_float4(x.x, x.y, x.z, x.w);
}
template <typename T16>
__device__ inline uint2 load4_bits_once(const T16* p) {
  typedef unsigned vec2 __attribute__((ext_vector_type(2)));
  const vec2 w = __builtin_nontemporal_load(reinterpret_cast<const vec2*>(p));
  return make_uint2(w.x, w.y);
}

// Wide loads at the element type's own alignment (global memory serves them at any such
// address): for rows whose length or start does not allow the naturally aligned ones.
typedef float float4_align4 __attribute__((ext_vector_type(4), aligned(4)));
typedef unsigned uint4_align2 __attribute__((ext_vector_type(4), aligned(2)));
typedef unsigned uint2_align2 __attribute__((ext_vector_type(2), aligned(2)));

// Elements v .. v+3 of a row of V elements at any alignment: one wide load when all four lie
// inside the row, else one by one with the index clamped to the row's last element.
__device__ inline float4 load4_any(const float* row, int v, int V) {
  if (v + 4 <= V) {
    const float4_align4 a = *reinterpret_cast<const float4_align4*>(row + v);
    return make_float4(a.x, a.y, a.z, a.w);
  }
  return make_float4(row[min(v, V - 1)], row[min(v + 1, V - 1)], row[min(v + 2, V - 1)],
                     row[min(v + 3, V - 1)]);
}
template <typename T16>
__device__ inline uint2 load4_any_bits(const T16* row, int v, int V) {
  if (v + 4 <= V) {
    const uint2_align2 a = *reinterpret_cast<const uint2_align2*>(row + v);
    return make_uint2(a.x, a.y);
  }
  return make_uint2(
      (unsigned)row[min(v, V - 1)].bits | ((unsigned)row[min(v + 1, V - 1)].bits << 16),
      (unsigned)row[min(v + 2, V - 1)].bits | ((unsigned)row[min(v + 3, V - 1)].bits << 16));
}
__device__ inline float4 load4_any_bits(const float* row, int v, int V) {
  return load4_any(row, v, V);
}
__device__ inline float4 load4_any(const bf16_t* row, int v, int V) {
  return widen4(load4_any_bits(row, v, V), row);
}
__device__ inline float4 load4_any(const f16_t* row, int v, int V) {
  return widen4(load4_any_bits(row, v, V), row);
}

// Eight consecutive elements of a row as they sit in registers after the load.
template <typename T>
struct Raw8;
template <>
struct Raw8<float> {
  float4 lo, hi;
};
template <>
struct Raw8<bf16_t> {
  uint4 w;
};
template <>
struct Raw8<f16_t> {
  uint4 w;
};

// Elements v .. v+7 of `row`, with the start clamped so that the load stays inside a row of V
// elements: fp32 rows (V % 4 == 0) clamp each group of four to the last group, bf16 rows
// (V % 8 == 0) the whole eight to the last eight.  Both are 16-byte loads.
__device__ inline Raw8<float> load8(const float* row, int v, int V) {
  Raw8<float> r;
  r.lo = *reinterpret_cast<const float4*>(row + min(v, V - 4));
  r.hi = *reinterpret_cast<const float4*>(row + min(v + 4, V - 4));
  return r;
}
__device__ inline Raw8<bf16_t> load8(const bf16_t* row, int v, int V) {
  Raw8<bf16_t> r;
  r.w = *reinterpret_cast<const uint4*>(row + min(v, V - 8));
  return r;
}

__device__ inline Raw8<f16_t> load8(const f16_t* row, int v, int V) {
  Raw8<f16_t> r;
  r.w = *reinterpret_cast<const uint4*>(row + min(v, V - 8));
  return r;
}
__device__ inline void expand(const Raw8<f16_t>& r, float (&e)[8]) {
  const unsigned w[4] = {r.w.x, r.w.y, r.w.z, r.w.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    e[2 * i] = f16_to_float((unsigned short)(w[i] & 0xffffu));
    e[2 * i + 1] = f16_to_float((unsigned short)(w[i] >> 16));
  }
}

__device__ inline void expand(const Raw8<float>& r, float (&e)[8]) {
  e[0] = r.lo.x; e[1] = r.lo.y; e[2] = r.lo.z; e[3] = r.lo.w;
  e[4] = r.hi.x; e[5] = r.hi.y; e[6] = r.hi.z; e[7] = r.hi.w;
}
__device__ inline void expand(const Raw8<bf16_t>& r, float (&e)[8]) {
  e[0] = __uint_as_float(r.w.x << 16); e[1] = __uint_as_float(r.w.x & 0xffff0000u);
  e[2] = __uint_as_float(r.w.y << 16); e[3] = __uint_as_float(r.w.y & 0xffff0000u);
  e[4] = __uint_as_float(r.w.z << 16); e[5] = __uint_as_float(r.w.z & 0xffff0000u);
  e[6] = __uint_as_float(r.w.w << 16); e[7] = __uint_as_float(r.w.w & 0xffff0000u);
}

// The same eight elements of a row whose length or start does not allow aligned 16-byte loads
// (a vocabulary that is not a multiple of the vector width, an unaligned array).  Eight that lie
// inside the row come in as loads of the same width at the element type's own alignment, which
// global memory serves; the row's last, partial eight are fetched one by one, each index clamped
// to the row's last element.
__device__ inline Raw8<float> load8_any(const float* row, int v, int V) {
  Raw8<float> r;
  if (v + 8 <= V) {
    const float4_align4 a = *reinterpret_cast<const float4_align4*>(row + v);
    const float4_align4 b = *reinterpret_cast<const float4_align4*>(row + v + 4);
    r.lo = make_float4(a.x, a.y, a.z, a.w);
    r.hi = make_float4(b.x, b.y, b.z, b.w);
    return r;
  }
  r.lo = make_float4(row[min(v, V - 1)], row[min(v + 1, V - 1)], row[min(v + 2, V - 1)],
                     row[min(v + 3, V - 1)]);
  r.hi = make_float4(row[min(v + 4, V - 1)], row[min(v + 5, V - 1)], row[min(v + 6, V - 1)],
                     row[min(v + 7, V - 1)]);
  return r;
}
template <typename T16>
__device__ inline uint4 load8_any_bits(const T16* row, int v, int V) {
  if (v + 8 <= V) {
    const uint4_align2 a = *reinterpret_cast<const uint4_align2*>(row + v);
    return make_uint4(a.x, a.y, a.z, a.w);
  }
  unsigned w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = (unsigned)row[min(v + 2 * i, V - 1)].bits |
           ((unsigned)row[min(v + 2 * i + 1, V - 1)].bits << 16);
  return make_uint4(w[0], w[1], w[2], w[3]);
}
__device__ inline Raw8<bf16_t> load8_any(const bf16_t* row, int v, int V) {
  Raw8<bf16_t> r;
  r.w = load8_any_bits(row, v, V);
  return r;
}
__device__ inline Raw8<f16_t> load8_any(const f16_t* row, int v, int V) {
  Raw8<f16_t> r;
  r.w = load8_any_bits(row, v, V);
  return r;
}

// Vector width (elements) that makes a row start 16-byte aligned.
template <typename T>
struct RowAlign;
template <>
struct RowAlign<float> {
  static constexpr int kElems = 4;
};
template <>
struct RowAlign<bf16_t> {
  static constexpr int kElems = 8;
};
template <>
struct RowAlign<f16_t> {
  static constexpr int kElems = 8;
};

}  // namespace rnnt
