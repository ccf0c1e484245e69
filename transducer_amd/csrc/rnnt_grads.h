// Constants and small helpers shared by the dense-gradient kernels (rnnt_grads.hip: the two
// separate contractions; rnnt_fused.hip: both from one walk over the frames).
#pragma once

#include <hip/hip_runtime.h>

namespace rnnt {
namespace {

constexpr float kNegInf = -__builtin_huge_valf();
constexpr float kLog2e = 1.44269504088896340736f;

// exp(e - m) for a reference m that is used for many e: m comes in already multiplied by log2(e)
// (once per frame, as the slab is staged), so an exponential is one fused multiply-add and one
// v_exp_f32 instead of a subtraction, a multiplication and the v_exp_f32.  The rounding of that
// product scales every exponential of the frame by one common factor, which the W planes carry
// the inverse of (frame_exp_correction, rnnt_internal.h).
__device__ inline float exp_minus_scaled(float e, float m_log2e) {
  return __builtin_amdgcn_exp2f(__builtin_fmaf(e, kLog2e, -m_log2e));
}


__device__ inline float f4at(const float4& v, int q) {
  return q == 0 ? v.x : (q == 1 ? v.y : (q == 2 ? v.z : v.w));
}

constexpr int kEsMaxS = 7;               // steps of 16 label positions kept in registers
constexpr int kEsPitch = 16 * kEsMaxS + 8;  // LDS row pitch of a W-slab plane in halfwords (240 B:
                                            // 16-byte reads of 8 consecutive rows spread over all banks)
constexpr int kEsPlane = 32 * kEsPitch;
constexpr int kEsPrefetch = 2;          // labels per 32-column block whose sparse terms are prefetched
constexpr int kMaxLabels = 1024;        // labels whose terms the egrads write-out can fold in

// Row of the 32x32 output block that register r of lane-half h holds.
__device__ inline int mfma_row(int r, int h) { return 8 * (r >> 2) + 4 * h + (r & 3); }

// W^T slab in LDS: three bf16 planes of 128 rows (u) x 32 frames, row pitch 40 halfwords (80 B:
// the 16-byte fragment reads of 8 consecutive rows fall into distinct bank groups).
constexpr int kPsPitch = 40;
constexpr int kPsPlane = 128 * kPsPitch;
constexpr int kPsFlush = 8;  // slabs of 32 frames between two flushes of the running sums

// Blank / label terms of the 128 rows of one tile, staged in LDS for the write-out.
struct PRowTerms {
  float gB[128], gL[128];
  int label[128];
};

}  // namespace
}  // namespace rnnt
