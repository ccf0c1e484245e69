// Lattice recursions of the RNN-T loss for gfx950: alpha, dalpha and the viterbi best path,
// plus the small data-movement kernels that feed them.
//
// One wavefront walks one utterance's (t,u) lattice along anti-diagonals.  Lane L owns C
// consecutive label positions u = L*C .. L*C+C-1 and, at step s, the cells (t = s-u, u).  A
// finished cell pushes two scores forward, with the reference's exact association
// (transducer/transducer_cpu.cpp:45-48, 61-69):
//     stay(t,u) = ((x + E[t,blank]) + P[u,blank]) - LN[t,u]   -> consumed by (t+1,u), same lane
//     emit(t,u) = ((x + E[t,l_u])   + P[u,l_u])   - LN[t,u]   -> consumed by (t,u+1)
// The hand-over to the next label position stays in registers inside a lane and crosses lanes
// with one DPP wave shift; there is no barrier and no memory access on the dependent chain.
// Operands are read from "skewed" planes, indexed by anti-diagonal t+u in groups of four
// (plane_at in rnnt_internal.h), so that four steps are one 16-byte load per lane and the lanes'
// loads are neighbours in memory; they are requested several groups ahead.  This file is compiled with -ffp-contract=off: the rounding
// sequence of every cell must equal the reference's.
#include <atomic>
#include <mutex>
#include <type_traits>

#include "rnnt_internal.h"
#include "rnnt_libm.h"
#include "rnnt_split.h"

namespace rnnt {

namespace {

constexpr float kNegInf = -__builtin_huge_valf();
// Label-move score handed on by a cell outside the lattice in the alpha walk: far below any
// alpha, so a log-sum-exp returns the other operand untouched -- as -inf would -- but FINITE.
// The blank-move score of such a cell is -inf; an idle lane therefore forms
// lse(kOutside, -inf) = kOutside on the fast path, never inf - inf (which only the library path
// can sort out, and an idle lane would then send its whole wavefront there at every step).
// A cell INSIDE the lattice never sees this value: its left neighbour is inside too, and the
// first column is handed -inf (below), so -inf scores of the caller propagate exactly as in
// the reference (transducer/transducer_cpu.cpp:16-24,43-60).
constexpr float kOutside = -1.0e30f;
constexpr float kPosInf = __builtin_huge_valf();

// lane L receives the value of lane L-1; lane 0 receives `fill`.
__device__ inline float wave_shr1(float x, float fill) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(x),
                                                    0x138 /* wave_shr:1 */, 0xf, 0xf, false));
}
// lane L receives the value of lane L+1; lane 63 receives `fill`.
__device__ inline float wave_shl1(float x, float fill) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(x),
                                                    0x130 /* wave_shl:1 */, 0xf, 0xf, false));
}

// exp(x) for x <= 0 and log(w) for w in [1,2] straight on the hardware transcendental units
// (v_exp_f32 / v_log_f32 work in base 2 and are good to about one ulp).  In the one place they
// are used -- log1p(exp(-|a-b|)) below -- the rounding of x*log2(e) costs at most 2.4e-8
// absolute in the result (it is largest where exp(x) is small), i.e. less than half an ulp of
// the value log 2 that the result never exceeds.
__device__ inline float exp_neg(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896341f); }
__device__ inline float log_1to2(float w) { return __builtin_amdgcn_logf(w) * 0.693147180559945309f; }

// log1p(y) for y in [0,1]:  log(1+y) with the rounding error of the sum 1+y folded back in.
// Within about one ulp of the correctly rounded value over the whole range.
__device__ inline float log1p_unit(float y) {
  const float w = 1.0f + y;
  const float lost = y - (w - 1.0f);
  return log_1to2(w) + lost * __builtin_amdgcn_rcpf(w);
}

// log1p(exp(d)) for d <= 0 on the hardware transcendental units: within a few ulp of the C
// library's value at a seventh of its instructions.
__device__ inline float softplus_fast(float d) { return log1p_unit(exp_neg(d)); }

// Bound on |softplus_fast(d) - log1pf(expf(d))| (the library's floats) as a function of the fast
// value lf: lf * (kFastRelA + kFastRelB * |d|) + 2^-125.  The first term covers the rounding of both
// evaluations (a few ulp of lf), the second the rounding of d * log2(e) ahead of v_exp_f32,
// whose effect on the result grows with |d|.  The bound is not taken from data sheets: the
// fast value is compared with the exact one for EVERY float d <= 0 (rnnt_hip_lse_bound_check,
// run by the tests on the device itself).  Measured on gfx950, in units of 2^-23 lf: at most 2.2
// for |d| <= 1.5, 3.9 up to 4, 6.8 up to 8, 0.46 (5 + 1.25 |d|) beyond; the constants leave an
// eighth on top of that everywhere.  They are what decides how often a wavefront of the alpha
// walk takes the library path (its chance per lane is bound / half the sum's spacing), so they
// are not rounder than that: with 5 and 1.25 the walk of B=32 T=2000 U=100 was a tenth slower.
constexpr float kFastRelA = 2.75f * 0x1p-23f;
constexpr float kFastRelB = 0.65f * 0x1p-23f;
// The bound for fast value lf at argument d.  The clamp keeps 0 * inf out of it at d = -inf;
// the added 2^-125 covers d below -87.3, where the library's value is a subnormal number and
// the hardware units return 0.
__device__ inline float fast_bound(float lf, float d) {
  return __builtin_fmaf(lf, __builtin_fmaf(-kFastRelB, fmaxf(d, -256.0f), kFastRelA), 0x1p-125f);
}

// transducer/transducer_cpu.cpp:16-24 with the C library's own expf and log1pf (rnnt_libm.h):
// the same bits as the reference's CPU backend for every pair of operands.
__device__ inline float lse2_libm(float a, float b, const unsigned long long* tab) {
  // One operand -inf: |a - b| = inf, expf gives 0, log1pf(0) = 0 and the sum is the other
  // operand exactly, as the reference's early returns have it; only both -inf needs a guard.
  const float hi = a > b ? a : b;
  const float r = hi + log1pf_glibc(expf_glibc_nonpositive(-fabsf(a - b), tab));
  return (hi == kNegInf) ? kNegInf : r;
}

// The same bits, mostly without the library's ~100 instructions.  What the recursion keeps is
// r = fl(hi + l) with l = log1pf(expf(d)) at most log 2, and from a few hundred steps into a
// lattice |hi| is in the thousands: the sum's spacing is then thousands of times the
// uncertainty of a fast l, so nearly every fast sum is provably the library's sum.  Per lane:
//   r = fl(hi + lf), t = lf - (r - hi): the exact remainder (hi + lf) - r whenever |hi| >= lf;
//   the library's sum rounds to the same r if |t| + bound(lf) stays below half the spacing of
//   floats on the narrower side of r (the spacing at the float just below |r|: halves when r is
//   a power of two).
// Where |hi| < lf the remainder is not exact, but then |r| < 2 lf, the half spacing is below
// 2^-23 lf and bound(lf) >= 2.75 * 2^-23 lf alone exceeds it: the test fails by itself.  r = 0, NaN
// operands and two operands of -inf (inf - inf) fail it too.  Lanes that fail take the library
// path; a wavefront skips it when none does (Ziv's strategy).  Either way the result is the
// library's, bit for bit.
__device__ inline float lse2_checked(float a, float b, const unsigned long long* tab) {
  const float hi = a > b ? a : b;
  const float d = -fabsf(a - b);
  const float lf = softplus_fast(d);
  float r = hi + lf;
  const float t = lf - (r - hi);
  const float bound = fast_bound(lf, d);
  const int below = (__float_as_int(r) - 1) & 0x7f800000;  // exponent of the float below |r|
  const float half_spacing = __int_as_float(below - (24 << 23));
  if (!(fabsf(t) + bound < half_spacing)) r = lse2_libm(a, b, tab);
  return r;
}

// The same on the hardware units alone (no check): for the chain-latency probe.
__device__ inline float lse2(float a, float b) {
  // One operand -inf: |a - b| = inf, exp gives 0, log1p(0) = 0 and the sum is the other operand
  // exactly, as the reference's early returns have it; only both -inf (inf - inf) needs a guard.
  const float hi = fmaxf(a, b);
  const float r = hi + log1p_unit(exp_neg(-fabsf(a - b)));
  return (hi == kNegInf) ? kNegInf : r;
}

// Raises the device's trouble flag.  A store to GLOBAL memory by its address space: through a
// generic pointer it would be a flat instruction, which may go to LDS as well, and with one of
// those possibly in flight the compiler waits for every load in flight at the next use of any
// loaded value -- on the walk's fast path too, where the branch that raises the flag is never
// taken.
__device__ inline void raise_trouble(int* trouble) {
  typedef __attribute__((address_space(1))) int global_int;
  __hip_atomic_store((global_int*)trouble, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The wait of an upper wavefront for the progress counter of the one below it (LDS, same
// workgroup).  The lower wavefront never waits for an upper one, so the counter always gets
// there; the trip bound only turns a logic slip of a future edit into an error report instead
// of a hung device: when it runs out the wavefront raises the device's trouble flag, stops
// waiting for good (returns a count no later `need` exceeds) and finishes its walk on whatever
// the hand-over array holds.  The host reads the flag with rnnt_hip_check_kernels().
__device__ inline int bounded_wait(const int* counter, int have, int need, int spin_limit,
                                   int* __restrict__ trouble) {
  int spins = 0;
  while (have < need) {
    have = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    asm volatile("" ::: "memory");
    if (have < need) {
      if (spins++ >= spin_limit) {
        if ((threadIdx.x & 63) == 0) raise_trouble(trouble);
        return 0x7fffffff;
      }
      __builtin_amdgcn_s_sleep(1);
    }
  }
  return have;
}

__device__ inline float f4get(const float4& v, int j) {
  return j == 0 ? v.x : (j == 1 ? v.y : (j == 2 ? v.z : v.w));
}
__device__ inline void f4set(float4& v, int j, float x) {
  if (j == 0) v.x = x; else if (j == 1) v.y = x; else if (j == 2) v.z = x; else v.w = x;
}

// ------------------------------------------------------------------ skew / unskew
// row-major [B,T,U] <-> skewed planes.  A block takes 64 label positions x 64 anti-diagonals
// (16 groups of four: 1 KB of contiguous plane memory each) and their 127 frames t = dd - u, and
// transposes through LDS so that the plane side moves 16-byte pieces next to each other and the
// row-major side rows of consecutive label positions.  Only cells inside the utterance's
// (T_b, U_b) extent are touched.  Grid: (anti-diagonal blocks, label blocks, B).
__global__ __launch_bounds__(256) void skew_kernel(const float* __restrict__ src,
                                                   float* __restrict__ dstS,
                                                   const int* __restrict__ inLen,
                                                   const int* __restrict__ labLen, Dims d) {
  __shared__ float tile[64][65];  // [label position][anti-diagonal]
  const int b = blockIdx.z, dd0 = blockIdx.x * 64, u0 = blockIdx.y * 64;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const int t_first = dd0 - u0 - 63;  // frames t_first .. t_first + 126 meet the tile
  if (u0 >= Ub || t_first >= Tb || t_first + 126 < 0) return;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const float* s = src + (size_t)b * d.T * d.U;
  // (all of a thread's 32 values are requested before the first goes to LDS: taken one by one,
  // each waited a memory round trip -- 0.45 ms for the 128 MB of B=8 T=10000 U=401)
  float v[32];
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const int r = ty + 4 * i, t = t_first + r, u = u0 + tx, c = tx + r - 63;
    const bool wanted = c >= 0 && c < 64 && t >= 0 && t < Tb && u < Ub;
    v[i] = wanted ? s[(size_t)t * d.U + u] : 0.0f;
  }
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const int c = tx + ty + 4 * i - 63;
    if (c >= 0 && c < 64) tile[tx][c] = v[i];
  }
  __syncthreads();
  const size_t plane_b = (size_t)b * d.Ua * d.Dp;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int f = k * 256 + threadIdx.x, gl = f >> 6, ul = f & 63;
    const int u = u0 + ul, g = (dd0 >> 2) + gl, tq = 4 * g - u;  // frame of the group's first cell
    if (u >= Ub || tq + 3 < 0 || tq >= Tb) continue;
    float* dst = dstS + plane_b + ((size_t)g * d.Ua + u) * 4;
    if (tq >= 0 && tq + 3 < Tb) {
      *reinterpret_cast<float4*>(dst) = make_float4(tile[ul][4 * gl], tile[ul][4 * gl + 1],
                                                    tile[ul][4 * gl + 2], tile[ul][4 * gl + 3]);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (tq + j >= 0 && tq + j < Tb) dst[j] = tile[ul][4 * gl + j];
    }
  }
}

__global__ __launch_bounds__(256) void unskew_kernel(const float* __restrict__ srcS,
                                                     float* __restrict__ dst,
                                                     const int* __restrict__ inLen,
                                                     const int* __restrict__ labLen, Dims d) {
  __shared__ float tile[64][65];  // [label position][anti-diagonal]
  const int b = blockIdx.z, dd0 = blockIdx.x * 64, u0 = blockIdx.y * 64;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const int t_first = dd0 - u0 - 63;
  if (u0 >= Ub || t_first >= Tb || t_first + 126 < 0) return;
  const size_t plane_b = (size_t)b * d.Ua * d.Dp;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int f = k * 256 + threadIdx.x, gl = f >> 6, ul = f & 63;
    const int u = u0 + ul, g = (dd0 >> 2) + gl, tq = 4 * g - u;
    float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    // (a group that holds a cell of the lattice lies inside the plane: 4g < T + U)
    if (u < Ub && tq + 3 >= 0 && tq < Tb)
      v = *reinterpret_cast<const float4*>(srcS + plane_b + ((size_t)g * d.Ua + u) * 4);
    tile[ul][4 * gl] = v.x;
    tile[ul][4 * gl + 1] = v.y;
    tile[ul][4 * gl + 2] = v.z;
    tile[ul][4 * gl + 3] = v.w;
  }
  __syncthreads();
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  float* o = dst + (size_t)b * d.T * d.U;
  for (int i = 0; i < 32; ++i) {
    const int r = ty + 4 * i, t = t_first + r, u = u0 + tx, c = tx + r - 63;
    if (c >= 0 && c < 64 && t >= 0 && t < Tb && u < Ub) o[(size_t)t * d.U + u] = tile[tx][c];
  }
}

// ------------------------------------------------------------------ gather
// elS(u, t+u) = E[t, label_u]; eb[t] = E[t, blank]; pb[u] = P[u, blank]; pl[u] = P[u, label_u].
// Tiles of 64 label positions x 64 anti-diagonals like skew_kernel (same grid), the source being
// E[t, label_u] instead of a row-major [T, U] array: a wavefront reads one frame's scores of 64
// labels (scattered over the frame's row either way), and the plane side is written as 16-byte
// pieces next to each other.  (One block per label position and 256 frames, every thread writing
// its own 4-byte cell: 0.38 ms against 0.13 at B=8 T=10000 U=401 V=32.)  The blocks of the first
// label tile also leave eb for their 64 anti-diagonals' frames, those of the first anti-diagonal
// block pb and pl for their 64 positions.
template <typename TIO>
__global__ __launch_bounds__(256) void gather_kernel(const TIO* __restrict__ E,
                                                     const TIO* __restrict__ P,
                                                     const int* __restrict__ labels,
                                                     const int* __restrict__ inLen,
                                                     const int* __restrict__ labLen, Planes p,
                                                     Dims d) {
  __shared__ float tile[64][65];  // [label position][anti-diagonal]
  const int b = blockIdx.z, dd0 = blockIdx.x * 64, u0 = blockIdx.y * 64;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  if (u0 >= Ub) return;
  const TIO* Eb = E + (size_t)b * d.T * d.V;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  if (blockIdx.y == 0 && threadIdx.x < 64) {  // frames dd0 .. dd0 + 63 (dd0 runs past T)
    const int t = dd0 + threadIdx.x;
    if (t < Tb) p.eb[(size_t)b * d.Tp + d.Eo + t] = ldf(Eb + (size_t)t * d.V + d.blank);
  }
  const int u_mine = u0 + tx;
  const bool has_label = labels != nullptr && u_mine + 1 < Ub;
  const int l = has_label ? label_at(labels, d, b, u_mine) : d.blank;
  if (blockIdx.x == 0 && ty == 0 && u_mine < Ub) {
    const TIO* Pu = P + ((size_t)b * d.U + u_mine) * d.V;
    p.pb[(size_t)b * d.Ua + u_mine] = ldf(Pu + d.blank);
    p.pl[(size_t)b * d.Ua + u_mine] = has_label ? ldf(Pu + l) : 0.0f;
  }
  const int t_first = dd0 - u0 - 63;  // frames t_first .. t_first + 126 meet the tile
  if (labels == nullptr || t_first >= Tb || t_first + 126 < 0) return;
  float v[32];
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const int r = ty + 4 * i, t = t_first + r, c = tx + r - 63;
    const bool wanted = c >= 0 && c < 64 && t >= 0 && t < Tb && has_label;
    v[i] = wanted ? ldf(Eb + (size_t)t * d.V + l) : 0.0f;
  }
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const int c = tx + ty + 4 * i - 63;
    if (c >= 0 && c < 64) tile[tx][c] = v[i];
  }
  __syncthreads();
  const size_t plane_b = (size_t)b * d.Ua * d.Dp;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int f = k * 256 + threadIdx.x, gl = f >> 6, ul = f & 63;
    const int u = u0 + ul, g = (dd0 >> 2) + gl, tq = 4 * g - u;  // frame of the group's first cell
    if (u + 1 >= Ub || tq + 3 < 0 || tq >= Tb) continue;         // (the last position has no label)
    float* dst = p.elS + plane_b + ((size_t)g * d.Ua + u) * 4;
    if (tq >= 0 && tq + 3 < Tb) {
      *reinterpret_cast<float4*>(dst) = make_float4(tile[ul][4 * gl], tile[ul][4 * gl + 1],
                                                    tile[ul][4 * gl + 2], tile[ul][4 * gl + 3]);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (tq + j >= 0 && tq + j < Tb) dst[j] = tile[ul][4 * gl + j];
    }
  }
}

// The same per cell: grid (ceil(T/256), U, B), a block serves 256 frames of one label position
// and every thread writes its own cell.  For large vocabularies, where a frame's scores of 64
// labels are 64 cache lines whichever way they are read and this form keeps more requests in
// flight (B=32 T=2000 U=101 V=10000: 0.17 ms a launch against 0.185 by tiles).
template <typename TIO>
__global__ __launch_bounds__(256) void gather_cells_kernel(const TIO* __restrict__ E,
                                                           const TIO* __restrict__ P,
                                                           const int* __restrict__ labels,
                                                           const int* __restrict__ inLen,
                                                           const int* __restrict__ labLen,
                                                           Planes p, Dims d) {
  const int b = blockIdx.z, u = blockIdx.y;
  const int t = blockIdx.x * 256 + threadIdx.x;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  if (u >= Ub) return;
  const bool has_label = labels != nullptr && (u + 1 < Ub);
  const int l = has_label ? label_at(labels, d, b, u) : d.blank;
  const TIO* Eb = E + (size_t)b * d.T * d.V;
  if (t < Tb) {
    if (has_label) p.elS[plane_at(d, b, u, t + u)] = ldf(Eb + (size_t)t * d.V + l);
    if (u == 0) p.eb[(size_t)b * d.Tp + d.Eo + t] = ldf(Eb + (size_t)t * d.V + d.blank);
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    const TIO* Pu = P + ((size_t)b * d.U + u) * d.V;
    p.pb[(size_t)b * d.Ua + u] = ldf(Pu + d.blank);
    p.pl[(size_t)b * d.Ua + u] = has_label ? ldf(Pu + l) : 0.0f;
  }
}

// ------------------------------------------------------------------ alpha
// transducer/transducer_cpu.cpp:30-79 (one utterance per wavefront).
// A cell that has not started yet (t < 0) hands on "nothing" -- -inf upwards (blank move),
// kOutside to the right (label move) -- which makes the log-sum-exp of a first-row or
// first-column cell return its one real operand untouched: exactly the reference's special
// cases (:49-60), also when that operand is -inf (both operands are then -inf and the library
// path returns -inf).  Cells past the utterance (t >= T_b, u >= U_b) hand on the same and are
// never read by a valid cell.
// W > 1: the label positions are dealt to W wavefronts of one workgroup (wavefront w owns
// positions [64 C w, 64 C (w+1))), because the walk is bound by how fast ONE wavefront issues
// the ~22 instructions of a cell: a step costs about 30 + 65 C ns.  The only value that crosses
// a wavefront boundary is the label-move score of the boundary cell, one float per step: the
// lower wavefront leaves it in an LDS array indexed by step and then publishes how far it has
// got; the upper one runs a few groups behind, so it finds its inputs there without waiting and
// re-reads the progress counter only once every few groups.  The lowest
// wavefront waits for nobody and every wavefront runs all groups, so the waits are bounded.
// A label axis longer than one workgroup's 64 C W positions is walked block by block, one launch
// per block of 64 C W positions (u_base = its first one), lowest block first.  The only values
// that cross a block boundary are the label-move scores of the block's last column, one per
// step: a launch leaves them in `ghout` ([B][hand_stride], entry s = score entering step s;
// null for the last block) and the next one reads them from `ghin` (null for the first block).
// kMulti: this launch is one of several blocks (the hand-over code is compiled in only then: in
// the single-block kernel even an unused hand-over load costs the walk its prefetch distance).
// kLive (with kMulti): the live_n blocks of 64 C W positions of a label axis run at the same
// time, as live_n workgroups on as many CUs of one XCD (with few utterances and many label
// positions one CU's wavefronts are what holds the walk).  The scores of a boundary column then
// cross in `live` (live_n - 1 arrays of [B][hand_stride] 64-bit words, zero before the launch):
// entry s is the score entering step s with s + 1 in its upper half, so that a reader can tell
// a written entry by itself -- one store, no fence, no separate counter.  A block asks for the
// entries of the block below it four groups ahead like every other operand (lane j for entry
// 4g + j), checks the tags when it comes to use them, and asks again (bounded, like the waits
// inside a workgroup) if the block below has not got there yet; it starts kLiveLag groups
// behind it, so that in the steady state what it asks for has long been written.  Workgroups
// are dispatched in launch order and a block has a smaller index than the block above it, so
// the block that is waited for is always running or done.
constexpr int kLiveLag = 12;
constexpr int kBetaLiveLag = 24;  // (the dalpha walk asks eight groups ahead, not four)
constexpr int kLiveWaveLag = 2;  // groups between the wavefronts of a live block at the start (8 elsewhere)
template <int C, int W, bool kMulti, bool kLive = false>
__global__ __launch_bounds__(64 * W) void alpha_kernel(Planes p, const int* __restrict__ inLen,
                                                       const int* __restrict__ labLen,
                                                       float* __restrict__ costs, Dims d,
                                                       int hand_stride, int spin_limit,
                                                       int* __restrict__ trouble, int u_base,
                                                       const float* __restrict__ ghin,
                                                       float* __restrict__ ghout,
                                                       unsigned long long* __restrict__ live,
                                                       int live_n) {
  static_assert(kMulti || !kLive, "live blocks are blocks");
  extern __shared__ __attribute__((aligned(16))) float hand[];  // [W-1][hand_stride]: entry s =
                                                                // score handed to step s
  __shared__ int done[W];          // steps a wavefront has published
  __shared__ unsigned long long etab[32];  // expf's table (rnnt_libm.h)
  // live blocks: workgroups go round the 8 XCDs in launch order; ids i, i + 8, i + 16 .. share
  // one, and with it the L2 the boundary scores cross in.  Eight utterances take 8 live_n
  // consecutive ids, block by block, lowest block first.
  const int live_block = kLive ? (int)(blockIdx.x >> 3) % live_n : 0;
  const int b = kLive ? (int)(blockIdx.x / (8 * live_n)) * 8 + (blockIdx.x & 7) : blockIdx.x;
  const int lane = threadIdx.x & 63;
  if (kLive) {
    if (b >= d.B) return;
    u_base = live_block * 64 * C * W;
  }
  const int wave = W > 1 ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : 0;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  if (Tb == 0 || Ub == 0) {  // :39-41
    if (threadIdx.x == 0 && u_base == 0) costs[b] = kPosInf;
    return;
  }
  if (u_base >= Ub) return;  // a block past this utterance's labels: nobody reads what it would leave
  const int nsteps = Tb + Ub - 1;
  const int ngroups = (nsteps + 3) >> 2;
  const int u0 = u_base + (wave * 64 + lane) * C;
  const int gstride = plane_group_stride(d);
  const bool first_column = u_base == 0 && wave == 0;  // lane 0 owns the lattice's column u = 0
  const float* gin = (kMulti && !kLive && ghin) ? ghin + (size_t)b * hand_stride : nullptr;
  float* gout = (kMulti && !kLive && ghout) ? ghout + (size_t)b * hand_stride : nullptr;
  if (kMulti && gout && threadIdx.x == 0) gout[0] = kOutside;  // nothing enters step 0
  // live blocks: block h reads the entries of boundary h - 1 and writes those of boundary h
  // (live_n - 1 arrays of [B][hand_stride] entries; the lowest block asks at its own boundary,
  // for nothing)
  const bool live_in = kLive && live_block > 0, live_out = kLive && live_block < live_n - 1;
  const unsigned long long* lrow =
      kLive ? live + ((size_t)max(live_block - 1, 0) * d.B + b) * hand_stride : nullptr;
  unsigned long long* lrow_out =
      kLive ? live + ((size_t)min(live_block, max(live_n - 2, 0)) * d.B + b) * hand_stride
            : nullptr;
  auto live_entry = [](int s, float x) -> unsigned long long {
    return ((unsigned long long)(unsigned)(s + 1) << 32) | (unsigned long long)__float_as_uint(x);
  };
  auto live_load = [&](int s) -> unsigned long long {
    return __hip_atomic_load(lrow + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  // Asking again for an entry that was not there yet: the load and its wait are one opaque
  // statement, so that the compiler's count of the loads in flight in the walk's main loop (the
  // operands of the next four groups) stays exact -- a loop around a load it knows of makes it
  // wait for all of them at every use.
  auto live_reload = [&](int s) -> unsigned long long {
    unsigned long long e;
    const unsigned long long* q = lrow + s;
    asm volatile("global_load_dwordx2 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)"
                 : "=&v"(e)
                 : "v"(q)
                 : "memory");
    return e;
  };
  if (live_out && threadIdx.x == 0)  // nothing enters step 0
    __hip_atomic_store(lrow_out, live_entry(0, kOutside), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  exp2_table_to_lds(etab);
  if (W > 1) {
    if (threadIdx.x < W) done[threadIdx.x] = 0;
    if (threadIdx.x < W - 1) hand[threadIdx.x * hand_stride] = kOutside;  // nothing enters step 0
  }
  __syncthreads();
  float* hand_out = hand + wave * hand_stride;                     // wave < W-1
  const float* hand_in = hand + (wave > 0 ? wave - 1 : 0) * hand_stride;  // wave > 0
  // E[t,blank] for the cells of step s sits at ebp[s - u]; column c at step s = 4g+j reads
  // ebl[4g + j - c], so one run of C+3 values serves all columns of a group
  const float* ebl = p.eb + (size_t)b * d.Tp + d.Eo - u0;

  float stay[C], emit[C], pbv[C], plv[C];
  unsigned tlim[C];  // frames of this column: T_b, or 0 for a label position past the utterance
  const float* lnp[C];
  const float* elp[C];
  float* ap[C];
#pragma unroll
  for (int c = 0; c < C; ++c) {
    tlim[c] = (u0 + c < Ub) ? (unsigned)Tb : 0u;
    const size_t row = plane_group0(d, b, u0 + c);  // u0 + c < Ua always
    lnp[c] = p.lnS + row;
    elp[c] = p.elS + row;
    ap[c] = p.aS + row;
    pbv[c] = p.pb[(size_t)b * d.Ua + u0 + c];
    plv[c] = p.pl[(size_t)b * d.Ua + u0 + c];
    // :43 alpha[0,0] = 0: cell (0,0) finds 0 coming up from below and nothing from the left
    stay[c] = (u0 + c == 0) ? 0.0f : kNegInf;
    emit[c] = kOutside;
  }

  struct Group {
    float4 ln[C], el[C];
    float eb[C + 3];
    float4 gh;  // scores entering the block's first column from the block below
    unsigned long long lv;  // the same, tagged, from the block running beside this one: lane j holds entry 4g + j
  };
  auto load_group = [&](int g) -> Group {
    Group r;
#pragma unroll
    for (int c = 0; c < C; ++c) {
      r.ln[c] = *reinterpret_cast<const float4*>(lnp[c] + (size_t)g * gstride);
      r.el[c] = *reinterpret_cast<const float4*>(elp[c] + (size_t)g * gstride);
    }
#pragma unroll
    for (int k = 0; k < C + 3; ++k) r.eb[k] = ebl[4 * g + k - (C - 1)];
    if constexpr (kMulti) {
      r.gh = make_float4(kOutside, kOutside, kOutside, kOutside);
      if (gin) r.gh = *reinterpret_cast<const float4*>(gin + 4 * g);  // uniform
      if constexpr (kLive) {
        // every wavefront of both blocks asks (only wavefront 0 of the upper block takes the
        // answer): a load under a condition would have its result copied, hence waited for,
        // right where it is asked for -- and so would a load from an address all lanes share,
        // which the compiler moves to scalar registers at once
        r.lv = live_load(4 * g + (lane & 3));
      }
    }
    return r;
  };

  unsigned live_sink = 0;
  int avail = 0;  // steps the wavefront below is known to have published
  auto wait_for = [&](int need) {
    // LDS serves a wavefront's requests in order, so no hardware fence is needed on either
    // side (a release/acquire pair would also wait for the global prefetches in flight);
    // the empty asm statements only keep the compiler from moving LDS accesses across
    avail = bounded_wait(&done[wave - 1], avail, need, spin_limit, trouble);
  };
  // kWhole: all four steps of the group exist (every group but the last; no test per step)
  auto run_group = [&](int g, const Group& cur, auto whole) {
    constexpr bool kWhole = decltype(whole)::value;
    float4 aout[C];
    // what enters the wavefront's first column from the left: for the lattice's own first
    // column (u = 0) nothing, which is -inf while its cells are inside the lattice (:49-52 adds
    // nothing there, so a -inf blank score must come out as -inf) and kOutside once they are
    // past the last frame (the idle lane's pair is then (kOutside, -inf) again)
    float4 hin;
#pragma unroll
    for (int j = 0; j < 4; ++j) f4set(hin, j, (first_column && 4 * g + j < Tb) ? kNegInf : kOutside);
    if constexpr (kMulti) {
      if (gin) hin = cur.gh;  // wavefront 0: from the block below
      if constexpr (kLive) {
        // Wavefront 0 of the upper block takes what it asked for: lanes 0 .. 3 hold the four
        // entries and check their tags.  Every other wavefront folds the answer into a word
        // that is looked at once, at the very end: a result nobody reads would have its
        // registers reused at once, and that reuse waits for the load.
        if (live_in && wave == 0) {  // uniform
          unsigned long long e = cur.lv;
          if (__builtin_amdgcn_ballot_w64(lane < 4 &&
                                          (unsigned)(e >> 32) != (unsigned)(4 * g + lane + 1))) {
            // An entry was not written when it was asked for: the lower block is closer than it
            // should be.  Let it get kLiveLag groups ahead again (or finish) before going on --
            // asking only for what is missing would leave this block right behind it, late at
            // every group.  Lanes 0 .. 3 ask for their entries again, the others for the far one.
            const int mine = lane < 4 ? 4 * g + lane : min(4 * ngroups, 4 * (g + kLiveLag));
            int spins = 0;
            do {
              if (spins++ >= spin_limit) {
                if (lane == 0) raise_trouble(trouble);
                break;
              }
              __builtin_amdgcn_s_sleep(4);
              e = live_reload(mine);
            } while (__builtin_amdgcn_ballot_w64((unsigned)(e >> 32) != (unsigned)(mine + 1)));
          }
#pragma unroll
          for (int j = 0; j < 4; ++j)
            f4set(hin, j, __int_as_float(__builtin_amdgcn_readlane((int)(unsigned)e, j)));
        } else {
          live_sink ^= (unsigned)cur.lv;
        }
      }
    }
    if (W > 1 && wave > 0) {
      wait_for(4 * g + 3);  // the scores entering steps 4g .. 4g+3 left steps 4g-1 .. 4g+2
      hin = *reinterpret_cast<const float4*>(hand_in + 4 * g);
    }
    float hout[4];
    float gsend[4];  // what this lane's last column hands to the right after each step
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = 4 * g + j;
      if constexpr (kMulti) gsend[j] = kOutside;
      if (kWhole || s < nsteps) {  // uniform; a step past the last must not touch the scores
        const float from_left = wave_shr1(emit[C - 1], f4get(hin, j));  // lane 0: hin
#pragma unroll
        for (int c = C - 1; c >= 0; --c) {
          const float left = (c == 0) ? from_left : emit[c - 1];
          const float a = lse2_checked(left, stay[c], etab);
          const float ln = f4get(cur.ln[c], j);
          float sb = a + cur.eb[j - c + (C - 1)];
          sb = sb + pbv[c];
          sb = sb - ln;
          float se = a + f4get(cur.el[c], j);
          se = se + plv[c];
          se = se - ln;
          // a cell of the lattice: 0 <= t = s - u < T_b (one unsigned comparison).  Cells before
          // the first frame or past the last one hand kOutside on, so whatever the planes hold
          // outside the utterance never enters a log-sum-exp (where it would cost the whole
          // wavefront the library path).
          const bool inside = (unsigned)(s - (u0 + c)) < tlim[c];
          stay[c] = inside ? sb : kNegInf;
          emit[c] = inside ? se : kOutside;
          f4set(aout[c], j, a);
        }
        if constexpr (kMulti) gsend[j] = emit[C - 1];
      }
      if (W > 1)
        hout[j] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(emit[C - 1]), 63));
    }
#pragma unroll
    for (int c = 0; c < C; ++c) *reinterpret_cast<float4*>(ap[c] + (size_t)g * gstride) = aout[c];
    if constexpr (kMulti) {
      if (gout && wave == W - 1 && lane == 63) {  // entries 4g+1 .. 4g+4 for the block above
#pragma unroll
        for (int j = 0; j < 4; ++j) gout[4 * g + 1 + j] = gsend[j];
      }
      if constexpr (kLive) {
        if (live_out && wave == W - 1 && lane == 63) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            __hip_atomic_store(lrow_out + 4 * g + 1 + j, live_entry(4 * g + 1 + j, gsend[j]),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    if (W > 1 && wave < W - 1 && lane == 0) {  // entries 4g+1 .. 4g+4, then the progress
#pragma unroll
      for (int j = 0; j < 4; ++j) hand_out[4 * g + 1 + j] = hout[j];
      asm volatile("" ::: "memory");
      __hip_atomic_store(&done[wave], 4 * g + 4, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  };
  // four register sets rotate (no copies): a group's loads are requested four groups (16
  // steps, more than a microsecond) ahead -- the planes of a long batch do not fit L2
  auto clamp_g = [&](int g) { return g < ngroups ? g : ngroups - 1; };
  if constexpr (kLive) {
    if (live_in && wave == 0) {  // the upper block starts kLiveLag groups behind (or when the lower is done)
      const int far = min(4 * ngroups, 4 * kLiveLag);
      int spins = 0;
      while ((unsigned)(live_load(far) >> 32) != (unsigned)(far + 1)) {
        if (spins++ >= spin_limit) {
          if (lane == 0) raise_trouble(trouble);
          break;
        }
        __builtin_amdgcn_s_sleep(8);
      }
    }
  }
  Group q0 = load_group(0), q1 = load_group(clamp_g(1)), q2 = load_group(clamp_g(2)),
        q3 = load_group(clamp_g(3));
  if (W > 1 && wave > 0) wait_for(min(4 * ngroups, 4 * (kLive ? kLiveWaveLag : 8) * wave));  // fall a few groups behind
  const std::true_type whole;
  const std::false_type partial;
  const int nwhole = nsteps >> 2;  // groups with all four steps
  int g = 0;
  for (; g + 4 <= nwhole; g += 4) {
    run_group(g, q0, whole);
    q0 = load_group(clamp_g(g + 4));
    run_group(g + 1, q1, whole);
    q1 = load_group(clamp_g(g + 5));
    run_group(g + 2, q2, whole);
    q2 = load_group(clamp_g(g + 6));
    run_group(g + 3, q3, whole);
    q3 = load_group(clamp_g(g + 7));
  }
  // the last one to four groups, the very last of which may be partial
  if (g < ngroups) run_group(g, q0, partial);
  if (g + 1 < ngroups) run_group(g + 1, q1, partial);
  if (g + 2 < ngroups) run_group(g + 2, q2, partial);
  if (g + 3 < ngroups) run_group(g + 3, q3, partial);
  // :73-78 the blank move out of the last cell, negated; that cell was the last one its
  // column processed
#pragma unroll
  for (int c = 0; c < C; ++c)
    if (u0 + c == Ub - 1) costs[b] = -stay[c];
  if constexpr (kLive) {
    if (spin_limit < 0 && live_sink == 1u) raise_trouble(trouble);  // never
  }
}


// ------------------------------------------------------------------ transition weights
// Everything of the dalpha recursion that does not depend on dalpha itself
// (transducer/transducer_cpu.cpp:124-135): one thread per lattice cell.  Every entry of the two
// weight planes is written -- zero where there is no such move or no such cell -- so the
// recursion below needs no bounds of its own.
__global__ __launch_bounds__(256) void weights_kernel(Planes p, const int* __restrict__ inLen,
                                                      const int* __restrict__ labLen, Dims d) {
  __shared__ unsigned long long etab[32];  // expf's table (rnnt_libm.h)
  exp2_table_to_lds(etab);
  __syncthreads();
  // one thread per plane entry, in memory order: entry i of the utterance's plane is
  // anti-diagonal 4 (i / 4Ua) + i % 4 of label position (i % 4Ua) / 4 (Ua is a power of two)
  const int b = blockIdx.z;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= d.Ua * d.Dp) return;
  const int per_group = 4 * d.Ua;  // a power of two
  const int u = (i & (per_group - 1)) >> 2;
  const int dg = 4 * (i >> (31 - __clz(per_group))) + (i & 3);
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const int t = dg - u;
  const size_t o = (size_t)b * d.Ua * d.Dp + i;  // = plane_at(d, b, u, dg)
  float wb = 0.0f, we = 0.0f;
  if (u < Ub && t >= 0 && t < Tb) {
    const float a = p.aS[o], ln = p.lnS[o];
    const size_t o1 = plane_at(d, b, u, dg + 1);
    if (t + 1 < Tb) {
      float x = a + p.eb[(size_t)b * d.Tp + d.Eo + t];
      x = x + p.pb[(size_t)b * d.Ua + u];
      x = x - ln;
      x = x - p.aS[o1];
      wb = expf_glibc(x, etab);
    }
    if (u + 1 < Ub) {
      float x = a + p.elS[o];
      x = x + p.pl[(size_t)b * d.Ua + u];
      x = x - ln;
      x = x - p.aS[o1 + 4];
      we = expf_glibc(x, etab);
    }
  }
  p.wB[o] = wb;
  p.wE[o] = we;
}

// ------------------------------------------------------------------ dalpha
// transducer/transducer_cpu.cpp:81-143 with the exponentials already taken:
// dalpha[t,u] = dalpha[t+1,u]*wB[t,u] + dalpha[t,u+1]*wE[t,u], walked from the last diagonal
// back to the first; the last cell is seeded with 1 (:95) before the walk.  Each lane also
// keeps the running sums that the reference subtracts from pgrads[u,blank] and pgrads[u,l_u],
// in the reference's own order (t descending).  Operands are prefetched beta_depth(C) groups
// of four steps ahead through as many rotating register sets.
// A label axis longer than 64 C positions is walked block by block (u_base = first position of
// the block), HIGHEST block first: what crosses a boundary here is dalpha of the upper block's
// first column, one value per diagonal, left in `ghout` ([B][hand_stride], entry s = its dalpha
// on diagonal s; null for the lowest block) and read by the block below from `ghin` (null for
// the highest block).
// register sets of the dalpha walk's prefetch: eight where a set is small, three (the first
// version's) where a lane owns so many label positions that more sets would spill
constexpr int beta_depth(int C) { return C <= 2 ? 8 : C <= 4 ? 4 : 3; }
// W wavefronts (one launch covering the whole label axis only): wavefront w owns positions
// (64 w + lane) C .. + C-1, so the HIGHEST wavefront leads.  Each but the lowest leaves dalpha of
// its first column in LDS, one value per diagonal, and counts the groups it has finished; the
// wavefront below reads them one group later (the same hand-over as between blocks, with the
// bounded wait of alpha_kernel).  Every wavefront runs all groups, past the utterance's labels
// too (zeros), so nobody waits for a wavefront that has left.
// kLive: the live_n blocks of 64 C W positions of a label axis as live_n workgroups running at
// the same time, as in alpha_kernel with the directions turned round: the HIGHEST block leads
// (and has the smallest workgroup index, so it is dispatched first), lane 0 of a block's
// wavefront 0 leaves dalpha of the block's first column in `live` (entry s: the value on
// diagonal s, s + 1 in the upper word; zero before the launch), and the highest wavefront of the
// block below asks for them, lane j for entry 4g + 1 + j, with its weights, checks the tags when
// it uses them and asks again, bounded, for what was not there yet.  A block above an
// utterance's last label leaves at once, and the utterance's highest block takes nothing.
template <int C, int W, bool kMulti, bool kLive = false>
__global__ __launch_bounds__(64 * W) void beta_kernel(Planes p, const int* __restrict__ labels,
                                                      const int* __restrict__ inLen,
                                                      const int* __restrict__ labLen, Dims d,
                                                      int hand_stride, int u_base,
                                                      const float* __restrict__ ghin,
                                                      float* __restrict__ ghout, int spin_limit,
                                                      int* __restrict__ trouble,
                                                      unsigned long long* __restrict__ live,
                                                      int live_n) {
  static_assert(W == 1 || !kMulti, "several wavefronts only when one launch covers the label axis");
  static_assert(!kLive || (!kMulti && W > 1), "live halves are dealt to several wavefronts");
  extern __shared__ __attribute__((aligned(16))) float hand[];  // [W-1][hand_stride]: entry s =
                                                                // dalpha on diagonal s
  __shared__ int done[W];  // groups a wavefront has published
  // live blocks: as in alpha_kernel, the highest block first
  const int live_block = kLive ? live_n - 1 - (int)(blockIdx.x >> 3) % live_n : 0;
  const int b = kLive ? (int)(blockIdx.x / (8 * live_n)) * 8 + (blockIdx.x & 7) : blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = W > 1 ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : 0;
  if (kLive) {
    if (b >= d.B) return;
    u_base = live_block * 64 * C * W;
  }
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  if (Tb == 0 || Ub == 0) return;  // :92-94
  if (u_base >= Ub) return;        // a block past this utterance's labels
  if (W > 1) {
    if (threadIdx.x < W) done[threadIdx.x] = 0;
    __syncthreads();
  }
  const int nsteps = Tb + Ub - 1;
  const int last = nsteps - 1;  // diagonal of the last cell
  // kSpread: a lane's C positions are 64 apart (u0 + 64 c), so that the 64 lanes of a load or
  // store touch neighbouring 16-byte pieces of the plane, whole cache lines together; the price
  // is a lane-to-scalar move per position and step (lane 63's right neighbour is lane 0's next
  // position).  With two positions a lane next to each other (u0 + c) a load still fills half
  // of every line it touches, and the walk of up to 128 label positions is faster that way
  // (B=32 T=2000 U=100: 38.6 against 45.4 ns a step; two wavefronts of one position: 52.5).
  constexpr bool kSpread = W > 1 || C > 2;
  constexpr int kApart = kSpread ? 64 : 1;
  const int u0 = u_base + wave * 64 * C + (kSpread ? lane : lane * C);
  const int gstride = plane_group_stride(d);
  float* hand_out = hand + (wave > 0 ? wave - 1 : 0) * hand_stride;  // wave > 0
  const float* hand_in = hand + wave * hand_stride;                  // wave < W-1
  const int g_first = last >> 2;  // the group that holds the seed: the first one run
  int avail = 0;                  // groups the wavefront above is known to have published
  auto wait_for = [&](int need) {
    avail = bounded_wait(&done[wave + 1], avail, need, spin_limit, trouble);
  };
  // the block above exists for this utterance only if its first column does
  const float* gin =
      (kMulti && ghin && u_base + 64 * C < Ub) ? ghin + (size_t)b * hand_stride : nullptr;
  float* gout = (kMulti && ghout) ? ghout + (size_t)b * hand_stride : nullptr;
  // live halves: the upper one writes the entries; the highest wavefront of the lower one takes
  // them if the utterance has an upper half at all
  // block h writes the entries of boundary h - 1 and takes those of boundary h, if the utterance
  // has a block above it at all (the highest block asks at its own boundary, for nothing)
  const unsigned long long* lrow =
      kLive ? live + ((size_t)min(live_block, max(live_n - 2, 0)) * d.B + b) * hand_stride
            : nullptr;
  unsigned long long* lrow_out =
      kLive ? live + ((size_t)max(live_block - 1, 0) * d.B + b) * hand_stride : nullptr;
  const bool live_out = kLive && live_block > 0;
  const bool live_takes = kLive && live_block < live_n - 1 && wave == W - 1 &&
                          u_base + 64 * C * W < Ub;
  auto live_load = [&](int s) -> unsigned long long {
    return __hip_atomic_load(lrow + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  // (one opaque statement: see alpha_kernel)
  auto live_reload = [&](int s) -> unsigned long long {
    unsigned long long e;
    const unsigned long long* q = lrow + s;
    asm volatile("global_load_dwordx2 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)"
                 : "=&v"(e)
                 : "v"(q)
                 : "memory");
    return e;
  };
  unsigned live_sink = 0;

  float dcol[C], accB[C], accL[C];
  bool fold[C];  // label of this position equals blank: both sums share one accumulator
  const float* wbp[C];
  const float* wep[C];
  float* dp[C];
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int u = u0 + kApart * c;
    const size_t row = plane_group0(d, b, u);
    wbp[c] = p.wB + row;
    wep[c] = p.wE + row;
    dp[c] = p.dS + row;
    dcol[c] = (u == Ub - 1) ? 1.0f : 0.0f;   // :95
    accB[c] = (u == Ub - 1) ? -1.0f : 0.0f;  // :97
    accL[c] = 0.0f;
    fold[c] = (u + 1 < Ub) && label_at(labels, d, b, u) == d.blank;
  }

  struct Group {
    float4 wb[C], we[C];
    float gh[4];  // dalpha of the block above's first column on diagonals 4g+1 .. 4g+4
    unsigned long long lv;  // the same, tagged, from the half running beside this one: lane j
                            // holds the entry of diagonal 4g + 1 + j
  };
  auto load_group = [&](int g) -> Group {
    Group r;
    const int gc = g > 0 ? g : 0;
#pragma unroll
    for (int c = 0; c < C; ++c) {
      r.wb[c] = *reinterpret_cast<const float4*>(wbp[c] + (size_t)gc * gstride);
      r.we[c] = *reinterpret_cast<const float4*>(wep[c] + (size_t)gc * gstride);
    }
    if constexpr (kMulti) {
#pragma unroll
      for (int j = 0; j < 4; ++j) r.gh[j] = gin ? gin[4 * gc + 1 + j] : 0.0f;  // uniform
    }
    if constexpr (kLive) r.lv = live_load(4 * gc + 1 + (lane & 3));  // every wavefront asks
    return r;
  };
  // steps last-1 .. 0 are computed; the slot of step `last` receives the seed and the slots
  // after it (same group of four) zeros
  // with_fold: some position of this wavefront has the blank as its label, whose two sums then
  // share one accumulator.  Real transcripts have none, and the walk without the two selects per
  // cell is a fifth shorter (x - 0 is x, so the sums come out the same bits either way).
  // seeded: the group that holds the last diagonal (the first one run).  Every other group has
  // all four of its steps below `last`, and is compiled without the test per step (a scalar
  // compare, two mask moves and two branches: eight of the walk's sixteen instructions a step).
  auto run_group = [&](int g, const Group& w, auto with_fold, auto seeded) {
    constexpr bool kFold = decltype(with_fold)::value;
    constexpr bool kSeeded = decltype(seeded)::value;
    float4 dout[C];
    float gsend[4];  // dalpha of this lane's first column after each step
    float hh[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // dalpha of the wavefront above's first column on
                                             // diagonals 4g+1 .. 4g+4
    if (W > 1 && wave < W - 1) {
      wait_for(g_first - g + 1);  // diagonals 4g+1 .. 4g+3 are of its group g
#pragma unroll
      for (int j = 0; j < 4; ++j) hh[j] = hand_in[4 * g + 1 + j];  // uniform
    }
    if constexpr (kLive) {
      if (live_takes) {  // uniform
        // diagonals past the seed's group are never written, and never used either
        const int top = 4 * g_first + 3;
        unsigned long long e = w.lv;
        if (__builtin_amdgcn_ballot_w64(lane < 4 && 4 * g + 1 + lane <= top &&
                                        (unsigned)(e >> 32) != (unsigned)(4 * g + 2 + lane))) {
          // (as in alpha_kernel: let the upper half get kBetaLiveLag groups ahead again)
          const int mine = (lane < 4 && 4 * g + 1 + lane <= top) ? 4 * g + 1 + lane
                                                                 : 4 * max(g - kBetaLiveLag, 0);
          int spins = 0;
          do {
            if (spins++ >= spin_limit) {
              if (lane == 0) raise_trouble(trouble);
              break;
            }
            __builtin_amdgcn_s_sleep(4);
            e = live_reload(mine);
          } while (__builtin_amdgcn_ballot_w64((unsigned)(e >> 32) != (unsigned)(mine + 1)));
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
          hh[j] = __int_as_float(__builtin_amdgcn_readlane((int)(unsigned)e, j));
      } else {
        live_sink ^= (unsigned)w.lv;  // (kept until the end: see alpha_kernel)
      }
    }
#pragma unroll
    for (int j = 3; j >= 0; --j) {
      const int s = 4 * g + j;
      if (kSeeded && s >= last) {  // uniform
#pragma unroll
        for (int c = 0; c < C; ++c) f4set(dout[c], j, s == last ? dcol[c] : 0.0f);
        if constexpr (kMulti || W > 1) gsend[j] = s == last ? dcol[0] : 0.0f;
      } else {
        // dalpha of the position to the right on the diagonal just done, s + 1: the next lane's,
        // and for lane 63 lane 0's next position -- or, right of the wavefront's last position,
        // what the block or the wavefront above handed over (nothing above: 0)
        float right[C];
        float above = 0.0f;  // right of the wavefront's last position
        if constexpr (kMulti) above = gin ? w.gh[j] : 0.0f;
        if (W > 1) above = (wave < W - 1 || live_takes) ? hh[j] : 0.0f;
        if constexpr (kSpread) {
#pragma unroll
          for (int c = 0; c < C; ++c) {
            const float past =  // what lane 63 receives
                c < C - 1 ? __int_as_float(__builtin_amdgcn_readlane(__float_as_int(dcol[c + 1]), 0))
                          : above;
            right[c] = wave_shl1(dcol[c], past);
          }
        } else {
#pragma unroll
          for (int c = 0; c < C; ++c) right[c] = c < C - 1 ? dcol[c + 1] : wave_shl1(dcol[0], above);
        }
#pragma unroll
        for (int c = 0; c < C; ++c) {
          const float ne = dcol[c] * f4get(w.wb[c], j);
          const float em = right[c] * f4get(w.we[c], j);
          const float dn = ne + em;
          if constexpr (kFold) {
            const float em_b = fold[c] ? em : 0.0f, em_l = fold[c] ? 0.0f : em;
            accB[c] = (accB[c] - ne) - em_b;
            accL[c] = accL[c] - em_l;
          } else {
            accB[c] = accB[c] - ne;
            accL[c] = accL[c] - em;
          }
          dcol[c] = dn;
          f4set(dout[c], j, dn);
        }
        if constexpr (kMulti || W > 1) gsend[j] = dcol[0];
      }
    }
#pragma unroll
    for (int c = 0; c < C; ++c) *reinterpret_cast<float4*>(dp[c] + (size_t)g * gstride) = dout[c];
    if constexpr (kMulti) {
      if (gout && lane == 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) gout[4 * g + j] = gsend[j];
      }
    }
    if constexpr (kLive) {
      if (live_out && wave == 0 && lane == 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          __hip_atomic_store(lrow_out + 4 * g + j,
                             ((unsigned long long)(unsigned)(4 * g + j + 1) << 32) |
                                 (unsigned long long)__float_as_uint(gsend[j]),
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (W > 1 && wave > 0 && lane == 0) {  // entries 4g .. 4g+3, then the progress
#pragma unroll
      for (int j = 0; j < 4; ++j) hand_out[4 * g + j] = gsend[j];
      asm volatile("" ::: "memory");  // (LDS serves a wavefront's requests in order)
      __hip_atomic_store(&done[wave], g_first - g + 1, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  };

  // beta_depth(C) register sets rotate (no copies): a group's weights are requested that many
  // groups ahead.  A step of this walk is a dozen instructions, so eight groups are 32 steps or
  // about a microsecond -- what a load that misses L2 takes; with two groups ahead (the first
  // version) the walk waited for its weights at nearly every group: 78 ns a step at U = 101.
  auto walk = [&](auto with_fold) __attribute__((always_inline)) {
    constexpr int kBetaDepth = beta_depth(C);
    int g = g_first;
    if constexpr (kLive) {
      if (live_takes) {  // start kBetaLiveLag groups behind the upper half (or when it is done)
        const int far = 4 * max(g_first - kBetaLiveLag, 0);
        int spins = 0;
        while ((unsigned)(live_load(far) >> 32) != (unsigned)(far + 1)) {
          if (spins++ >= spin_limit) {
            if (lane == 0) raise_trouble(trouble);
            break;
          }
          __builtin_amdgcn_s_sleep(8);
        }
      }
    }
    Group q[kBetaDepth];
#pragma unroll
    for (int i = 0; i < kBetaDepth; ++i) q[i] = load_group(g - i);
    // fall a few groups behind the wavefront above, so that the wait per group finds its
    // counter there already
    if (W > 1 && wave < W - 1) wait_for(min(g_first + 1, (kLive ? kLiveWaveLag : 8) * (W - 1 - wave)));
    // the first round, whose first group holds the seed (a short lattice may end inside it)
    const std::true_type seeded;
    const std::false_type plain;
    run_group(g, q[0], with_fold, seeded);
    q[0] = load_group(g - kBetaDepth);
#pragma unroll
    for (int i = 1; i < kBetaDepth; ++i) {
      if (g - i >= 0) run_group(g - i, q[i], with_fold, plain);
      q[i] = load_group(g - i - kBetaDepth);
    }
    g -= kBetaDepth;
    for (; g >= kBetaDepth - 1; g -= kBetaDepth) {
#pragma unroll
      for (int i = 0; i < kBetaDepth; ++i) {
        run_group(g - i, q[i], with_fold, plain);
        q[i] = load_group(g - i - kBetaDepth);
      }
    }
#pragma unroll
    for (int i = 0; i < kBetaDepth - 1; ++i)
      if (g - i >= 0) run_group(g - i, q[i], with_fold, plain);
  };
  bool any_fold = false;
#pragma unroll
  for (int c = 0; c < C; ++c) any_fold = any_fold || fold[c];
  if (__ballot(any_fold) != 0) walk(std::true_type{});
  else walk(std::false_type{});

#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int u = u0 + kApart * c;
    if (u < Ub) {
      p.gB[(size_t)b * d.Ua + u] = accB[c];
      p.gL[(size_t)b * d.Ua + u] = accL[c];
    }
  }
  if constexpr (kLive) {
    if (spin_limit < 0 && live_sink == 1u) raise_trouble(trouble);  // never
  }
}

// ------------------------------------------------------------------ sparse gradient terms
// The blank/label terms of transducer/transducer_cpu.cpp:95-141, scattered into egrads from what
// frame_terms_block (below) leaves: bsum[b][t], the finished value of column `blank` of frame t,
// and emT[b][u][t], the label move's term of every cell.  One thread per frame walks the label
// positions from last to first, which is the order in which the reference subtracts into a row
// of egrads, so repeated labels round the same way; a label position's terms of 256 consecutive
// frames are 1 KB in a row.  pgrads comes from the sums the dalpha kernel kept.  add == 0: the
// terms are stored (the arrays were zero-filled); add != 0: scale[b] (1 when scale is null)
// times the term is added to what the arrays hold.
__global__ __launch_bounds__(256) void sparse_e_kernel(const float* __restrict__ bsum,
                                                       const float* __restrict__ emT,
                                                       float* __restrict__ egrads,
                                                       const int* __restrict__ labels,
                                                       const int* __restrict__ inLen,
                                                       const int* __restrict__ labLen,
                                                       const float* __restrict__ scale, int add,
                                                       Dims d) {
  const int b = blockIdx.y;
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  if (Ub == 0 || t >= Tb) return;
  float* __restrict__ row = egrads + ((size_t)b * d.T + t) * d.V;
  const int* __restrict__ lab = labels + (size_t)b * (d.U - 1);
  const float* __restrict__ em = emT + (size_t)b * d.U * d.T + t;
  const float sc = scale ? scale[b] : 1.0f;
  const float blank_total = bsum[(size_t)b * d.T + t];
  // Positions are taken eight at a time, last to first; the terms of the next eight are
  // requested before the current eight are folded in, so the loop runs at the rate of the
  // memory pipe rather than one round trip per label position.
  constexpr int kChunk = 8;
  struct Chunk { float em[kChunk]; };
  auto load_chunk = [&](int uhi) -> Chunk {  // positions uhi, uhi-1, ..., uhi-7 (those >= 0)
    Chunk c;
#pragma unroll
    for (int k = 0; k < kChunk; ++k) c.em[k] = em[(size_t)max(uhi - k, 0) * d.T];
    return c;
  };
  Chunk cur = load_chunk(Ub - 2);  // the last position has no label move
  for (int uhi = Ub - 2; uhi >= 0; uhi -= kChunk) {
    const Chunk nxt = load_chunk(uhi - kChunk);
#pragma unroll
    for (int k = 0; k < kChunk; ++k) {
      const int u = uhi - k;
      if (u >= 0) {
        const int l = clampi(lab[u], 0, d.V - 1);
        // Label columns are updated with no-return hardware adds: nothing waits on them,
        // and since this thread alone touches row t and its requests to one address stay
        // in order, repeated labels still accumulate in the reference's order.  (A label move
        // whose label is the blank is already part of the blank total.)
        if (l != d.blank) unsafeAtomicAdd(&row[l], add ? sc * (-cur.em[k]) : -cur.em[k]);
      }
    }
    cur = nxt;
  }
  if (add) row[d.blank] += sc * blank_total;
  else row[d.blank] = blank_total;
}

// The same terms for a small vocabulary, added (times scale[b]) onto an egrads that holds the
// dense part.  With few columns the hardware adds of sparse_e_kernel all land in a few cache
// lines per row and queue up at L2 (B=8, T=2000, U=100, V=100: 0.08 ms for 1.6 M adds), so
// here a wavefront keeps its 64 frames' rows in LDS (64 x V floats, odd pitch: lane t owns row
// t, all lanes hit column l together, no conflicts), subtracts the terms there in the
// reference's order, and then adds the rows to egrads with row-contiguous accesses.
// Dynamic LDS: 64 * (V | 1) floats.
__global__ __launch_bounds__(64) void sparse_e_rows_kernel(const float* __restrict__ bsum,
                                                           const float* __restrict__ emT,
                                                           float* __restrict__ egrads,
                                                           const int* __restrict__ labels,
                                                           const int* __restrict__ inLen,
                                                           const int* __restrict__ labLen,
                                                           const float* __restrict__ scale,
                                                           Dims d) {
  extern __shared__ float rows[];
  const int b = blockIdx.y, t0 = blockIdx.x * 64, lane = threadIdx.x;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  if (Ub == 0 || t0 >= Tb) return;
  const int pitch = d.V | 1;
  for (int i = lane; i < 64 * pitch; i += 64) rows[i] = 0.0f;
  __syncthreads();
  const int t = min(t0 + lane, Tb - 1);  // lanes past the utterance walk its last frame, unused
  float* mine = rows + lane * pitch;
  const int* __restrict__ lab = labels + (size_t)b * (d.U - 1);
  const float* __restrict__ em = emT + (size_t)b * d.U * d.T + t;
  constexpr int kChunk = 16;
  for (int uhi = Ub - 2; uhi >= 0; uhi -= kChunk) {
    float e[kChunk];
#pragma unroll
    for (int k = 0; k < kChunk; ++k) e[k] = em[(size_t)max(uhi - k, 0) * d.T];
#pragma unroll
    for (int k = 0; k < kChunk; ++k) {
      const int u = uhi - k;
      if (u >= 0) {  // uniform
        const int l = clampi(lab[u], 0, d.V - 1);
        if (l != d.blank) mine[l] -= e[k];
      }
    }
  }
  mine[d.blank] += bsum[(size_t)b * d.T + t];
  __syncthreads();
  const float sc = scale ? scale[b] : 1.0f;
  const int nrows = min(64, Tb - t0);
  // eight rows at a time, their loads requested together (a row-by-row read-add-write would pay
  // one round trip per row)
  float* base = egrads + ((size_t)b * d.T + t0) * d.V;
  for (int v = lane; v < d.V; v += 64) {
    for (int r0 = 0; r0 < nrows; r0 += 8) {
      float have[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) have[k] = base[(size_t)min(r0 + k, nrows - 1) * d.V + v];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const float x = rows[min(r0 + k, nrows - 1) * pitch + v];
        if (r0 + k < nrows && x != 0.0f) base[(size_t)(r0 + k) * d.V + v] = have[k] + sc * x;
      }
    }
  }
}

// What the reference subtracts from egrads besides the dense part, per lattice cell
// (transducer/transducer_cpu.cpp:96,106,138), in the form the dense egrads kernel folds into its
// write-out:
//   bsum[b][t]    the total that lands in column `blank` of frame t: -1 for the last frame (:96),
//                 every blank move's dalpha[t+1,u] wB[t,u], and the label moves whose label is the
//                 blank -- the value sparse_e_kernel would leave in that column;
//   emT[b][u][t]  the label move's dalpha[t,u+1] wE[t,u] of every cell ([B][U][T]: the kernel that
//                 folds them in reads one label position's frames in a row).
// One lane per frame subtracts its frame's terms in the reference's order, label positions last
// to first; a wavefront takes 64 frames and works alone (no workgroup barrier).  The operands
// come through LDS: for eight label positions at a time the wavefront copies the groups of
// anti-diagonals its 64 frames meet there -- 128 contiguous bytes a group and plane -- with
// 16-byte loads, requested one chunk ahead, and each lane then picks its own cells (read straight
// from the planes, the 64 frames would touch 17 cache lines per load).
constexpr int kBsFrames = 64, kBsPos = 8;
constexpr int kBsGroups = (kBsFrames + kBsPos + 3) / 4 + 1;  // groups of four anti-diagonals a chunk meets
// floats per staged group; the pitches put the 16-byte pieces of consecutive groups on different banks
constexpr int kBsPitch = 4 * kBsPos + 4;         // wB, wE: eight positions
constexpr int kBsPitchD = 4 * (kBsPos + 1) + 8;  // dalpha: nine (a cell's label move enters position u+1)
constexpr int kBsPieces = (kBsGroups * kBsPos + 63) / 64;         // 16-byte pieces a lane copies per plane
constexpr int kBsPiecesD = (kBsGroups * (kBsPos + 1) + 63) / 64;
constexpr int kBsWave = kBsGroups * (2 * kBsPitch + kBsPitchD);   // floats of LDS a wavefront stages in
constexpr int kPostBetaLds = 4 * kBsWave > 64 * 65 ? 4 * kBsWave : 64 * 65;  // floats: either kind of block
__device__ __forceinline__ void frame_terms_block(const Planes& p, float* __restrict__ bsum,
                                                  float* __restrict__ emT,
                                                  const int* __restrict__ labels,
                                                  const int* __restrict__ inLen,
                                                  const int* __restrict__ labLen, const Dims& d,
                                                  int bx, int b, float* __restrict__ lds) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t0 = (4 * bx + wave) * kBsFrames, t = t0 + lane;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  if (Ub == 0 || t0 >= Tb) return;  // the whole wavefront
  const bool active = t < Tb;
  const int* __restrict__ lab = labels + (size_t)b * (d.U - 1);
  const float* __restrict__ dS = p.dS;
  const float* __restrict__ wB = p.wB;
  const float* __restrict__ wE = p.wE;
  float* stW = lds + wave * kBsWave;        // wB of anti-diagonal groups gbase ..
  float* stE = stW + kBsGroups * kBsPitch;  // wE
  float* stD = stE + kBsGroups * kBsPitch;  // dalpha
  const size_t plane_b = (size_t)b * d.Ua * d.Dp;
  const int ngroups_plane = d.Dp >> 2;
  const bool has_stay = t + 1 < Tb;
  float acc = (t == Tb - 1) ? -1.0f : 0.0f;
  // cell (t,u) reads the weights on anti-diagonal t+u and dalpha on t+u+1: positions ua .. ua+7
  // of the wavefront's frames meet groups (t0 + ua) / 4 .. (t0 + ua + 64 + 7) / 4
  struct Pieces { float4 w[kBsPieces], e[kBsPieces], d[kBsPiecesD]; };
  const float4 zero4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  auto request = [&](int ua) -> Pieces {
    Pieces r;
    const int gbase = (t0 + max(ua, 0)) >> 2;
#pragma unroll
    for (int i = 0; i < kBsPieces; ++i) {
      const int f = 64 * i + lane, g = gbase + f / kBsPos, ul = f % kBsPos;
      r.w[i] = zero4;
      r.e[i] = zero4;
      if (ua >= 0 && f < kBsGroups * kBsPos && g < ngroups_plane) {  // (ua + ul < Ua: a multiple of 64)
        const size_t o = plane_b + ((size_t)g * d.Ua + ua + ul) * 4;
        r.w[i] = *reinterpret_cast<const float4*>(wB + o);
        r.e[i] = *reinterpret_cast<const float4*>(wE + o);
      }
    }
#pragma unroll
    for (int i = 0; i < kBsPiecesD; ++i) {
      const int f = 64 * i + lane, g = gbase + f / (kBsPos + 1), ul = f % (kBsPos + 1);
      r.d[i] = zero4;
      // (position ua + 8 may be Ua itself: the address is then position 0 of the next group,
      // inside the plane since g + 1 groups exist, and no cell uses the value)
      if (ua >= 0 && f < kBsGroups * (kBsPos + 1) && g + 1 < ngroups_plane)
        r.d[i] = *reinterpret_cast<const float4*>(dS + plane_b + ((size_t)g * d.Ua + ua + ul) * 4);
    }
    return r;
  };
  const int ua_first = (Ub - 1) & ~(kBsPos - 1);
  Pieces cur = request(ua_first);
  for (int ua = ua_first; ua >= 0; ua -= kBsPos) {
    const int gbase = (t0 + ua) >> 2;
    // (LDS serves a wavefront's accesses in order; the fences only hold the compiler to it)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < kBsPieces; ++i) {
      const int f = 64 * i + lane;
      if (f < kBsGroups * kBsPos) {
        *reinterpret_cast<float4*>(stW + (f / kBsPos) * kBsPitch + 4 * (f % kBsPos)) = cur.w[i];
        *reinterpret_cast<float4*>(stE + (f / kBsPos) * kBsPitch + 4 * (f % kBsPos)) = cur.e[i];
      }
    }
#pragma unroll
    for (int i = 0; i < kBsPiecesD; ++i) {
      const int f = 64 * i + lane;
      if (f < kBsGroups * (kBsPos + 1))
        *reinterpret_cast<float4*>(stD + (f / (kBsPos + 1)) * kBsPitchD + 4 * (f % (kBsPos + 1))) =
            cur.d[i];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    cur = request(ua - kBsPos);
    if (active) {
#pragma unroll
      for (int k = kBsPos - 1; k >= 0; --k) {
        const int u = ua + k;
        if (u < Ub) {  // uniform
          const int dd = t + u;
          const int here = ((dd >> 2) - gbase) * kBsPitch + 4 * k + (dd & 3);
          const int next = (((dd + 1) >> 2) - gbase) * kBsPitchD + 4 * k + ((dd + 1) & 3);
          const float ne = stD[next] * stW[here];      // dalpha[t+1,u] wB[t,u]
          const float em = stD[next + 4] * stE[here];  // dalpha[t,u+1] wE[t,u]
          acc -= has_stay ? ne : 0.0f;
          const bool has_label = u + 1 < Ub;
          if (has_label && clampi(lab[u], 0, d.V - 1) == d.blank) acc -= em;
          emT[((size_t)b * d.U + u) * d.T + t] = has_label ? em : 0.0f;
        }
      }
    }
  }
  if (active) bsum[(size_t)b * d.T + t] = acc;
}

// W from the skewed planes the lattice kernels leave behind (dalpha and LN): no un-skewed copy of
// dalpha is needed first.  A block takes 64 label positions x 64 anti-diagonals (16 groups of
// four: 1 KB of contiguous memory a group and plane, read with 16-byte loads), forms W of those
// cells, and writes them to both orientations through an LDS tile.  Its frames are the 127
// t = dd - u; the blocks (64 by, 64 bx) over all anti-diagonals below Tw + Up tile the planes.
// Same arithmetic per cell as wplanes_kernel, same bits.
__device__ __forceinline__ void wplanes_skewed_block(
    const float* __restrict__ dS, const float* __restrict__ lnS, const float* __restrict__ mE,
    const float* __restrict__ mP, float* __restrict__ Wn, float* __restrict__ Wt,
    const int* __restrict__ inLen, const int* __restrict__ labLen, const Dims& d, int Up, int Tw,
    float (*tile)[65], int bx, int by, int b) {
  const int dd0 = bx * 64, u0 = by * 64;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const size_t plane_b = (size_t)b * d.Ua * d.Dp;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int f = k * 256 + threadIdx.x, gl = f >> 6, ul = f & 63;
    const int u = u0 + ul, g = (dd0 >> 2) + gl;
    const int tq = 4 * g - u;  // frame of the group's first anti-diagonal
    float w[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (u < Ub && tq + 3 >= 0 && tq < Tb) {  // (so 4g < T + U: the group lies inside the plane)
      const size_t o = plane_b + ((size_t)g * d.Ua + u) * 4;
      const float4 d4 = *reinterpret_cast<const float4*>(dS + o);
      const float4 l4 = *reinterpret_cast<const float4*>(lnS + o);
      const float mp = mP[(size_t)b * d.U + u];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int t = tq + j;
        if (t >= 0 && t < Tb) {
          const float me = mE[(size_t)b * d.T + t];
          w[j] = f4get(d4, j) * expf((me + mp) - f4get(l4, j)) * frame_exp_correction(me);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) tile[ul][4 * gl + j] = w[j];  // [label position][anti-diagonal]
  }
  __syncthreads();
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {  // rows of Wt: one label position, 64 consecutive frames
    const int ul = ty + 4 * i, u = u0 + ul, t = dd0 + tx - u;
    if (t >= 0 && t < Tw && u < Up) Wt[((size_t)b * Up + u) * Tw + t] = tile[ul][tx];
  }
  for (int i = 0; i < 32; ++i) {  // rows of Wn: one frame, the label positions it has in the tile
    const int r = ty + 4 * i;     // frame dd0 - u0 - 63 + r meets position u0 + tx on dd0 + tx + r - 63
    const int t = dd0 - u0 - 63 + r, u = u0 + tx, c = tx + r - 63;
    if (c >= 0 && c < 64 && t >= 0 && t < Tw && u < Up)
      Wn[((size_t)b * Tw + t) * Up + u] = tile[tx][c];
  }
}

// W of 64 frames x 64 label positions as bf16 pieces, in the two slab images the fused gradient
// kernel copies into LDS as they are (WImages).  Same arithmetic per cell as above.
__device__ __forceinline__ void wimages_block(
    const float* __restrict__ dS, const float* __restrict__ lnS, const float* __restrict__ mE,
    const float* __restrict__ mP, const int* __restrict__ inLen, const int* __restrict__ labLen,
    const Dims& d, int Tw, float (*tile)[65], int bx, int by, int b, const WImages& img) {
  const int t0 = bx * 64, u0 = by * 64;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int u = u0 + ty + 4 * i, t = t0 + tx;
    float w = 0.0f;
    if (t < Tb && u < Ub) {
      const size_t o = plane_at(d, b, u, t + u);
      const float me = mE[(size_t)b * d.T + t];
      w = dS[o] * expf((me + mP[(size_t)b * d.U + u]) - lnS[o]) * frame_exp_correction(me);
    }
    tile[ty + 4 * i][tx] = w;  // [label position][frame]
  }
  __syncthreads();
  const int ntile = Tw >> 5;
  // frames x label positions (the egrads operand): pairs of neighbouring label positions
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int id = k * 256 + threadIdx.x, tl = id >> 5, j = id & 31;
    const int u = u0 + 2 * j;
    if (u < WImages::kCols) {
      unsigned ph, pm, pl;
      split_pair(tile[2 * j][tl], tile[2 * j + 1][tl], ph, pm, pl);
      unsigned* dst = img.e + ((size_t)b * ntile + ((t0 + tl) >> 5)) * (3 * WImages::kEPlane) +
                      ((t0 + tl) & 31) * (WImages::kCols / 2) + (u >> 1);
      dst[0] = ph;
      dst[WImages::kEPlane] = pm;
      dst[2 * WImages::kEPlane] = pl;
    }
  }
  // label positions x frames (the pgrads operand), the frames of a slab in the order the fused
  // kernel feeds them to the matrix instruction: slot = frame with bits 2 and 3 swapped (its own
  // inverse; pairs of neighbouring frames stay pairs)
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int id = k * 256 + threadIdx.x, ul = id >> 5, q = id & 31;
    const int sel = q >> 4, slot = 2 * (q & 15);
    const int f = (slot & 16) | ((slot & 4) << 1) | ((slot & 8) >> 1) | (slot & 2);
    unsigned ph, pm, pl;
    split_pair(tile[ul][32 * sel + f], tile[ul][32 * sel + f + 1], ph, pm, pl);
    unsigned* dst = img.p + ((size_t)b * ntile + (t0 >> 5) + sel) * (3 * WImages::kPPlane) +
                    (u0 + ul) * 16 + (slot >> 1);
    dst[0] = ph;
    dst[WImages::kPPlane] = pm;
    dst[2 * WImages::kPPlane] = pl;
  }
}


// W planes and per-frame blank totals in one launch: both only need the finished dalpha plane and
// neither needs the other, so the blocks of the second fill the device beside the first's
// instead of waiting behind a kernel boundary.  The last nw blocks form W (tile bx, by of
// utterance b; with `img` the tiles are 64 frames x 64 label positions and go to the slab images
// instead), the blocks before them the per-frame terms bsum and emT (bsum == nullptr: none).
__global__ __launch_bounds__(256) void post_beta_kernel(Planes p, const float* __restrict__ mE,
                                                        const float* __restrict__ mP,
                                                        float* __restrict__ Wn,
                                                        float* __restrict__ Wt,
                                                        float* __restrict__ bsum,
                                                        float* __restrict__ emT,
                                                        const int* __restrict__ labels,
                                                        const int* __restrict__ inLen,
                                                        const int* __restrict__ labLen, Dims d,
                                                        int Up, int Tw, int wx, int wy, int nw,
                                                        int sx, WImages img) {
  __shared__ __attribute__((aligned(16))) float lds[kPostBetaLds];
  float (*tile)[65] = reinterpret_cast<float (*)[65]>(lds);
  // the per-frame blocks come first in the grid: each runs longer than a W tile, and started
  // last they would be the kernel's tail
  const int ns = gridDim.x - nw;
  if ((int)blockIdx.x >= ns) {
    const int n = blockIdx.x - ns;
    const int b = n / (wx * wy), r = n - b * (wx * wy);
    if (img.e)
      wimages_block(p.dS, p.lnS, mE, mP, inLen, labLen, d, Tw, tile, r % wx, r / wx, b, img);
    else
      wplanes_skewed_block(p.dS, p.lnS, mE, mP, Wn, Wt, inLen, labLen, d, Up, Tw, tile, r % wx,
                           r / wx, b);
  } else {
    const int m = blockIdx.x;
    frame_terms_block(p, bsum, emT, labels, inLen, labLen, d, m % sx, m / sx, lds);
  }
}

__global__ __launch_bounds__(256) void sparse_p_kernel(Planes p, float* __restrict__ pgrads,
                                                       const int* __restrict__ labels,
                                                       const int* __restrict__ inLen,
                                                       const int* __restrict__ labLen,
                                                       const float* __restrict__ scale, int add,
                                                       Dims d) {
  const int b = blockIdx.y;
  const int u = blockIdx.x * 256 + threadIdx.x;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  if (Tb == 0 || u >= Ub) return;
  float* row = pgrads + ((size_t)b * d.U + u) * d.V;
  const float gb = p.gB[(size_t)b * d.Ua + u], gl = p.gL[(size_t)b * d.Ua + u];
  const bool has_label = u + 1 < Ub;
  const int l = has_label ? label_at(labels, d, b, u) : d.blank;
  if (add) {
    const float sc = scale ? scale[b] : 1.0f;
    row[d.blank] += sc * gb;
    if (has_label && l != d.blank) row[l] += sc * gl;
  } else {
    row[d.blank] = gb;
    if (has_label && l != d.blank) row[l] = gl;
  }
}

// ------------------------------------------------------------------ max-plus table
// best[t,u] = max over v != blank of E[t,v]+P[u,v], arg = lowest such v
// (transducer/transducer_cpu.cpp:158-171).  Pure vector-ALU work (max-plus has no matrix form),
// so the kernel is laid out to spend its instructions on the add and the max:
//   * a workgroup of 8 wavefronts owns 128 frames x 64 label positions; a wavefront owns 8 label
//     positions, a lane two frames (lane, lane+64): 16 cells per lane (two workgroups share a
//     CU; with 16 wavefronts and 128 label positions per workgroup only one fits, and the
//     wavefronts idling past a short utterance's last label cost a whole slot);
//   * E and P stream through LDS in chunks of 32 columns (double-buffered, one barrier per
//     chunk); E is staged with the blank column, columns past V and frames past the utterance at
//     -inf; a lane reads its two rows of E 16 bytes at a time (row pitch 36 floats:
//     conflict-free), and the P values of the wavefront's 8 rows, which are the same for all its
//     lanes, with broadcast reads (one address per wavefront).  Scalar loads would bring them in
//     as scalar operands, but they return out of order, so only one row could be in flight and
//     the L2 latency of every row showed: measured 5.5 ms against 6.8 ms for a 4x4-cells
//     LDS-tiled first version;
//   * the running maximum is exact and order-free; per chunk a cell only notes whether the
//     chunk raised it, and the index is recovered afterwards by rescanning the first chunk that
//     reached the maximum.
// Wavefronts whose label positions lie past the utterance only help staging.
constexpr int kMpT = 128, kMpK = 32, kMpPitch = 36, kMpRows = 8;
constexpr int kMpWaves = 8, kMpU = kMpWaves * kMpRows, kMpThreads = 64 * kMpWaves;
constexpr int kMpEPasses = kMpT * (kMpK / 4) / kMpThreads;  // 16-byte pieces of the E chunk per thread

// kVec: V is a multiple of 4, so four consecutive elements never straddle a row's end and every
// group of four is naturally aligned (16 bytes in fp32, 8 in bf16).
template <bool kVec, typename TIO>
__global__ __launch_bounds__(kMpThreads) void maxplus_kernel(const TIO* __restrict__ E,
                                                       const TIO* __restrict__ P,
                                                       const int* __restrict__ inLen,
                                                       const int* __restrict__ labLen,
                                                       float* __restrict__ best,
                                                       int* __restrict__ arg, Dims d,
                                                       const int* __restrict__ tile_fail,
                                                       const int* __restrict__ lists_on,
                                                       int fail_limit) {
  __shared__ __attribute__((aligned(16))) float Es[2][kMpT * kMpPitch];
  __shared__ __attribute__((aligned(16))) float Ps[2][kMpU * kMpK];
  const int b = blockIdx.z, t0 = blockIdx.x * kMpT, u0 = blockIdx.y * kMpU;
  // after the list pass (if it went past its sample): only the tiles in which too many cells
  // failed its test are redone
  if (tile_fail && lists_on[0] != 0 &&
      tile_fail[((size_t)b * gridDim.x + blockIdx.x) * gridDim.y + blockIdx.y] <= fail_limit)
    return;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  if (t0 >= Tb || u0 >= Ub) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const TIO* Eb = E + (size_t)b * d.T * d.V;
  const TIO* Pb = P + (size_t)b * d.U * d.V;
  const int ur0 = u0 + wave * kMpRows;  // first label position of this wavefront
  const bool active = ur0 < Ub;

  // staging role: thread -> row srow of the P tile and rows srow + (kMpThreads/8) * i of the E
  // tile, four columns from sc4
  const int srow = tid >> 3, sc4 = (tid & 7) * 4;
  const TIO* esrc[kMpEPasses];
  bool erow_ok[kMpEPasses];
#pragma unroll
  for (int i = 0; i < kMpEPasses; ++i) {
    const int t = t0 + srow + (kMpThreads / 8) * i;
    erow_ok[i] = t < Tb;
    esrc[i] = Eb + (size_t)min(t, Tb - 1) * d.V;
  }
  const TIO* psrc = Pb + (size_t)min(u0 + srow, Ub - 1) * d.V;  // rows past the utterance are
                                                                  // computed and dropped
  // the raw values are requested before a chunk's arithmetic and stored after it, so the wait
  // for them falls behind the arithmetic
  auto fetch = [&](const TIO* src, int k) -> float4 {
    const int v = k * kMpK + sc4;
    float4 x;
    if (kVec) {  // columns past V are re-read from the row's last four (E: masked below; P: any
                 // finite value will do there, E is -inf)
      x = load4(src + min(v, d.V - 4));
    } else {  // one wide load at the element's own alignment, one by one at the row's end
      x = load4_any(src, min(v, d.V - 1), d.V);
    }
    return x;
  };
  struct Staged {
    float4 e[kMpEPasses], p;
  };
  auto fetch_all = [&](int k) -> Staged {
    Staged r;
#pragma unroll
    for (int i = 0; i < kMpEPasses; ++i) r.e[i] = fetch(esrc[i], k);
    r.p = fetch(psrc, k);
    return r;
  };
  auto stash = [&](int buf, int k, const Staged& r) {
    const int v = k * kMpK + sc4;
#pragma unroll
    for (int i = 0; i < kMpEPasses; ++i) {
      float4 x = r.e[i];
      x.x = (erow_ok[i] && v < d.V && v != d.blank) ? x.x : kNegInf;
      x.y = (erow_ok[i] && v + 1 < d.V && v + 1 != d.blank) ? x.y : kNegInf;
      x.z = (erow_ok[i] && v + 2 < d.V && v + 2 != d.blank) ? x.z : kNegInf;
      x.w = (erow_ok[i] && v + 3 < d.V && v + 3 != d.blank) ? x.w : kNegInf;
      *reinterpret_cast<float4*>(&Es[buf][(srow + (kMpThreads / 8) * i) * kMpPitch + sc4]) = x;
    }
    *reinterpret_cast<float4*>(&Ps[buf][srow * kMpK + sc4]) = r.p;
  };

  float top[2][kMpRows];
  int chunk[2][kMpRows];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < kMpRows; ++r) { top[i][r] = kNegInf; chunk[i][r] = -1; }

  const int nchunks = (d.V + kMpK - 1) / kMpK;
  int cur = 0;
  stash(0, 0, fetch_all(0));
  __syncthreads();
  for (int k = 0; k < nchunks; ++k) {
    const int kn = min(k + 1, nchunks - 1);  // the last chunk re-reads its own
    const Staged nxt = fetch_all(kn);
    if (active) {
      float cm[2][kMpRows];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int r = 0; r < kMpRows; ++r) cm[i][r] = kNegInf;
#pragma unroll
      for (int sub = 0; sub < kMpK / 8; ++sub) {
        float e[2][8];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const float4 lo =
              *reinterpret_cast<const float4*>(&Es[cur][(lane + 64 * i) * kMpPitch + sub * 8]);
          const float4 hi =
              *reinterpret_cast<const float4*>(&Es[cur][(lane + 64 * i) * kMpPitch + sub * 8 + 4]);
          e[i][0] = lo.x; e[i][1] = lo.y; e[i][2] = lo.z; e[i][3] = lo.w;
          e[i][4] = hi.x; e[i][5] = hi.y; e[i][6] = hi.z; e[i][7] = hi.w;
        }
        const float* pw = &Ps[cur][wave * kMpRows * kMpK + sub * 8];
#pragma unroll
        for (int r = 0; r < kMpRows; ++r) {
          const float4 plo = *reinterpret_cast<const float4*>(pw + r * kMpK);
          const float4 phi = *reinterpret_cast<const float4*>(pw + r * kMpK + 4);
          const float pv[8] = {plo.x, plo.y, plo.z, plo.w, phi.x, phi.y, phi.z, phi.w};
#pragma unroll
          for (int c = 0; c < 8; c += 2) {
            cm[0][r] = fmaxf(fmaxf(cm[0][r], e[0][c] + pv[c]), e[0][c + 1] + pv[c + 1]);
            cm[1][r] = fmaxf(fmaxf(cm[1][r], e[1][c] + pv[c]), e[1][c + 1] + pv[c + 1]);
          }
        }
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int r = 0; r < kMpRows; ++r)
          if (cm[i][r] > top[i][r]) { top[i][r] = cm[i][r]; chunk[i][r] = k; }
    }
    stash(cur ^ 1, kn, nxt);
    __syncthreads();
    cur ^= 1;
  }
  if (!active) return;
  // Recover the lowest index inside the winning chunk: the chunk's 32 columns of the cell's two
  // rows come in as sixteen 16-byte loads, all requested before the first is looked at, and the
  // sums are compared in registers.  (Looked up column by column, the way the reference scans,
  // this was two dependent loads and a wait per column and cell: five hundred memory round
  // trips in a row at the end of every wavefront.)  Every lane goes through the loads with
  // clamped rows; only cells of the utterance are written.
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < kMpRows; ++r) {
      const int t = t0 + lane + 64 * i, u = ur0 + r;
      const bool cell = t < Tb && u < Ub;
      const int v0 = max(chunk[i][r], 0) * kMpK;
      const TIO* e = Eb + (size_t)min(t, Tb - 1) * d.V;
      const TIO* q = Pb + (size_t)min(u, Ub - 1) * d.V;
      float4 ev[kMpK / 4], pv[kMpK / 4];
#pragma unroll
      for (int g = 0; g < kMpK / 4; ++g) {
        const int v = v0 + 4 * g;
        // (kVec: a group of four is inside the row or past it as a whole, and one past it is
        // never looked at, so the clamped start only keeps the load inside the array)
        ev[g] = kVec ? load4(e + min(v, d.V - 4)) : load4_any(e, min(v, d.V - 1), d.V);
        pv[g] = kVec ? load4(q + min(v, d.V - 4)) : load4_any(q, min(v, d.V - 1), d.V);
      }
      int at = 0;  // :160 the scan starts from index 0 and keeps it if nothing beats -inf
      if (chunk[i][r] >= 0) {
        const float want = top[i][r];
        // from the last column down, so that the lowest match is what remains
#pragma unroll
        for (int g = kMpK / 4 - 1; g >= 0; --g) {
          const float sum[4] = {ev[g].x + pv[g].x, ev[g].y + pv[g].y, ev[g].z + pv[g].z,
                                ev[g].w + pv[g].w};
#pragma unroll
          for (int j = 3; j >= 0; --j) {
            const int v = v0 + 4 * g + j;
            if (v < d.V && v != d.blank && sum[j] == want) at = v;
          }
        }
      }
      if (cell) {
        // straight into the skewed planes the lattice walk reads
        const size_t o = plane_at(d, b, u, t + u);
        best[o] = top[i][r];
        arg[o] = at;
      }
    }
}

// ------------------------------------------------------------------ viterbi
// transducer/transducer_cpu.cpp:145-222.  Scores walk the lattice like alpha with
// max in place of log-sum-exp: no transcendental anywhere, so given the same LN the path is
// bit-exact.  Association: blank move ((s + e) + p) - LN (:192-195), label move
// (s + best) - LN (:197-199); "emit > stay" takes the label, ties go to blank (:200-206).
// The decision of every cell is one bit; each step's 64-lane ballot goes to `bits`
// (LDS when it fits, else global), and lane 0 walks them backwards at the end (:208-219).
// C cells per lane, W wavefronts (the label positions dealt to them as in alpha_kernel, with
// the same hand-over of the boundary score).
// The decision of a cell is one bit.  A lane keeps the bits of its own cells, 32 steps to a
// word, and stores a word when it is full: column u of the table `cols` holds the decisions of
// label position u over all steps.  The backtrace then does not walk the ~T+U moves one by one:
// at position u, reached at step s, the move that entered u is the highest set bit at or below
// s in column u (everything above it is blank moves), found with one or two word reads and a
// count-leading-zeros; U-1 such searches, by one lane, and the labels are fetched by all lanes
// afterwards.
// Dynamic LDS: one int per label position (steps at which labels were taken), the hand-over
// array (W > 1), the columns (kLdsBits; else they live in global memory).
// kLive (with kMulti, columns in global memory): live_n blocks of 64 C W label positions side by
// side, one workgroup each, the boundary column's scores crossing in tagged 64-bit entries as in
// alpha_kernel (same order of workgroups, same bounded waits).  Such a launch only walks; the
// path is traced by a launch of its own afterwards (traces != 0, u_base past every label).
template <int C, int W, bool kLdsBits, bool kMulti, bool kLive = false>
__global__ __launch_bounds__(64 * W) void viterbi_kernel(Planes p, const float* __restrict__ bestS,
                                                         const float* __restrict__ argS,
                                                         const int* __restrict__ inLen,
                                                         const int* __restrict__ labLen,
                                                         unsigned* __restrict__ gcols,
                                                         int* __restrict__ labels_out, Dims d,
                                                         int hand_stride, int nw, int spin_limit,
                                                         int* __restrict__ trouble, int u_base,
                                                         const float* __restrict__ ghin,
                                                         float* __restrict__ ghout,
                                                         int traces,
                                                         unsigned long long* __restrict__ live,
                                                         int live_n) {
  static_assert(!kLive || (kMulti && !kLdsBits), "live blocks keep their columns in global memory");
  extern __shared__ __attribute__((aligned(16))) int dyn[];
  __shared__ int done[W];  // steps a wavefront has published
  const int live_block = kLive ? (int)(blockIdx.x >> 3) % live_n : 0;
  const int b = kLive ? (int)(blockIdx.x / (8 * live_n)) * 8 + (blockIdx.x & 7) : blockIdx.x;
  const int lane = threadIdx.x & 63, tidx = threadIdx.x;
  const int wave = W > 1 ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : 0;
  if (kLive) {
    if (b >= d.B) return;
    u_base = live_block * 64 * C * W;
  }
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  if (Tb == 0 || Ub == 0) return;  // :152-154
  // A label axis longer than 64 C W positions is walked block by block, lowest first, as in
  // alpha_kernel (u_base, ghin, ghout); the decision columns then live in global memory and the
  // launch of the highest block (traces != 0) follows the path back through all of them.
  const bool walks = u_base < Ub;
  if (!walks && !traces) return;
  const int nsteps = Tb + Ub - 1;
  const int ngroups = (nsteps + 3) >> 2;
  int* taken = dyn;                             // [U rounded up to 4] (not in a live launch)
  float* hand = reinterpret_cast<float*>(dyn + (kLive ? 0 : (d.U + 3) & ~3));  // [W-1][hand_stride]
  unsigned* cols = kLdsBits
      ? reinterpret_cast<unsigned*>(hand + (W - 1) * hand_stride)     // [64 C W][nw]
      : gcols + (size_t)b * d.Ua * nw;                                // [Ua][nw]
  const float* gin = (kMulti && !kLive && ghin) ? ghin + (size_t)b * hand_stride : nullptr;
  float* gout = (kMulti && !kLive && ghout && walks) ? ghout + (size_t)b * hand_stride : nullptr;
  if (kMulti && gout && tidx == 0) gout[0] = kNegInf;  // nothing enters step 0
  // live blocks: block h reads the entries of boundary h - 1 and writes those of boundary h
  const bool live_in = kLive && live_block > 0, live_out = kLive && live_block < live_n - 1;
  const unsigned long long* lrow =
      kLive ? live + ((size_t)max(live_block - 1, 0) * d.B + b) * hand_stride : nullptr;
  unsigned long long* lrow_out =
      kLive ? live + ((size_t)min(live_block, max(live_n - 2, 0)) * d.B + b) * hand_stride
            : nullptr;
  auto live_entry = [](int s, float x) -> unsigned long long {
    return ((unsigned long long)(unsigned)(s + 1) << 32) | (unsigned long long)__float_as_uint(x);
  };
  auto live_load = [&](int s) -> unsigned long long {
    return __hip_atomic_load(lrow + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  // (one opaque statement: see alpha_kernel)
  auto live_reload = [&](int s) -> unsigned long long {
    unsigned long long e;
    const unsigned long long* q = lrow + s;
    asm volatile("global_load_dwordx2 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)"
                 : "=&v"(e)
                 : "v"(q)
                 : "memory");
    return e;
  };
  unsigned live_sink = 0;
  if (live_out && tidx == 0)  // nothing enters step 0
    __hip_atomic_store(lrow_out, live_entry(0, kNegInf), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  if (W > 1) {
    if (tidx < W) done[tidx] = 0;
    if (tidx < W - 1) hand[tidx * hand_stride] = kNegInf;  // nothing enters step 0
  }
  if (!kLive)
    for (int u = tidx; u < Ub; u += 64 * W) taken[u] = -1;
  __syncthreads();
  float* hand_out = hand + wave * hand_stride;                            // wave < W-1
  const float* hand_in = hand + (wave > 0 ? wave - 1 : 0) * hand_stride;  // wave > 0
  // (a launch that only traces asks for its first groups' operands like any other, and never
  // uses them: it asks where the lowest block would, inside the arrays)
  const int u0 = (walks ? u_base : 0) + (wave * 64 + lane) * C;
  // E[t,blank] for the cells of step s sits at ebl[s - u]; column c at step 4g+j reads
  // ebl[4g + j - c], so one run of C+3 values serves all columns of a group
  const float* ebl = p.eb + (size_t)b * d.Tp + d.Eo - u0;
  const int gstride = plane_group_stride(d);

  float stay[C], emit[C], pbv[C];
  unsigned wbits[C];
  const float* lnp[C];
  const float* bsp[C];
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int u = u0 + c, uc = u < d.U ? u : d.U - 1;
    const size_t row = plane_group0(d, b, uc);
    lnp[c] = p.lnS + row;
    bsp[c] = bestS + row;
    pbv[c] = p.pb[(size_t)b * d.Ua + uc];
    stay[c] = kNegInf;
    emit[c] = kNegInf;
    wbits[c] = 0u;
  }
  struct Group {
    float4 ln[C], bs[C];
    float eb[C + 3];
    float4 gh;  // scores entering the block's first column from the block below
    unsigned long long lv;  // the same, tagged, from the block running beside this one: lane j
                            // holds entry 4g + j
  };
  auto load_group = [&](int g) -> Group {
    Group r;
#pragma unroll
    for (int c = 0; c < C; ++c) {
      r.ln[c] = *reinterpret_cast<const float4*>(lnp[c] + (size_t)g * gstride);
      r.bs[c] = *reinterpret_cast<const float4*>(bsp[c] + (size_t)g * gstride);
    }
#pragma unroll
    for (int k = 0; k < C + 3; ++k) r.eb[k] = ebl[4 * g + k - (C - 1)];
    if constexpr (kMulti) {
      r.gh = make_float4(kNegInf, kNegInf, kNegInf, kNegInf);
      if (gin) r.gh = *reinterpret_cast<const float4*>(gin + 4 * g);  // uniform
      if constexpr (kLive) r.lv = live_load(4 * g + (lane & 3));  // every wavefront asks
    }
    return r;
  };
  int avail = 0;  // steps the wavefront below is known to have published (see alpha_kernel)
  auto wait_for = [&](int need) {
    avail = bounded_wait(&done[wave - 1], avail, need, spin_limit, trouble);
  };
  // A cell that has not started (t < 0) keeps -inf scores and never takes a label; cells past
  // the utterance run on whatever the planes hold and are never consulted by the backtrace.
  auto run_group = [&](int g, const Group& cur) {
    float4 hin = {kNegInf, kNegInf, kNegInf, kNegInf};
    if constexpr (kMulti) hin = cur.gh;  // wavefront 0: from the block below (or nothing)
    if constexpr (kLive) {
      if (live_in && wave == 0) {  // uniform; as in alpha_kernel
        unsigned long long e = cur.lv;
        if (__builtin_amdgcn_ballot_w64(lane < 4 &&
                                        (unsigned)(e >> 32) != (unsigned)(4 * g + lane + 1))) {
          const int mine = lane < 4 ? 4 * g + lane : min(4 * ngroups, 4 * (g + kLiveLag));
          int spins = 0;
          do {
            if (spins++ >= spin_limit) {
              if (lane == 0) raise_trouble(trouble);
              break;
            }
            __builtin_amdgcn_s_sleep(4);
            e = live_reload(mine);
          } while (__builtin_amdgcn_ballot_w64((unsigned)(e >> 32) != (unsigned)(mine + 1)));
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
          f4set(hin, j, __int_as_float(__builtin_amdgcn_readlane((int)(unsigned)e, j)));
      } else {
        live_sink ^= (unsigned)cur.lv;
      }
    }
    if (W > 1 && wave > 0) {
      wait_for(4 * g + 3);
      hin = *reinterpret_cast<const float4*>(hand_in + 4 * g);
    }
    float hout[4];
    float gsend[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = 4 * g + j;
      const unsigned sbit = 1u << (s & 31);  // uniform
      float from_left = wave_shr1(emit[C - 1], kNegInf);
      if (W > 1 || kMulti) from_left = (lane == 0) ? f4get(hin, j) : from_left;
#pragma unroll
      for (int c = C - 1; c >= 0; --c) {
        const float left = (c == 0) ? from_left : emit[c - 1];
        const bool take = left > stay[c];  // :200-206 ties go to blank
        float x = take ? left : stay[c];
        if (j == 0 && g == 0) x = (u0 + c == 0) ? 0.0f : x;
        wbits[c] |= take ? sbit : 0u;
        const float ln = f4get(cur.ln[c], j);
        float sb = x + cur.eb[j - c + (C - 1)];
        sb = sb + pbv[c];
        sb = sb - ln;
        float se = x + f4get(cur.bs[c], j);
        se = se - ln;
        const bool started = s >= u0 + c;
        stay[c] = started ? sb : kNegInf;
        emit[c] = started ? se : kNegInf;
      }
      if constexpr (kMulti) gsend[j] = emit[C - 1];
      if (W > 1)
        hout[j] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(emit[C - 1]), 63));
    }
    if constexpr (kMulti) {
      if (gout && wave == W - 1 && lane == 63) {  // entries 4g+1 .. 4g+4 for the block above
#pragma unroll
        for (int j = 0; j < 4; ++j) gout[4 * g + 1 + j] = gsend[j];
      }
      if constexpr (kLive) {
        if (live_out && wave == W - 1 && lane == 63) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            __hip_atomic_store(lrow_out + 4 * g + 1 + j, live_entry(4 * g + 1 + j, gsend[j]),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    if ((g & 7) == 7 || g == ngroups - 1) {  // uniform: a word of 32 steps is complete
#pragma unroll
      for (int c = 0; c < C; ++c) {
        cols[(size_t)(u0 + c) * nw + (g >> 3)] = wbits[c];
        wbits[c] = 0u;
      }
    }
    if (W > 1 && wave < W - 1 && lane == 0) {  // entries 4g+1 .. 4g+4, then the progress
#pragma unroll
      for (int j = 0; j < 4; ++j) hand_out[4 * g + 1 + j] = hout[j];
      asm volatile("" ::: "memory");
      __hip_atomic_store(&done[wave], 4 * g + 4, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  };
  // four register sets rotate (no copies): a group's loads are requested four groups ahead
  auto clamp_g = [&](int g) { return g < ngroups ? g : ngroups - 1; };
  if constexpr (kLive) {
    if (live_in && wave == 0) {  // start kLiveLag groups behind the block below (or when it is done)
      const int far = min(4 * ngroups, 4 * kLiveLag);
      int spins = 0;
      while ((unsigned)(live_load(far) >> 32) != (unsigned)(far + 1)) {
        if (spins++ >= spin_limit) {
          if (lane == 0) raise_trouble(trouble);
          break;
        }
        __builtin_amdgcn_s_sleep(8);
      }
    }
  }
  Group q0 = load_group(0), q1 = load_group(clamp_g(1)), q2 = load_group(clamp_g(2)),
        q3 = load_group(clamp_g(3));
  const int nwalk = walks ? ngroups : 0;  // a block past the utterance's labels only traces
  if (W > 1 && wave > 0 && walks)
    wait_for(min(4 * ngroups, 4 * (kLive ? kLiveWaveLag : 8) * wave));  // fall a few groups behind
  for (int g = 0; g < nwalk; g += 4) {
    run_group(g, q0);
    q0 = load_group(clamp_g(g + 4));
    if (g + 1 < ngroups) run_group(g + 1, q1);
    q1 = load_group(clamp_g(g + 5));
    if (g + 2 < ngroups) run_group(g + 2, q2);
    q2 = load_group(clamp_g(g + 6));
    if (g + 3 < ngroups) run_group(g + 3, q3);
    q3 = load_group(clamp_g(g + 7));
  }
  if constexpr (kLive) {
    if (spin_limit < 0 && live_sink == 1u) raise_trouble(trouble);  // never
  }
  if (!kLdsBits) __threadfence();  // the columns in global memory, before another lane reads them
  __syncthreads();
  if (!traces) return;
  // Backtrace (:208-219): from (T_b - 1, U_b - 1); a set bit at (step, u) means "entered from
  // u - 1 with a label", a clear one "entered from t - 1 with a blank".
  if (tidx == 0) {
    int u = Ub - 1, s = nsteps - 1;
    while (u > 0) {
      int wi = s >> 5;
      unsigned m = cols[(size_t)u * nw + wi] & (0xFFFFFFFFu >> (31 - (s & 31)));
      while (m == 0u && wi > 0) {
        --wi;
        m = cols[(size_t)u * nw + wi];
      }
      if (m == 0u) break;  // ran out of frames: cannot happen on a lattice that was walked
      const int st = 32 * wi + 31 - __clz(m);
      taken[u - 1] = st;
      u -= 1;
      s = st - 1;
    }
  }
  __syncthreads();
  int* out = labels_out + (size_t)b * (d.U - 1);
  const int* argI = reinterpret_cast<const int*>(argS);
  for (int u1 = tidx; u1 < Ub - 1; u1 += 64 * W) {
    const int st = taken[u1];
    // (a label is never taken at step 0 on a lattice that was walked; the clamp keeps the read
    // inside the plane whatever the decision bits hold)
    if (st >= 0) out[u1] = argI[plane_at(d, b, u1, max(st - 1, 0))];
  }
}

// ------------------------------------------------------------------ chain-latency floor
// What ONE step of a lattice walk costs when nothing but its dependent chain is left: operands
// in registers, no loads, no stores, no bookkeeping, one wavefront alone on its SIMD.
//   kind 0: a cell of alpha_kernel -- DPP hand-over, log-sum-exp on the hardware units with
//           the check that its sum is the C library's (lse2_checked; the operands are large, so
//           no lane falls back), then the three additions of a move;
//   kind 1: a cell of beta_kernel -- DPP hand-over, two multiplies and an add;
//   kind 2: kind 0 with every lane on the library path (rnnt_libm.h: ~100 instructions, two of
//           them divisions): what a step costs while any lane of the wavefront falls back.
// The walks cannot run faster than steps x this; the ratio is what the prefetch, the stores and
// the second wavefront's hand-over cost on top.
template <int kKind>
__global__ __launch_bounds__(64) void chain_floor_kernel(float* __restrict__ sink, int steps,
                                                         float e, float p, float ln, float w) {
  __shared__ unsigned long long etab[32];
  exp2_table_to_lds(etab);
  __syncthreads();
  const int lane = threadIdx.x;
  float stay = -5000.0f - 0.37f * lane, emit = -5000.0f - 0.61f * lane, dcol = 1.0f / (1 + lane);
#pragma unroll 4
  for (int s = 0; s < steps; ++s) {
    if (kKind != 1) {
      const float left = wave_shr1(emit, kOutside);
      const float a = kKind == 0 ? lse2_checked(left, stay, etab) : lse2_libm(left, stay, etab);
      float sb = a + e;
      sb = sb + p;
      sb = sb - ln;
      float se = a + p;
      se = se + e;
      se = se - ln;
      stay = sb;
      emit = se;
    } else {
      const float right = wave_shl1(dcol, 0.0f);
      const float ne = dcol * w;
      const float em = right * w;
      dcol = ne + em;
    }
  }
  sink[lane] = kKind != 1 ? stay + emit : dcol;
}

}  // namespace

namespace {
// The two library functions applied elementwise, for the tests that hold them to the host's C
// library bit for bit.
__global__ __launch_bounds__(256) void libm_probe_kernel(const float* __restrict__ x,
                                                         float* __restrict__ e,
                                                         float* __restrict__ l, long n) {
  __shared__ unsigned long long etab[32];
  exp2_table_to_lds(etab);
  __syncthreads();
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  e[i] = expf_glibc(x[i], etab);
  l[i] = log1pf_glibc(x[i]);
}
}  // namespace

namespace {
// For every float d with bit pattern in [lo, hi] (d <= 0): does the bound of lse2_checked cover
// the distance between the fast and the library value of log1p(exp(d))?  out[0] counts the
// patterns where it does not, out[1] keeps the largest ratio distance / bound (as float bits;
// ratios are non-negative, so their bit patterns order like integers).
__global__ __launch_bounds__(256) void lse_bound_kernel(unsigned lo, unsigned hi,
                                                        unsigned* __restrict__ out) {
  __shared__ unsigned long long etab[32];
  exp2_table_to_lds(etab);
  __syncthreads();
  unsigned bad = 0;
  float worst = 0.0f;
  const unsigned long long n = (unsigned long long)hi - lo + 1;
  for (unsigned long long i = (unsigned long long)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (unsigned long long)gridDim.x * 256) {
    const float d = __uint_as_float(lo + (unsigned)i);
    const float exact = log1pf_glibc(expf_glibc_nonpositive(d, etab));
    const float lf = softplus_fast(d);
    const float bound = fast_bound(lf, d);
    const float dist = fabsf(lf - exact);
    if (!(dist <= bound)) {
      ++bad;
    } else if (bound > 0.0f) {
      worst = fmaxf(worst, dist / bound);
    }
  }
  if (bad) atomicAdd(&out[0], bad);
  atomicMax(&out[1], __float_as_uint(worst));
}
}  // namespace

int launch_lse_bound_check(unsigned lo, unsigned hi, unsigned* out, hipStream_t s) {
  hipLaunchKernelGGL(lse_bound_kernel, dim3(4096), dim3(256), 0, s, lo, hi, out);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return check_hip(err, "launch lse_bound_kernel", __FILE__, __LINE__);
  return kOk;
}

int launch_libm_probe(const float* x, float* e, float* l, long n, hipStream_t s) {
  if (n == 0) return kOk;
  const long blocks = (n + 255) / 256;
  if (blocks > 0x7fffffffl) return fail(kInvalid, "libm_probe: too many elements");
  hipLaunchKernelGGL(libm_probe_kernel, dim3((unsigned)blocks), dim3(256), 0, s, x, e, l, n);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return check_hip(err, "launch libm_probe_kernel", __FILE__, __LINE__);
  return kOk;
}

int launch_chain_floor(int kind, int steps, hipStream_t s) {
  int* words = nullptr;
  RNNT_TRY(trouble_flag(&words));
  float* sink = reinterpret_cast<float*>(words + 64);
  // scores that keep the recursion near zero: a step adds log 2 and takes it off again
  if (kind == 0)
    hipLaunchKernelGGL(chain_floor_kernel<0>, dim3(1), dim3(64), 0, s, sink, steps, 0.3f, 0.2f,
                       0.5f + 0.693147f, 0.5f);
  else if (kind == 2)
    hipLaunchKernelGGL(chain_floor_kernel<2>, dim3(1), dim3(64), 0, s, sink, steps, 0.3f, 0.2f,
                       0.5f + 0.693147f, 0.5f);
  else
    hipLaunchKernelGGL(chain_floor_kernel<1>, dim3(1), dim3(64), 0, s, sink, steps, 0.3f, 0.2f,
                       0.5f, 0.5f);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return check_hip(e, "launch chain_floor_kernel", __FILE__, __LINE__);
  return kOk;
}

// ------------------------------------------------------------------ trouble flag
// One int per device, raised by a lattice kernel whose bounded wait ran out (bounded_wait).  The
// array's name is a host-side handle, not a device address: the address is looked up once per
// device, with that device current, and kernels are given that pointer.
static __device__ int g_trouble_word[128];  // [0]: the flag; [64..127]: sink of the floor probe
constexpr int kMaxDevices = 64;
static int* g_trouble_ptr[kMaxDevices];
static std::mutex g_trouble_mutex;
int g_spin_limit = kDefaultSpinLimit;

int trouble_flag(int** out) {
  int dev = 0;
  RNNT_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(kInvalid, "device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_trouble_mutex);
  if (g_trouble_ptr[dev] == nullptr) {
    void* p = nullptr;
    RNNT_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_trouble_word)));
    g_trouble_ptr[dev] = static_cast<int*>(p);
  }
  *out = g_trouble_ptr[dev];
  return kOk;
}

// ------------------------------------------------------------------ workspace layout
static size_t align_up(size_t x) { return (x + 255) & ~(size_t)255; }

// Blocks of label positions that the alpha and dalpha walks run side by side, one workgroup of
// `waves` wavefronts (one position a lane) each: four wavefronts, 256 positions, while their
// three hand-over arrays fit LDS (up to about 12000 anti-diagonals); two wavefronts, 128
// positions, with their one array up to about 36000.  0 blocks where one workgroup takes the
// label axis as well or better: up to 256 positions on four wavefronts, up to 128 on two; and,
// up to 1024 positions, where the batch would need more workgroups than the device has CUs to
// spare (with that many utterances the planes' traffic holds the walks either way).  Past 1024
// positions the blocks go side by side whatever the batch: workgroups are dispatched in order,
// a block after the block it follows, so more workgroups than CUs only queue -- and the other
// way there, a launch per 1024 positions with sixteen positions a lane, is many times slower.
int live_blocks(const Dims& d, int* waves) {
  const size_t one = sizeof(float) * (size_t)d.Dp;
  const int W = 3 * one <= 144 * 1024 ? 4 : one <= 144 * 1024 ? 2 : 0;
  if (waves) *waves = W;
  if (W == 0) return 0;
  const int n = (d.U + 64 * W - 1) / (64 * W);
  if (n < 2 || n > 16) return 0;
  if (d.B * n > 192 && d.U <= 1024) return 0;
  return n;
}
// The two hand-over vectors of the planes hold the walks' tagged 64-bit entries as well: one
// array of [B][Dp] entries per boundary between live blocks.  In units of [B][Dp] floats each.
static int hand_arrays(const Dims& d) {
  const int n = live_blocks(d, nullptr);
  return n > 2 ? n - 1 : 1;
}

size_t planes_bytes(const Dims& d, bool decode_only) {
  const size_t plane = align_up(sizeof(float) * (size_t)d.B * d.Ua * d.Dp + 64);
  return (decode_only ? 1 : 6) * plane + align_up(sizeof(float) * (size_t)d.B * d.Tp) +
         4 * align_up(sizeof(float) * (size_t)d.B * d.Ua) +
         2 * align_up(sizeof(float) * (size_t)d.B * d.Dp * hand_arrays(d));
}

void carve_planes(void* base, const Dims& d, Planes* p, bool decode_only) {
  char* c = static_cast<char*>(base);
  const size_t plane = align_up(sizeof(float) * (size_t)d.B * d.Ua * d.Dp + 64);
  auto take = [&](size_t n) { float* r = reinterpret_cast<float*>(c); c += n; return r; };
  p->lnS = take(plane);
  p->elS = p->aS = p->wB = p->wE = p->dS = nullptr;
  if (!decode_only) {
    p->elS = take(plane); p->aS = take(plane);
    p->wB = take(plane); p->wE = take(plane); p->dS = take(plane);
  }
  p->eb = take(align_up(sizeof(float) * (size_t)d.B * d.Tp));
  const size_t bu = align_up(sizeof(float) * (size_t)d.B * d.Ua);
  p->pb = take(bu); p->pl = take(bu); p->gB = take(bu); p->gL = take(bu);
  const size_t bh = align_up(sizeof(float) * (size_t)d.B * d.Dp * hand_arrays(d));
  p->hand[0] = take(bh); p->hand[1] = take(bh);
}

// ------------------------------------------------------------------ launchers
// tiles of 64 anti-diagonals x 64 label positions over all anti-diagonals t + u < T + U
static dim3 tile_grid(const Dims& d) {
  return dim3((d.T + d.U + 62) / 64, (d.U + 63) / 64, d.B);
}

int launch_skew(const float* src, float* dstS, const int* inLen, const int* labLen, const Dims& d,
                hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  hipLaunchKernelGGL(skew_kernel, tile_grid(d), dim3(256), 0, s, src, dstS, inLen, labLen, d);
  RNNT_LAUNCH_CHECK("skew_kernel");
  return kOk;
}

int launch_unskew(const float* srcS, float* dst, const int* inLen, const int* labLen,
                  const Dims& d, hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  hipLaunchKernelGGL(unskew_kernel, tile_grid(d), dim3(256), 0, s, srcS, dst, inLen, labLen, d);
  RNNT_LAUNCH_CHECK("unskew_kernel");
  return kOk;
}

template <typename TIO>
static int gather_any(const TIO* E, const TIO* P, const int* labels, const int* inLen,
                      const int* labLen, const Planes& p, const Dims& d, hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  if (d.V <= 1024)
    hipLaunchKernelGGL(gather_kernel<TIO>, tile_grid(d), dim3(256), 0, s, E, P, labels, inLen,
                       labLen, p, d);
  else
    hipLaunchKernelGGL(gather_cells_kernel<TIO>, dim3((d.T + 255) / 256, d.U, d.B), dim3(256), 0,
                       s, E, P, labels, inLen, labLen, p, d);
  RNNT_LAUNCH_CHECK("gather_kernel");
  return kOk;
}
int launch_gather(const float* E, const float* P, const int* labels, const int* inLen,
                  const int* labLen, const Planes& p, const Dims& d, hipStream_t s) {
  return gather_any(E, P, labels, inLen, labLen, p, d, s);
}
int launch_gather(const bf16_t* E, const bf16_t* P, const int* labels, const int* inLen,
                  const int* labLen, const Planes& p, const Dims& d, hipStream_t s) {
  return gather_any(E, P, labels, inLen, labLen, p, d, s);
}
int launch_gather(const f16_t* E, const f16_t* P, const int* labels, const int* inLen,
                  const int* labLen, const Planes& p, const Dims& d, hipStream_t s) {
  return gather_any(E, P, labels, inLen, labLen, p, d, s);
}

// Label positions one launch of a lattice walk covers: the whole axis up to 1024, else blocks of
// 1024 (64 lanes x 16 positions), one launch per block.
static int block_cells_per_lane(const Dims& d) { return min(cells_per_lane(d.U), 16); }
static int label_blocks(const Dims& d) {
  const int width = 64 * block_cells_per_lane(d);
  return (d.U + width - 1) / width;
}

__global__ void clear_words_kernel(int* x, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[i] = 0;
}

// Launches the side-by-side form of a walk (K: its kernel, W wavefronts of one position a lane)
// for n blocks: clears the tagged entries, then one workgroup per utterance and block, eight
// utterances' blocks in consecutive indices.
template <typename K, typename... Args>
static int launch_live(K kernel, const Planes& p, const Dims& d, int n, int W,
                       hipStream_t s, Args... args) {
  unsigned long long* live = reinterpret_cast<unsigned long long*>(p.hand[0]);
  const size_t lds = sizeof(float) * (size_t)(W - 1) * d.Dp;
  const int words = 2 * d.B * d.Dp * (n - 1);
  hipLaunchKernelGGL(clear_words_kernel, dim3((words + 255) / 256), dim3(256), 0, s,
                     reinterpret_cast<int*>(live), words);
  RNNT_LAUNCH_CHECK("clear_words_kernel");
  if (lds > 64 * 1024)
    RNNT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(kernel, dim3(8 * n * ((d.B + 7) / 8)), dim3(64 * W), lds, s, args..., live,
                     n);
  RNNT_LAUNCH_CHECK("lattice walk (blocks side by side)");
  return kOk;
}

int launch_alpha(const Planes& p, const int* inLen, const int* labLen, float* costs,
                 const Dims& d, hipStream_t s) {
  if (d.B == 0) return kOk;
  // cells per lane of a single wavefront; split over two wavefronts when the hand-over
  // array (one float per step and boundary) fits LDS
  const int cpl = block_cells_per_lane(d), nblocks = label_blocks(d);
  const int stride = d.Dp;
  // (two wavefronts up to 128 label positions, four beyond -- one, two or four positions a lane
  // -- if their three hand-over arrays fit LDS: a step costs a wavefront one log-sum-exp per
  // position it owns, and the step is what a lattice is bound by.  B=8 T=2000, 129..256 label
  // positions: 262 ns a step with two wavefronts of two positions, 160 with four of one, what
  // 101 positions on two wavefronts take)
  const bool single_block = nblocks == 1;
  const int W = (single_block && cpl >= 4 && 3 * stride * sizeof(float) <= 144 * 1024) ? 4
                : (cpl >= 2 && stride * sizeof(float) <= 144 * 1024) ? 2 : 1;
  const size_t lds = W > 1 ? sizeof(float) * (size_t)(W - 1) * stride : 0;
  int* trouble = nullptr;
  RNNT_TRY(trouble_flag(&trouble));
  // From 257 label positions, with few enough utterances that the device has the CUs: blocks
  // of 256 positions side by side on as many CUs, four wavefronts of one position a lane each
  // (B=8 T=10000, 401 positions: 176 ns a step against 235 on one CU; B=8 T=2000, 513 .. 1024
  // positions: 523 .. 539 ns on one CU with two to four positions a lane; from about a hundred
  // utterances on the planes' traffic holds every form, B=128 T=2000: 241 ns)
  int live_w = 0;
  if (const int n = live_blocks(d, &live_w)) {
    if (live_w == 4)
      return launch_live(alpha_kernel<1, 4, true, true>, p, d, n, 4, s, p, inLen, labLen, costs,
                         d, stride, g_spin_limit, trouble, 0, (const float*)nullptr,
                         (float*)nullptr);
    return launch_live(alpha_kernel<1, 2, true, true>, p, d, n, 2, s, p, inLen, labLen, costs, d,
                       stride, g_spin_limit, trouble, 0, (const float*)nullptr, (float*)nullptr);
  }
  for (int k = 0; k < nblocks; ++k) {  // lowest block first
    const float* ghin = k == 0 ? nullptr : p.hand[(k - 1) & 1];
    float* ghout = k == nblocks - 1 ? nullptr : p.hand[k & 1];
    const int u_base = k * 64 * cpl;
    switch ((nblocks > 1 ? 10000 : 0) + cpl / W * 100 + W) {
#define CASE(C, W, M)                                                                        \
  case (M ? 10000 : 0) + C * 100 + W:                                                        \
    if (lds > 64 * 1024)                                                                     \
      RNNT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(alpha_kernel<C, W, M>),     \
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));   \
    hipLaunchKernelGGL((alpha_kernel<C, W, M>), dim3(d.B), dim3(64 * W), lds, s, p, inLen,  \
                       labLen, costs, d, stride, g_spin_limit, trouble, u_base, ghin,        \
                       ghout, nullptr, 0);                                                   \
    break;
      CASE(1, 1, false) CASE(2, 1, false) CASE(4, 1, false) CASE(8, 1, false) CASE(16, 1, false)
      CASE(1, 2, false) CASE(2, 2, false) CASE(4, 2, false) CASE(8, 2, false)
      CASE(1, 4, false) CASE(2, 4, false) CASE(4, 4, false)
      CASE(16, 1, true) CASE(8, 2, true)  // several blocks: always 1024 positions each
#undef CASE
      default:
        return fail(kInvalid, "alpha: no kernel for %d label positions per lane", cpl);
    }
    RNNT_LAUNCH_CHECK("alpha_kernel");
  }
  return kOk;
}

int launch_weights(const Planes& p, const int* inLen, const int* labLen, const Dims& d,
                   hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  hipLaunchKernelGGL(weights_kernel, dim3((d.Ua * d.Dp + 255) / 256, 1, d.B), dim3(256), 0, s, p,
                     inLen, labLen, d);
  RNNT_LAUNCH_CHECK("weights_kernel");
  return kOk;
}

int launch_beta(const Planes& p, const int* labels, const int* inLen, const int* labLen,
                const Dims& d, hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  const int cpl = block_cells_per_lane(d), nblocks = label_blocks(d);
  // wavefronts: one up to 128 label positions (a step of this walk is a handful of
  // instructions a position, and the hand-over would cost as much again), four beyond (two if
  // only their hand-over array fits LDS); one per block when the axis takes several launches.
  // (129..256 label positions, B=8 T=2000: 70 ns a step with two wavefronts of two positions, 57
  // with four of one)
  const int stride = d.Dp;
  const bool single_block = nblocks == 1;
  const int W = !single_block ? 1
                : (cpl >= 4 && 3 * stride * sizeof(float) <= 144 * 1024) ? 4
                : (cpl >= 4 && stride * sizeof(float) <= 144 * 1024) ? 2 : 1;
  const size_t lds = W > 1 ? sizeof(float) * (size_t)(W - 1) * stride : 0;
  int* trouble = nullptr;
  RNNT_TRY(trouble_flag(&trouble));
  // from 257 label positions in few enough utterances: blocks of 256 positions side by side
  // (as in launch_alpha)
  int live_w = 0;
  if (const int n = live_blocks(d, &live_w)) {
    if (live_w == 4)
      return launch_live(beta_kernel<1, 4, false, true>, p, d, n, 4, s, p, labels, inLen, labLen,
                         d, stride, 0, (const float*)nullptr, (float*)nullptr, g_spin_limit,
                         trouble);
    return launch_live(beta_kernel<1, 2, false, true>, p, d, n, 2, s, p, labels, inLen, labLen, d,
                       stride, 0, (const float*)nullptr, (float*)nullptr, g_spin_limit, trouble);
  }
  for (int k = nblocks - 1; k >= 0; --k) {  // highest block first
    const float* ghin = k == nblocks - 1 ? nullptr : p.hand[(k + 1) & 1];
    float* ghout = k == 0 ? nullptr : p.hand[k & 1];
    const int u_base = k * 64 * cpl;
    switch ((nblocks > 1 ? 10000 : 0) + cpl / W * 100 + W) {
#define CASE(C, W, M)                                                                       \
  case (M ? 10000 : 0) + C * 100 + W:                                                       \
    if (lds > 64 * 1024)                                                                    \
      RNNT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(beta_kernel<C, W, M>),     \
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));  \
    hipLaunchKernelGGL((beta_kernel<C, W, M>), dim3(d.B), dim3(64 * W), lds, s, p, labels, \
                       inLen, labLen, d, stride, u_base, ghin, ghout, g_spin_limit,        \
                       trouble, nullptr, 0);                                                \
    break;
      CASE(1, 1, false) CASE(2, 1, false) CASE(4, 1, false) CASE(8, 1, false) CASE(16, 1, false)
      CASE(2, 2, false) CASE(4, 2, false) CASE(8, 2, false)
      CASE(1, 4, false) CASE(2, 4, false) CASE(4, 4, false)
      CASE(16, 1, true)
#undef CASE
      default:
        return fail(kInvalid, "dalpha: no kernel for %d label positions per lane", cpl);
    }
    RNNT_LAUNCH_CHECK("beta_kernel");
  }
  return kOk;
}

int launch_sparse(const Planes& p, const float* bsum, const float* emT, float* egrads,
                  float* pgrads, const int* labels, const int* inLen, const int* labLen,
                  const float* scale, bool add, const Dims& d, hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  if (!bsum || !emT) return fail(kInvalid, "sparse terms: the per-frame terms were not formed");
  const size_t rows_bytes = sizeof(float) * 64 * (size_t)(d.V | 1);
  // (a small vocabulary also when the terms are to be stored: the arrays are zero-filled then,
  // and adding to zeros leaves the same bits -- B=8 T=10000 U=400 V=32: 1.67 ms with one
  // hardware add per term, all of them into 128 bytes a frame)
  if (rows_bytes <= 64 * 1024 && labels != nullptr) {
    hipLaunchKernelGGL(sparse_e_rows_kernel, dim3((d.T + 63) / 64, d.B), dim3(64), rows_bytes, s,
                       bsum, emT, egrads, labels, inLen, labLen, add ? scale : nullptr, d);
    RNNT_LAUNCH_CHECK("sparse_e_rows_kernel");
  } else {
    hipLaunchKernelGGL(sparse_e_kernel, dim3((d.T + 255) / 256, d.B), dim3(256), 0, s, bsum, emT,
                       egrads, labels, inLen, labLen, scale, add ? 1 : 0, d);
    RNNT_LAUNCH_CHECK("sparse_e_kernel");
  }
  if (pgrads == nullptr) return kOk;  // the caller adds those terms itself
  hipLaunchKernelGGL(sparse_p_kernel, dim3((d.U + 255) / 256, d.B), dim3(256), 0, s, p, pgrads,
                     labels, inLen, labLen, scale, add ? 1 : 0, d);
  RNNT_LAUNCH_CHECK("sparse_p_kernel");
  return kOk;
}

int launch_post_beta(const Planes& p, const float* mE, const float* mP, float* Wn, float* Wt,
                     float* bsum, float* emT, const int* labels, const int* inLen,
                     const int* labLen, const Dims& d, hipStream_t s, const WImages& img) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  const int Up = wplane_up(d.U), Tw = wplane_tw(d.T);
  if (img.e && Up > WImages::kCols)
    return fail(kInvalid, "W images hold at most %d label positions", WImages::kCols);
  // W tiles: 64 label positions x 64 anti-diagonals (all anti-diagonals below Tw + Up), or for
  // the images 64 label positions x 64 frames
  // (Wn == nullptr: no W at all, only the per-frame terms)
  const int wx = img.e ? Tw / 64 : (Tw + Up + 62) / 64, wy = (Up + 63) / 64;
  const int nw = (Wn || img.e) ? wx * wy * d.B : 0;
  if ((bsum == nullptr) != (emT == nullptr))
    return fail(kInvalid, "post_beta: the blank totals and the label-move terms come together");
  const int sx = (d.T + 4 * kBsFrames - 1) / (4 * kBsFrames), ns = bsum ? sx * d.B : 0;
  if (nw + ns == 0) return kOk;
  hipLaunchKernelGGL(post_beta_kernel, dim3(nw + ns), dim3(256), 0, s, p, mE, mP, Wn, Wt, bsum,
                     emT, labels, inLen, labLen, d, Up, Tw, wx, wy, nw, sx, img);
  RNNT_LAUNCH_CHECK("post_beta_kernel");
  return kOk;
}

// 0: lists where they can pay (maxplus_lists_pay) and a sample of the cells says they do; 1: every
// column for every cell; 2: lists wherever the shape allows (tests run small shapes through them)
static std::atomic<int> g_maxplus_mode{0};
void set_maxplus_mode(int mode) { g_maxplus_mode.store(mode); }
int maxplus_plan(const Dims& d) {
  const int mode = g_maxplus_mode.load();  // read once per call: the plan is what the call follows
  if (mode == 1 || !maxplus_lists_possible(d)) return 0;
  if (mode == 2) return 2;
  return maxplus_lists_pay(d) ? 1 : 0;
}

template <typename TIO>
static int maxplus_any(const TIO* E, const TIO* P, const int* inLen, const int* labLen,
                       float* best, int* arg, const Dims& d, hipStream_t s, void* lists,
                       bool force) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  static_assert(kMpT == 128 && kMpU == 64, "the list pass counts failures per tile of this kernel");
  const int *tile_fail = nullptr, *lists_on = nullptr;
  if (lists) {  // (the caller made the plan, and reserved `lists` if it says lists)
    RNNT_TRY(launch_maxplus_lists(E, P, inLen, labLen, best, arg, d, lists, force, s));
    maxplus_lists_counters(lists, d, &tile_fail, &lists_on);
  }
  const dim3 grid((d.T + kMpT - 1) / kMpT, (d.U + kMpU - 1) / kMpU, d.B);
  const bool vec = d.V % 4 == 0 &&
                   ((reinterpret_cast<uintptr_t>(E) | reinterpret_cast<uintptr_t>(P)) &
                    (4 * sizeof(TIO) - 1)) == 0;
  if (vec)
    hipLaunchKernelGGL((maxplus_kernel<true, TIO>), grid, dim3(kMpThreads), 0, s, E, P, inLen,
                       labLen, best, arg, d, tile_fail, lists_on, maxplus_tile_limit());
  else
    hipLaunchKernelGGL((maxplus_kernel<false, TIO>), grid, dim3(kMpThreads), 0, s, E, P, inLen,
                       labLen, best, arg, d, tile_fail, lists_on, maxplus_tile_limit());
  RNNT_LAUNCH_CHECK("maxplus_kernel");
  if (tile_fail) RNNT_TRY(launch_maxplus_cells(E, P, inLen, labLen, best, arg, d, lists, s));
  return kOk;
}
int launch_maxplus(const float* E, const float* P, const int* inLen, const int* labLen,
                   float* best, int* arg, const Dims& d, hipStream_t s, void* lists, bool force) {
  return maxplus_any(E, P, inLen, labLen, best, arg, d, s, lists, force);
}
int launch_maxplus(const bf16_t* E, const bf16_t* P, const int* inLen, const int* labLen,
                   float* best, int* arg, const Dims& d, hipStream_t s, void* lists, bool force) {
  return maxplus_any(E, P, inLen, labLen, best, arg, d, s, lists, force);
}
int launch_maxplus(const f16_t* E, const f16_t* P, const int* inLen, const int* labLen,
                   float* best, int* arg, const Dims& d, hipStream_t s, void* lists, bool force) {
  return maxplus_any(E, P, inLen, labLen, best, arg, d, s, lists, force);
}

// 32-step words per column of the decision table (one spare)
static int viterbi_words(const Dims& d) { return (d.T + d.U + 31) / 32 + 1; }

int launch_viterbi(const Planes& p, const float* bestS, const float* argS,
                   unsigned long long* gbits, const int* inLen, const int* labLen,
                   int* labels_out, const Dims& d, hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U <= 1) return kOk;
  unsigned* gcols = reinterpret_cast<unsigned*>(gbits);
  const int cpl = block_cells_per_lane(d), nblocks = label_blocks(d);
  const int stride = d.Dp;
  const int nw = viterbi_words(d);
  // (four wavefronts from 129 label positions while their hand-over arrays fit: B=8 T=2000,
  // 209 -> 167 ns a step at 257 positions, 446 -> 254 at 513, 551 -> 340 at 1000)
  // (B=8 T=10000 U=400, the reference's kernel benchmark: 3.5 ms with one wavefront of eight
  // positions a lane, which is what 64 KB of LDS allowed)
  const size_t taken_lds = sizeof(int) * (size_t)((d.U + 3) & ~3);
  const int W = (nblocks == 1 && cpl >= 4 &&
                 taken_lds + 3 * stride * sizeof(float) <= 144 * 1024) ? 4
                : (cpl >= 2 && taken_lds + stride * sizeof(float) <= 144 * 1024) ? 2 : 1;
  // dynamic LDS: one int per label position, the hand-over arrays between the wavefronts,
  // and the decision columns when they fit (one block only: with several, every block's columns
  // must be there for the backtrace of the last launch)
  const size_t base_lds = sizeof(int) * (size_t)((d.U + 3) & ~3) +
                          (W > 1 ? sizeof(float) * (size_t)(W - 1) * stride : 0);
  const size_t cols_lds = sizeof(unsigned) * (size_t)64 * cpl * nw;
  const bool use_lds = nblocks == 1 && base_lds + cols_lds <= 60 * 1024;
  const size_t lds = base_lds + (use_lds ? cols_lds : 0);
  if (lds > 150 * 1024)
    return fail(kInvalid, "viterbi: %d label positions and %d steps need %zu bytes of LDS", d.U,
                stride, lds);
  int* trouble = nullptr;
  RNNT_TRY(trouble_flag(&trouble));
  // Blocks of 256 label positions side by side where alpha_kernel takes them so (four wavefronts
  // whose hand-over arrays fit LDS), then one launch that only traces the path (B=8 T=10000
  // U=400: 1.65 ms for the walk on one CU, four wavefronts of two positions a lane).
  int live_w = 0;
  if (const int n = live_blocks(d, &live_w); n && live_w == 4) {
    RNNT_TRY(launch_live(viterbi_kernel<1, 4, false, true, true>, p, d, n, 4, s, p, bestS, argS,
                         inLen, labLen, gcols, labels_out, d, stride, nw, g_spin_limit, trouble, 0,
                         (const float*)nullptr, (float*)nullptr, 0));
    const size_t trace_lds = sizeof(int) * (size_t)((d.U + 3) & ~3);
    hipLaunchKernelGGL((viterbi_kernel<1, 1, false, true>), dim3(d.B), dim3(64), trace_lds, s, p,
                       bestS, argS, inLen, labLen, gcols, labels_out, d, stride, nw, g_spin_limit,
                       trouble, d.Ua, (const float*)nullptr, (float*)nullptr, 1,
                       (unsigned long long*)nullptr, 0);
    RNNT_LAUNCH_CHECK("viterbi_kernel (trace)");
    return kOk;
  }
  for (int k = 0; k < nblocks; ++k) {  // lowest block first; the last launch traces the path
    const float* ghin = k == 0 ? nullptr : p.hand[(k - 1) & 1];
    float* ghout = k == nblocks - 1 ? nullptr : p.hand[k & 1];
    const int u_base = k * 64 * cpl, traces = k == nblocks - 1 ? 1 : 0;
    switch ((nblocks > 1 ? 10000 : 0) + cpl / W * 100 + W) {
#define CASE(C, W)                                                                             \
  case C * 100 + W:                                                                            \
    if (use_lds)                                                                               \
      hipLaunchKernelGGL((viterbi_kernel<C, W, true, false>), dim3(d.B), dim3(64 * W), lds,   \
                         s, p, bestS, argS, inLen, labLen, gcols, labels_out, d, stride, nw,   \
                         g_spin_limit, trouble, u_base, ghin, ghout, traces, nullptr, 0);      \
    else {                                                                                     \
      if (lds > 64 * 1024)                                                                     \
        RNNT_HIP(hipFuncSetAttribute(                                                          \
            reinterpret_cast<const void*>(viterbi_kernel<C, W, false, false>),                 \
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                            \
      hipLaunchKernelGGL((viterbi_kernel<C, W, false, false>), dim3(d.B), dim3(64 * W), lds,  \
                         s, p, bestS, argS, inLen, labLen, gcols, labels_out, d, stride, nw,   \
                         g_spin_limit, trouble, u_base, ghin, ghout, traces, nullptr, 0);      \
    }                                                                                          \
    break;
#define CASE_MULTI(C, W)                                                                       \
  case 10000 + C * 100 + W:                                                                    \
    if (lds > 64 * 1024)                                                                       \
      RNNT_HIP(hipFuncSetAttribute(                                                            \
          reinterpret_cast<const void*>(viterbi_kernel<C, W, false, true>),                    \
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                              \
    hipLaunchKernelGGL((viterbi_kernel<C, W, false, true>), dim3(d.B), dim3(64 * W), lds, s,  \
                       p, bestS, argS, inLen, labLen, gcols, labels_out, d, stride, nw,        \
                       g_spin_limit, trouble, u_base, ghin, ghout, traces, nullptr, 0);        \
    break;
      CASE(1, 1) CASE(2, 1) CASE(4, 1) CASE(8, 1) CASE(16, 1)
      CASE(1, 2) CASE(2, 2) CASE(4, 2) CASE(8, 2)
      CASE(1, 4) CASE(2, 4) CASE(4, 4)
      CASE_MULTI(16, 1) CASE_MULTI(8, 2)  // several blocks: always 1024 positions each
#undef CASE
#undef CASE_MULTI
      default:
        return fail(kInvalid, "viterbi: no kernel for %d label positions per lane", cpl);
    }
    RNNT_LAUNCH_CHECK("viterbi_kernel");
  }
  return kOk;
}

size_t viterbi_bits_bytes(const Dims& d) {
  return sizeof(unsigned) * (size_t)d.B * 64 * cells_per_lane(d.U) * viterbi_words(d);
}

}  // namespace rnnt
